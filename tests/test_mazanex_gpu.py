"""Mazanex on the GPU against the plain implementation (tests/plain_mazanex.py), in float32 and
in bfloat16: traces that cut the same requests in different ways; long prompts whose weights are
made so that far tokens matter (decays near one, sharp attention); the edges of chunks and pages
in prompts and in decoding; captured steps against eager ones; generation through the Python
entry point, the scheduler and the command line."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import pytest
import torch
from safetensors.torch import load_file, save_file

import mazanex_util as mu
import plain_mazanex as plain
import replay_util as ru
from conftest import ROOT

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# head sizes of 64 and 128 beside small ones, a group of four, a chunk that is no multiple of the page
WIDE = mu.config(300, 128, [
    mu.layer("gla", {"heads": 2, "dim": 64, "vdim": 64, "tau": 12.0, "rank": 8}, 192),
    mu.layer("parallel", {"left": mu.attention(4, 1, 64, 32, 4, 48, 32, scale=0.11), "right": {"heads": 2, "dim": 64, "rank": 8}}, 160),
    mu.layer("mlstm", {"heads": 2, "dim": 32, "vdim": 128, "gate_cap": 10.0}, None),
])
# keys and values of 128 in groups of two (in bfloat16 the matrix-core attention kernels serve it, chunks and sink
# included), key sizes of 128 and 136 in the recurrences (a wave per column of the state), a one-tap neighbour
MATRIX = mu.config(210, 160, [
    mu.layer("parallel", {"left": mu.attention(4, 2, 128, 128, 2, 40, 64, scale=0.09), "right": {"heads": 2, "dim": 128, "rank": 6}}, 200),
    mu.layer("mlstm", {"heads": 2, "dim": 136, "vdim": 24, "gate_cap": 9.0}, 120),
    mu.layer("gla", {"heads": 1, "dim": 128, "vdim": 72, "tau": 20.0, "rank": 4}, None),
    mu.layer("parallel", {"left": mu.attention(2, 2, 64, 64, 1, 33, 16, scale=0.12), "right": {"heads": 5, "dim": 16, "rank": 2}}, 96),
])
CONFIGS = {"A": mu.MIXED_A, "B": mu.MIXED_B, "W": WIDE, "M": MATRIX}
LENGTHS = {"A": (5, 1, 14, 27, 90), "B": (2, 9, 21, 33, 64), "W": (3, 50, 130, 97, 200), "M": (4, 45, 150, 83, 1)}
BLOCKS = {"A": 4, "B": 8, "W": 16, "M": 16}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: mu.write_model(raw, 31, tmp_path_factory.mktemp(f"mazanex_{name}")) for name, raw in CONFIGS.items()}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def expected(name, folder, cache, requests):
    key = (name, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in cache:
        cache[key] = mu.plain_logits(folder, requests)
    return cache[key]


def requests_of(name, seed, lengths):
    return ru.make_requests({"vocab_size": CONFIGS[name]["vocab"]}, seed, lengths)


TRACES = {
    "whole": ru.trace_whole,
    "tail": lambda r: ru.trace_tail(r, 32),
    "portions": ru.trace_portions,
    "mixed": lambda r: ru.trace_mixed(r, 5, max_live=4),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("mode", list(TRACES))
def test_replay_matches_plain(name, mode, dtype, folders, plain_cache, tmp_path):
    requests = requests_of(name, 3, LENGTHS[name])
    trace = TRACES[mode](requests)
    print(f"replay {name} {mode} {dtype}: {len(trace.steps)} steps", flush=True)
    got = ru.run_trace(folders[name], dtype, trace, tmp_path, block_size=BLOCKS[name])
    worst = mu.compare(got, expected(name, folders[name], plain_cache, requests), dtype)
    print(f"  worst difference {worst:.3e} of the spread", flush=True)


def long_memory(folder, target):
    """A copy of a model whose recurrent states forget slowly and whose attention is sharp, so that
    a token hundreds of positions back, or one just inside a chunk's edge, moves the logits."""
    raw, weights = mu.folder_weights(folder)
    for index, layer in enumerate(raw["layers"]):
        p = f"l{index}.mix."
        if layer["type"] == "parallel":
            weights[p + "right.w0"] = torch.full_like(weights[p + "right.w0"], -5.5)      # decay exp(-exp(-5.5)) = 0.996
            weights[p + "left.q"] = weights[p + "left.q"] * 6.0
            weights[p + "left.sink"] = torch.full_like(weights[p + "left.sink"], -2.0)
        elif layer["type"] == "gla":
            weights[p + "a2.b"] = torch.full_like(weights[p + "a2.b"], 7.0)
        else:
            weights[p + "f.b"] = torch.full_like(weights[p + "f.b"], 9.0)
            weights[p + "i.b"] = torch.full_like(weights[p + "i.b"], -1.0)
    target.mkdir(parents=True, exist_ok=True)
    (target / "config.json").write_text(json.dumps(raw))
    save_file({n: t.contiguous() for n, t in weights.items()}, str(target / "model.safetensors"))
    return target


def test_far_tokens_reach_the_logits_through_the_states(folders, tmp_path):
    """A control on the weights made below: with them, changing the third token of 600 changes the
    last token's logits by more than the float32 bound of these tests."""
    folder = long_memory(folders["W"], tmp_path / "long")
    raw, weights = mu.folder_weights(folder)
    tokens = requests_of("W", 41, (600,))["r0"]
    other = list(tokens)
    other[2] = (other[2] + 1) % raw["vocab"]
    a, b = plain.forward(raw, weights, tokens)[-1], plain.forward(raw, weights, other)[-1]
    assert float((a - b).abs().max() / (a - a.mean()).abs().max()) > 1e-3      # five times that bound


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_with_long_memory(dtype, folders, tmp_path):
    """600 and 333 tokens: whole, then most of it in one step and the rest token by token over two
    chunk edges, then in portions; every position compared."""
    folder = long_memory(folders["W"], tmp_path / "long")
    requests = requests_of("W", 41, (600, 333))
    want = mu.plain_logits(folder, requests)
    for label, trace in (("whole", ru.trace_whole(requests)), ("tail", ru.trace_tail(requests, 100)),
                         ("portions", ru.trace_portions(requests, sizes=(130, 2, 47, 3, 96, 17)))):
        got = ru.run_trace(folder, dtype, trace, tmp_path / label, block_size=16)
        print(f"long {label} {dtype}: worst {mu.compare(got, want, dtype):.3e}", flush=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps_equal_eager_steps(dtype, folders):
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model

    _, model = load_model(folders["W"], dtype=dtype, device=DEV)
    requests = requests_of("W", 8, (40, 9, 70))
    results = {}
    for graphs in (False, True):
        runner = ModelRunner(model, block_size=16, block_capacity=64, num_state_slots=4, use_graphs=graphs)
        rows = []
        for name, tokens in requests.items():
            runner.begin(name)
            rows.append(runner.step([StepEntry(name, tokens[:-6], [len(tokens) - 7])]).clone())
        for i in range(6, 0, -1):      # three requests decode together, step after step
            rows.append(runner.step([StepEntry(name, [tokens[-i]], [0]) for name, tokens in requests.items()]).clone())
        for name in requests:
            runner.end(name)
        if graphs:
            assert runner.graph_replays >= 5
        results[graphs] = torch.cat(rows).cpu()
    torch.testing.assert_close(results[True], results[False], atol=1e-5 if dtype == "float32" else 2e-2, rtol=1e-4)


def test_first_tokens_and_slot_reuse_start_from_zero_state(folders):
    """A request of one token, then another request in the same slot: its state starts at zero."""
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model

    _, model = load_model(folders["B"], dtype="float32", device=DEV)
    runner = ModelRunner(model, block_size=8, block_capacity=8, num_state_slots=1)
    requests = requests_of("B", 12, (30, 1, 17))
    want = mu.plain_logits(folders["B"], requests)
    for name, tokens in requests.items():
        runner.begin(name)
        logits = runner.step([StepEntry(name, tokens, list(range(len(tokens))))]).cpu()
        runner.end(name)
        mu.compare({(name, i): logits[i] for i in range(len(tokens))}, {k: v for k, v in want.items() if k[0] == name}, "float32")


def test_generation_through_the_entry_point_and_the_command_line(folders):
    from forge_engine_amd.config import SchedulerConfig
    from forge_engine_amd.engine import engine_from_folder
    from forge_engine_amd.sampling import SamplingParams

    prompts = list(requests_of("A", 13, (11, 3, 25)).values())
    want = [mu.plain_greedy(folders["A"], prompt, 8) for prompt in prompts]
    engine = engine_from_folder(folders["A"], scheduler_config=SchedulerConfig(block_size=4, block_capacity=128, token_budget=16),
                                dtype="float32", eos_token_ids=[])
    ids = [engine.submit(prompt, sampling_params=SamplingParams(max_new_tokens=8)) for prompt in prompts]
    engine.run_until_idle()
    assert [list(engine.request(i).output_token_ids) for i in ids] == want
    command = [sys.executable, str(ROOT / "bin" / "forge-engine"), "generate", "--model", str(folders["A"]), "--dtype", "float32",
               "--max-new-tokens", "8", "--block-size", "4", "--prompt-ids", ",".join(map(str, prompts[0]))]
    done = subprocess.run(command, capture_output=True, text=True, timeout=300, env=dict(os.environ))
    assert done.returncode == 0, done.stderr[-2000:]
    assert ",".join(map(str, want[0])) in done.stdout.replace(" ", "")


@pytest.fixture(scope="module")
def ops():
    from forge_engine_amd.kernels import ops as real_ops
    return real_ops


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk,block_size", [(24, 16), (7, 4), (64, 8), (80, 32), (5, 16)])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 32, 16), (6, 3, 64, 64), (8, 1, 128, 128)])
def test_a_key_just_outside_the_chunk_is_not_seen_and_one_just_inside_is(ops, dtype, chunk, block_size, heads, kv_heads, dim, vdim):
    """Keys whose scores would dominate sit just before every chunk's first position and at it;
    the attention kernel is compared with the plain chunked attention, for a prompt's portion and
    for single tokens, and the sink alone is seen by a chunk's first token.  Heads of 64 and 128 in
    bfloat16 with pages of 16 or more take the matrix-core kernels, the others the vector-ALU one."""
    g = torch.Generator().manual_seed(chunk)
    length = 3 * chunk + 5
    q = torch.randn(length, heads, dim, generator=g)
    k = torch.randn(length, kv_heads, dim, generator=g)
    v = torch.randn(length, kv_heads, vdim, generator=g)
    for edge in range(chunk, length, chunk):
        k[edge - 1] *= 8.0          # the last key of the chunk before: outside for every token from `edge` on
        k[edge] *= 4.0              # the chunk's first key: inside
    q, k, v = (t.to(dtype) for t in (q, k, v))
    sink = torch.tensor([0.5, -1.0, 3.0, 0.0, 6.0, -4.0, 1.0, 2.0])[:heads]
    positions = torch.arange(length)
    want = plain.chunked_sink_attention(q.double(), k.double(), v.double(), positions, scale=0.4, chunk=chunk,
                                        sink=sink.double()).reshape(length, heads * vdim).float()
    pages = -(-length // block_size)
    order = torch.randperm(pages + 2, generator=g)[:pages].to(torch.int32)
    key_pages = torch.zeros(pages + 2, kv_heads, block_size, dim, dtype=dtype)
    value_pages = torch.zeros(pages + 2, kv_heads, vdim, block_size, dtype=dtype)
    for p in range(length):
        key_pages[order[p // block_size], :, p % block_size] = k[p]
        value_pages[order[p // block_size], :, :, p % block_size] = v[p]
    common = dict(q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, scale=0.4, chunk=chunk, sink=sink.to(DEV))
    # a portion: the last 2 * chunk + 1 tokens as one step over a cache that holds everything
    first = length - (2 * chunk + 1)
    out = torch.zeros(length - first, heads * vdim, dtype=dtype, device=DEV)
    ops.masked_attention(q[first:].reshape(length - first, -1).to(DEV), key_pages.to(DEV), value_pages.to(DEV), out,
                         torch.tensor([0, length - first], dtype=torch.int32, device=DEV),
                         torch.tensor([length], dtype=torch.int32, device=DEV), order.view(1, -1).to(DEV), num_seqs=1,
                         max_q_len=length - first, **common)
    bound = dict(atol=2e-2, rtol=2e-2) if dtype == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(out.cpu().float(), want[first:], **bound)
    # single tokens: every position as a sequence of its own over the same pages
    singles = list(range(chunk - 1, length))
    n = len(singles)
    out = torch.zeros(n, heads * vdim, dtype=dtype, device=DEV)
    ops.masked_attention(q[singles].reshape(n, -1).to(DEV), key_pages.to(DEV), value_pages.to(DEV), out,
                         torch.arange(n + 1, dtype=torch.int32, device=DEV),
                         torch.tensor([p + 1 for p in singles], dtype=torch.int32, device=DEV),
                         order.view(1, -1).repeat(n, 1).to(DEV), num_seqs=n, max_q_len=1, **common)
    torch.testing.assert_close(out.cpu().float(), want[singles], **bound)
