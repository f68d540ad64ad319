"""Rekezen on the GPU: its kernels alone against their plain references (tests/kernel_refs.py), and
the model against the plain implementation (tests/plain_rekezen.py) in float32 and bfloat16 over
traces that cut the same requests in different ways."""

from __future__ import annotations

import pytest
import torch

import kernel_refs as refs
import rekezen_util as ku
import replay_util as ru

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

CONFIGS = dict(ku.CONFIGS, M=ku.MEDIUM)
LENGTHS = {"A": (5, 1, 14, 27, 90), "B": (2, 9, 21, 33, 64), "C": (7, 18, 3, 1, 40), "M": (4, 45, 150, 83, 1)}
BLOCKS = dict(ku.BLOCK_SIZE, M=16)


def close(got, want, dtype):
    if dtype == torch.float32:
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-5, atol=2e-5)
    else:
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-2, atol=2e-2)


# ------------------------------------------------------------------ kernels alone

@pytest.mark.parametrize("streams,width,parts", [(1, 40, 0), (3, 48, 1), (4, 256, 3), (8, 130, 2), (2, 4096, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hyper_norm_kernel(streams, width, parts, dtype):
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(streams * 100 + width)
    rows = 37
    x = torch.randn(streams, rows, width, generator=g) * 3
    update = None if parts == 0 else (torch.randn(rows, width, generator=g) if parts == 1 else torch.randn(parts, rows, width, generator=g))
    mix = torch.eye(streams) + 0.2 * torch.randn(streams, streams, generator=g)
    share, read = torch.randn(streams, generator=g), torch.randn(streams, generator=g)
    weight, bias = 1 + 0.1 * torch.randn(width, generator=g), 0.1 * torch.randn(width, generator=g)
    for use_mix, use_read, rms, chosen in ((True, True, False, None), (False, False, True, None), (True, False, False, [5, 0, 36, 5])):
        want_x = x.clone()
        pick = None if chosen is None else torch.tensor(chosen, dtype=torch.int32)
        n = rows if chosen is None else len(chosen)
        want = refs.hyper_norm(want_x, update, mix if use_mix else None, share if use_mix else None, read if use_read else None,
                               weight, None if rms else bias, 1e-5, torch.empty(n, width, dtype=dtype), rows=pick,
                               store=chosen is None, rms=rms)
        got_x = x.clone().to(DEV)
        got = ops.hyper_norm(got_x, None if update is None else update.to(DEV), mix.to(DEV) if use_mix else None,
                             share.to(DEV) if use_mix else None, read.to(DEV) if use_read else None, weight.to(DEV),
                             None if rms else bias.to(DEV), 1e-5, torch.empty(n, width, dtype=dtype, device=DEV),
                             rows=None if pick is None else pick.to(DEV), store=chosen is None, rms=rms)
        close(got, want, dtype)
        close(got_x, want_x, torch.float32)
    if update is not None:      # the update alone, nothing read
        want_x, got_x = x.clone(), x.clone().to(DEV)
        refs.hyper_norm(want_x, update, mix, share, None, None, None, 0.0, None)
        ops.hyper_norm(got_x, update.to(DEV), mix.to(DEV), share.to(DEV), None, None, None, 0.0, None)
        close(got_x, want_x, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_pair_embedding_kernel(dtype):
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    vocab, hidden, buckets = 70, 24, 13
    table, pairs = torch.randn(vocab, hidden, generator=g).to(dtype), torch.randn(buckets + 1, hidden, generator=g).to(dtype)
    # three sequences: one from its first token, one going on (its first token of the step reads the slot), one single token
    ids = torch.tensor([3, 9, 9, 60, 1, 2, 69], dtype=torch.int32)
    positions = torch.tensor([0, 1, 2, 7, 8, 9, 4], dtype=torch.int32)
    token_seq = torch.tensor([0, 0, 0, 1, 1, 1, 2], dtype=torch.int32)
    cu_q = torch.tensor([0, 3, 6, 7], dtype=torch.int32)
    slots = torch.tensor([2, 0, 3], dtype=torch.int32)
    previous = torch.tensor([[41], [7], [55], [12], [0]], dtype=torch.int32)
    want_prev, want = previous.clone(), torch.empty(7, hidden)
    refs.embed_token_pairs(ids, table, pairs, positions, token_seq, cu_q, slots, want_prev, want, num_seqs=3, buckets=buckets,
                           mul_prev=1000003, mul_cur=77)
    got_prev, got = previous.clone().to(DEV), torch.empty(7, hidden, device=DEV)
    ops.embed_token_pairs(ids.to(DEV), table.to(DEV), pairs.to(DEV), positions.to(DEV), token_seq.to(DEV), cu_q.to(DEV), slots.to(DEV),
                          got_prev, got, num_seqs=3, buckets=buckets, mul_prev=1000003, mul_cur=77)
    assert torch.equal(got.cpu(), want) and torch.equal(got_prev.cpu(), want_prev)
    assert want_prev[:, 0].tolist() == [2, 7, 9, 69, 0]


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot", [(4, 2, 16, 24, 8), (6, 2, 128, 128, 64), (2, 2, 12, 20, 12), (3, 1, 64, 8, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_norm_rope_write_kernel(heads, kv_heads, dim, vdim, rot, dtype):
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(heads + dim)
    tokens, block, pages = 9, 4, 12
    width = heads * dim + kv_heads * (dim + vdim) + 5
    qkv = (torch.randn(tokens, width, generator=g) * 2).to(dtype)
    qw, kw = 1 + 0.2 * torch.randn(heads * dim, generator=g), 1 + 0.2 * torch.randn(kv_heads * dim, generator=g)
    inv_freq = torch.rand(max(rot // 2, 1), generator=g)[:rot // 2]
    positions = torch.tensor([0, 1, 2, 3, 4, 17, 18, 19, 1000], dtype=torch.int32)
    token_seq = torch.tensor([0, 0, 0, 0, 0, 1, 1, 1, 2], dtype=torch.int32)
    table = torch.full((3, 251), -1, dtype=torch.int32)
    table[0, :2] = torch.tensor([3, 7])
    table[1, 4] = 1
    table[2, 250] = 11
    for write_kv in (True, False):
        want_k, want_v = torch.zeros(pages, kv_heads, block, dim, dtype=dtype), torch.zeros(pages, kv_heads, vdim, block, dtype=dtype)
        want_q = torch.empty(tokens, heads * dim, dtype=dtype)
        args = dict(q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, rotary_dim=rot, eps=1e-5, magnitude=1.3, write_kv=write_kv)
        refs.whole_norm_rope_write(qkv, qw, kw, inv_freq, positions, token_seq, table, want_k, want_v, want_q, **args)
        got_k, got_v, got_q = torch.zeros_like(want_k, device=DEV), torch.zeros_like(want_v, device=DEV), torch.empty_like(want_q, device=DEV)
        ops.whole_norm_rope_write(qkv.to(DEV), qw.to(DEV), kw.to(DEV), inv_freq.to(DEV), positions.to(DEV), token_seq.to(DEV), table.to(DEV),
                                  got_k, got_v, got_q, **args)
        # position 1000 turns by up to 1000 radians: float32 angles differ in their last bits
        for got, want in ((got_q, want_q), (got_k, want_k), (got_v, want_v)):
            torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-2 if dtype == torch.bfloat16 else 1e-4,
                                       atol=2e-2 if dtype == torch.bfloat16 else 5e-4)
        assert write_kv or not bool(got_k.any())


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 16, 24), (8, 2, 128, 128), (2, 2, 12, 20)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_masked_attention_with_cap_and_head_gates(heads, kv_heads, dim, vdim, dtype):
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(dim)
    block, pages = 8, 40
    q_lens, ctx = [1, 5, 30, 1], [70, 5, 47, 1]
    tokens = sum(q_lens)
    q = (torch.randn(tokens, heads * dim, generator=g) * 2).to(dtype)
    gate = torch.randn(tokens, heads + 3, generator=g).to(dtype)[:, 2:2 + heads]
    keys = torch.randn(pages, kv_heads, block, dim, generator=g).to(dtype)
    values = torch.randn(pages, kv_heads, vdim, block, generator=g).to(dtype)
    cu_q = torch.tensor([0, 1, 6, 36, 37], dtype=torch.int32)
    ctx_len = torch.tensor(ctx, dtype=torch.int32)
    perm = torch.randperm(pages, generator=g).to(torch.int32)
    table = torch.full((4, 9), -1, dtype=torch.int32)
    at = 0
    for s, n in enumerate(ctx):
        need = -(-n // block)
        table[s, :need] = perm[at:at + need]
        at += need
    args = dict(num_seqs=4, max_q_len=30, q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, scale=0.9, softcap=2.5,
                head_gate=True)
    want = refs.masked_attention(q, keys, values, torch.empty(tokens, heads * vdim, dtype=dtype), cu_q, ctx_len, table, gate=gate, **args)
    got = ops.masked_attention(q.to(DEV), keys.to(DEV), values.to(DEV), torch.empty(tokens, heads * vdim, dtype=dtype, device=DEV),
                               cu_q.to(DEV), ctx_len.to(DEV), table.to(DEV), gate=gate.to(DEV), num_decode=2, max_ctx=72, **args)
    close(got, want, dtype)


@pytest.mark.parametrize("tokens,hidden,experts,top,inner", [(1, 48, 5, 2, 20), (37, 64, 3, 1, 36), (150, 256, 6, 2, 96), (70, 40, 4, 4, 100), (600, 128, 4, 2, 160)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixture_of_experts_kernels(tokens, hidden, experts, top, inner, dtype):
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(tokens + experts)
    x = torch.randn(tokens, hidden, generator=g).to(dtype)
    router, bias = (torch.randn(experts, hidden, generator=g) * 0.5).to(dtype), torch.randn(experts, generator=g)
    gate_up = (torch.randn(experts, 2 * inner, hidden, generator=g) * 0.3).to(dtype)
    down = (torch.randn(experts, hidden, inner, generator=g) * 0.2).to(dtype)
    want_chosen, want_weights = refs.moe_route(x, router, bias, top)
    chosen, weights = ops.moe_route(x.to(DEV), router.to(DEV), bias.to(DEV), top)
    assert torch.equal(chosen.cpu(), want_chosen)
    torch.testing.assert_close(weights.cpu(), want_weights, rtol=1e-4, atol=1e-5)
    want = refs.moe_experts(x, want_chosen, want_weights, gate_up, down, torch.empty(top, tokens, hidden), limit=1.2, alpha=1.702)
    got = ops.moe_experts(x.to(DEV), chosen, weights, gate_up.to(DEV), down.to(DEV), torch.empty(top, tokens, hidden, device=DEV),
                          limit=1.2, alpha=1.702)
    close(got, want, dtype)
    for extra in (torch.randn(tokens, hidden, generator=g), torch.randn(3, tokens, hidden, generator=g)):   # what every token gets beside
        want = refs.moe_experts(x, want_chosen, want_weights, gate_up, down, torch.empty(top, tokens, hidden), limit=1.2, alpha=1.702,
                                extra=extra)
        got = ops.moe_experts(x.to(DEV), chosen, weights, gate_up.to(DEV), down.to(DEV), torch.empty(top, tokens, hidden, device=DEV),
                              limit=1.2, alpha=1.702, extra=extra.to(DEV))
        close(got, want, dtype)
    shared = (torch.randn(2 * inner, hidden, generator=g) * 0.3).to(dtype)
    close(ops.linear_gated(x.to(DEV), shared.to(DEV), limit=0.8, alpha=1.702), refs.linear_gated(x, shared, limit=0.8, alpha=1.702), dtype)


# ------------------------------------------------------------------ the model

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: ku.write_model(raw, 31, tmp_path_factory.mktemp(f"rekezen_{name}")) for name, raw in CONFIGS.items()}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def expected(name, folder, cache, requests):
    key = (name, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in cache:
        cache[key] = ku.plain_logits(folder, requests)
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
    worst = ku.compare(got, expected(name, folders[name], plain_cache, requests), dtype)
    print(f"  worst difference {worst:.3e}", flush=True)


def sharp(folder, target, factor=6.0):
    """A copy of a model whose attention is sharp (larger norm weights on q, no cap below the scores'
    range), so that one key among hundreds, however far back, moves the logits."""
    import json
    from safetensors.torch import save_file
    raw, weights = ku.folder_weights(folder)
    for index, layer in enumerate(raw["layers"]):
        weights[f"l{index}.mix.q.norm"] = weights[f"l{index}.mix.q.norm"] * factor
        if "softcap" in layer["mixer"]:
            layer["mixer"]["softcap"] = 40.0
    target.mkdir(parents=True, exist_ok=True)
    (target / "config.json").write_text(json.dumps(raw))
    save_file({n: t.contiguous() for n, t in weights.items()}, str(target / "model.safetensors"))
    return target


def test_far_tokens_reach_the_logits(folders, tmp_path):
    """A control on the weights made above: with them, changing the third token of 500 changes the
    last token's logits by more than the float32 bound of these tests."""
    folder = sharp(folders["M"], tmp_path / "sharp")
    cfg, weights = ku.folder_weights(folder)
    tokens = requests_of("M", 8, (500,))["r0"]
    other = list(tokens)
    other[2] = (other[2] + 1) % cfg["vocab"]
    a, b = ku.plain.forward(tokens, weights, cfg)[-1], ku.plain.forward(other, weights, cfg)[-1]
    assert float((a - b).abs().max()) > 1000 * (1e-5 + 1e-4 * float(a.abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_with_sharp_attention(dtype, folders, tmp_path):
    """Prompts of several hundred tokens whose far keys matter: whole, then the last 40 tokens one by
    one (across page borders), then in portions, then three at once."""
    folder = sharp(folders["M"], tmp_path / "sharp")
    requests = requests_of("M", 9, (500, 333, 129))
    want = ku.plain_logits(folder, requests)
    for mode, trace in (("whole", ru.trace_whole(requests)), ("tail", ru.trace_tail(requests, 40)),
                        ("portions", ru.trace_portions(requests, sizes=(64, 17, 2, 130, 3, 48, 16, 2, 33), want_all=False)),
                        ("mixed", ru.trace_mixed(requests, 11, max_live=3))):
        print(f"sharp {mode} {dtype}: {len(trace.steps)} steps", flush=True)
        got = ru.run_trace(folder, dtype, trace, tmp_path / mode, block_size=16)
        # scores of up to 40 turn an error of one part in 10**7 in a key into one of some parts in 10**5 in a
        # softmax weight: float32 differs from the plain implementation by up to 1e-4 here (the plain
        # implementation in float32 does too); a key left out moves these logits by a hundred times that
        ku.compare(got, want, dtype, fraction=0.1, float32_factor=10.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block_size", [4, 16, 32])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 32, 16), (6, 3, 64, 64), (8, 1, 128, 128)])
def test_one_far_key_among_hundreds_is_found(dtype, block_size, heads, kv_heads, dim, vdim):
    """Keys whose scores dominate sit at the first position, just before and at page borders and hundreds
    of positions back: the attention kernels (matrix cores for heads of 64 and 128 in bfloat16 with pages
    of 16 or more, the vector ALU otherwise) against the plain capped attention, for a prompt's portion
    behind cached keys and for single tokens; with a cap that the dominant scores reach."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(dim + block_size)
    length, cached = 420, 391          # the portion's 29 tokens lie behind 391 cached ones
    q = torch.randn(length, heads, dim, generator=g)
    k = torch.randn(length, kv_heads, dim, generator=g)
    v = torch.randn(length, kv_heads, vdim, generator=g)
    for far in (0, block_size - 1, block_size, 7 * block_size - 1, 7 * block_size, 200, cached - 1, cached):
        k[far] *= 5.0
    q, k, v = (t.to(dtype) for t in (q, k, v))
    cap, scale = 9.0, 0.3
    want = ku.plain.capped_causal_attention(q.double(), k.double(), v.double(), scale=scale, softcap=cap)
    gates = torch.randn(length, heads, generator=g).to(dtype)
    want = (want * torch.sigmoid(gates.double())[:, :, None]).reshape(length, heads * vdim).float()
    pages = -(-length // block_size)
    perm = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)
    key_pages = torch.zeros(pages + 3, kv_heads, block_size, dim, dtype=dtype)
    value_pages = torch.zeros(pages + 3, kv_heads, vdim, block_size, dtype=dtype)
    for p in range(length):
        key_pages[perm[p // block_size], :, p % block_size] = k[p]
        value_pages[perm[p // block_size], :, :, p % block_size] = v[p]
    key_pages, value_pages = key_pages.to(DEV), value_pages.to(DEV)
    table = perm.view(1, -1).to(DEV)
    common = dict(q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, scale=scale, softcap=cap, head_gate=True)
    # the portion
    out = torch.empty(length - cached, heads * vdim, dtype=dtype, device=DEV)
    ops.masked_attention(q[cached:].reshape(length - cached, -1).to(DEV), key_pages, value_pages, out,
                         torch.tensor([0, length - cached], dtype=torch.int32, device=DEV), torch.tensor([length], dtype=torch.int32, device=DEV),
                         table, num_seqs=1, max_q_len=length - cached, gate=gates[cached:].to(DEV), num_decode=0, max_ctx=length, **common)
    close(out, want[cached:], dtype)
    # single tokens: the same request at eight of its lengths, as eight sequences of one step
    places = [0, block_size - 1, block_size, 7 * block_size, 201, cached - 1, cached, length - 1]
    n = len(places)
    out = torch.empty(n, heads * vdim, dtype=dtype, device=DEV)
    ops.masked_attention(q[places].reshape(n, -1).to(DEV), key_pages, value_pages, out,
                         torch.arange(n + 1, dtype=torch.int32, device=DEV), torch.tensor([p + 1 for p in places], dtype=torch.int32, device=DEV),
                         table.expand(n, -1).contiguous(), num_seqs=n, max_q_len=1, gate=gates[places].to(DEV), num_decode=n,
                         max_ctx=length, **common)
    close(out, want[places], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps_equal_eager_steps_and_long_decoding(dtype, folders):
    """A prompt and then 150 single tokens, two requests side by side: steps replayed from captured graphs
    against the same steps run eagerly, and both against the plain implementation."""
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model
    _, model = load_model(folders["M"], dtype=dtype, device=DEV)
    requests = requests_of("M", 21, (160, 171))
    want = ku.plain_logits(folders["M"], requests)
    results = {}
    for graphs in (True, False):
        runner = ModelRunner(model, block_size=16, block_capacity=40, num_state_slots=3, use_graphs=graphs, eager_sightings=1)
        got = {}
        for name in requests:
            runner.begin(name)
        at = {"r0": 10, "r1": 21}
        logits = runner.step([StepEntry(n, requests[n][:at[n]], [at[n] - 1]) for n in requests])
        for row, n in zip(logits, requests):
            got[(n, at[n] - 1)] = row.cpu().clone()
        for _ in range(150):
            logits = runner.step([StepEntry(n, [requests[n][at[n]]], [0]) for n in requests])
            for row, n in zip(logits, requests):
                got[(n, at[n])] = row.cpu().clone()
                at[n] += 1
        assert runner.graph_replays >= (140 if graphs else 0) and (graphs or runner.graph_replays == 0)
        results[graphs] = got
        ku.compare(got, want, dtype, fraction=0.1)
    for key, row in results[True].items():
        torch.testing.assert_close(row, results[False][key], rtol=0, atol=0 if dtype == "float32" else 1e-2)


def test_first_tokens_and_slot_reuse(folders):
    """A request that takes over the state slot of one that ended: its first token has no token before
    it, whatever the slot still holds; requests of one and two tokens."""
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model
    _, model = load_model(folders["A"], dtype="float32", device=DEV)
    runner = ModelRunner(model, block_size=4, block_capacity=16, num_state_slots=1)
    cfg, weights = ku.folder_weights(folders["A"])
    for tokens in ([5, 90, 17, 3], [44], [7, 7], [90, 5, 17, 3, 3, 3, 8, 1, 2]):
        runner.begin("only")
        rows = []
        for token in tokens:          # token by token: every token's predecessor comes from the slot
            rows.append(runner.step([StepEntry("only", [token], [0])])[0].cpu().clone())
        runner.end("only")
        want = ku.plain.forward(tokens, weights, cfg)
        for got, expected in zip(rows, want):
            assert float((got.double() - expected).abs().max()) <= 1e-5 + 1e-4 * float(expected.abs().max())


def test_generation_through_the_entry_point_and_the_command_line(folders):
    import os
    import subprocess
    import sys
    from conftest import ROOT
    from forge_engine_amd.config import SchedulerConfig
    from forge_engine_amd.engine import engine_from_folder
    from forge_engine_amd.sampling import SamplingParams

    cfg, weights = ku.folder_weights(folders["A"])

    def greedy(prompt, count):
        tokens = list(prompt)
        for _ in range(count):
            tokens.append(int(ku.plain.forward(tokens, weights, cfg)[-1].argmax()))
        return tokens[len(prompt):]

    prompts = list(requests_of("A", 13, (11, 3, 25)).values())
    want = [greedy(prompt, 8) for prompt in prompts]
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
