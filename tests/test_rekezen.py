"""Rekezen through the engine on the CPU, with the kernels' plain references patched in, against
the plain implementation (tests/plain_rekezen.py): configuration and tensor names, and that logits
do not depend on how requests are cut into steps, batched, or placed in pages and state slots.
The kernels themselves run in the GPU tests."""

from __future__ import annotations

import pytest
import torch

import kernel_refs
import rekezen_util as ku
import replay_util as ru
from forge_engine_amd.config import ConfigError, SchedulerConfig, load_model_config
from forge_engine_amd.engine import build_engine, load_model
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.weights.random_init import declared_tensors

LENGTHS = {"A": (5, 1, 14, 27), "B": (2, 9, 21, 33), "C": (7, 18, 3, 1)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: ku.write_model(raw, 11, tmp_path_factory.mktemp(f"rekezen_{name}")) for name, raw in ku.CONFIGS.items()}


def requests_of(name, seed, lengths):
    return ru.make_requests({"vocab_size": ku.CONFIGS[name]["vocab"]}, seed, lengths)


def test_configuration_names_and_shapes():
    config = load_model_config(ku.SMALL_A)
    assert config.architecture == "Rekezen" and load_model_config(config.to_dict()) == config
    tensors = declared_tensors(config)
    for name, shape in {"embed": (96, 48), "bigram": (54, 48), "final.norm": (48,), "final.norm.b": (48,), "l0.norm1": (48,),
                        "l0.norm2.b": (48,), "l0.mix.q": (64, 48), "l0.mix.k": (32, 48), "l0.mix.v": (48, 48),
                        "l0.mix.q.norm": (64,), "l0.mix.k.norm": (32,), "l0.mix.g": (4, 48), "l0.mix.o": (48, 96),
                        "l0.mlp.router": (5, 48), "l0.mlp.router.b": (5,), "l0.mlp.e4.gate": (20, 48), "l0.mlp.e0.down": (48, 20),
                        "l0.mlp.shared.up": (28, 48), "l0.hc1.in": (3,), "l0.hc2.mix": (3, 3), "l1.hc1.out": (3,),
                        "l2.mix.q": (64, 48), "l2.mix.g": (4, 48), "l2.mlp.e2.up": (36, 48)}.items():
        assert tuple(tensors[name].shape) == shape, name
    # a layer that borrows keys and values has no tensors for them; a layer without a feed-forward none of its
    assert not any(n in tensors for n in ("l2.mix.k", "l2.mix.v", "l2.mix.k.norm", "l1.norm2", "l1.hc2.in", "l2.mlp.shared.up", "head"))
    assert not any(n.startswith("l1.mlp") for n in tensors)
    plain = declared_tensors(load_model_config(ku.SMALL_C))
    assert "bigram" not in plain and not any(".hc" in n for n in plain)
    borrowed = ku.layer(ku.attention(4, 2, 16, 24, 8, kv_from=1), None)
    for broken in ({**ku.SMALL_A, "layers": []},
                   {**ku.SMALL_A, "layers": [{**ku.SMALL_A["layers"][0], "type": "conv"}]},
                   {**ku.SMALL_A, "layers": [ku.layer(ku.attention(3, 2, 8, 8, 4), None)]},
                   {**ku.SMALL_A, "layers": [ku.layer(ku.attention(2, 2, 8, 8, 10), None)]},
                   {**ku.SMALL_A, "layers": [ku.SMALL_A["layers"][0], borrowed]},                # the source is no earlier layer
                   {**ku.SMALL_A, "layers": [*ku.SMALL_A["layers"], ku.layer(ku.attention(4, 2, 16, 24, 8, kv_from=2), None)]},   # the source borrows itself
                   {**ku.SMALL_A, "layers": [ku.SMALL_A["layers"][0], ku.layer(ku.attention(4, 2, 8, 24, 8, kv_from=0), None)]},  # another key size
                   {**ku.SMALL_A, "layers": [ku.layer(ku.attention(2, 2, 8, 8, 4), ku.moe(2, 3, 8, 1.0))]},
                   {k: v for k, v in ku.SMALL_A.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            load_model_config(broken)


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(name, mode, folders, tmp_path, monkeypatch):
    """Whole prompts; a prompt and then token by token; portions down to two tokens; up to three
    live requests, portions beside single tokens."""
    kernel_refs.install(monkeypatch)
    requests = requests_of(name, 3, LENGTHS[name])
    trace = {"whole": ru.trace_whole, "tail": lambda r: ru.trace_tail(r, 16), "portions": ru.trace_portions,
             "mixed": lambda r: ru.trace_mixed(r, 5, max_live=3)}[mode](requests)
    got = ru.run_trace(folders[name], "float32", trace, tmp_path, block_size=ku.BLOCK_SIZE[name], device="cpu", on_cpu=True)
    ku.compare(got, ku.plain_logits(folders[name], requests), "float32")


def test_pages_and_state_slots_are_used_again(folders, tmp_path, monkeypatch):
    """Seven requests through four state slots and a pool smaller than their sum: the token before a
    request's first one is nobody's, whoever held the slot before."""
    kernel_refs.install(monkeypatch)
    requests = requests_of("A", 4, (12, 20, 7, 16, 9, 3, 11))
    trace = ru.trace_mixed(requests, 9, max_live=4)
    assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens
    got = ru.run_trace(folders["A"], "float32", trace, tmp_path, block_size=4, device="cpu", on_cpu=True)
    ku.compare(got, ku.plain_logits(folders["A"], requests), "float32")


def test_greedy_generation_through_the_scheduler(folders, monkeypatch):
    kernel_refs.install(monkeypatch)
    _, model = load_model(folders["A"], dtype="float32", device="cpu")
    engine = build_engine(model, scheduler_config=SchedulerConfig(block_size=4, block_capacity=64, token_budget=8, max_batch_size=3),
                          eos_token_ids=())
    prompts = list(requests_of("A", 6, (11, 4, 17)).values())
    ids = [engine.submit(prompt, sampling_params=SamplingParams(max_new_tokens=6)) for prompt in prompts]
    engine.run_until_idle()
    cfg, weights = ku.folder_weights(folders["A"])
    for request_id, prompt in zip(ids, prompts):
        tokens = list(prompt)
        for _ in range(6):
            tokens.append(int(ku.plain.forward(tokens, weights, cfg)[-1].argmax()))
        assert list(engine.request(request_id).output_token_ids) == tokens[len(prompt):]


# ------------------------------------------------------------------ each mechanism alone

def _ctx():
    from forge_engine_amd.parts.base import BuildContext
    return BuildContext(torch.device("cpu"), torch.float32)


def _batch(q_lens, before, slots):
    """The metadata of a step: sequence i brings q_lens[i] tokens behind before[i] cached ones."""
    from types import SimpleNamespace
    positions, token_seq, cu_q = [], [], [0]
    for i, (n, b) in enumerate(zip(q_lens, before)):
        positions += list(range(b, b + n))
        token_seq += [i] * n
        cu_q.append(cu_q[-1] + n)
    return SimpleNamespace(num_tokens=cu_q[-1], num_seqs=len(q_lens), positions=torch.tensor(positions, dtype=torch.int32),
                           token_seq=torch.tensor(token_seq, dtype=torch.int32), cu_q=torch.tensor(cu_q, dtype=torch.int32),
                           state_slots=torch.tensor(slots, dtype=torch.int32))


def test_token_pair_embedding_across_steps(monkeypatch):
    """Two sequences fed in pieces of unequal size through one part: the token before a piece's first
    token comes from the slot; multipliers whose products pass 2**31."""
    from forge_engine_amd.cache.spec import CacheView
    from forge_engine_amd.parts.embedding import TokenPairEmbedding
    kernel_refs.install(monkeypatch)
    g = torch.Generator().manual_seed(1)
    vocab, width, buckets, mul_prev, mul_cur = 50000, 12, 97, 1000003, 999983
    part = TokenPairEmbedding(_ctx(), "embed", vocab_size=vocab, hidden_size=width, buckets=buckets, mul_prev=mul_prev,
                              mul_cur=mul_cur, leaf="", pair_name="bigram")
    w = {"embed": torch.randn(vocab, width, generator=g), "bigram": torch.randn(buckets + 1, width, generator=g)}
    for name, tensor in w.items():
        part.set_param(name, tensor)
    cfg = {"embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}
    sequences = [torch.randint(0, vocab, (9,), generator=g).tolist(), torch.randint(40000, vocab, (5,), generator=g).tolist()]
    want = [ku.plain.embed(tokens, {k: v.double() for k, v in w.items()}, cfg) for tokens in sequences]
    state = {part.PREVIOUS: torch.full((4, 1), 12345, dtype=torch.int32)}      # what an earlier request left in the slots
    state[part.PREVIOUS][[3, 1]] = 0                                              # ... cleared when these two began
    cuts = [[(0, 4), (0, 1)], [(4, 5), (1, 3)], [(5, 9), (3, 5)]]
    for step in cuts:
        batch = _batch([b - a for a, b in step], [a for a, _ in step], [3, 1])
        batch.token_ids = torch.tensor([t for (a, b), tokens in zip(step, sequences) for t in tokens[a:b]], dtype=torch.int32)
        h = part.forward(batch, CacheView(states=state)).h
        at = 0
        for (a, b), expected in zip(step, want):
            assert torch.allclose(h[at:at + b - a].double(), expected[a:b], atol=1e-6)
            at += b - a


def test_rotary_tables():
    """Frequencies and magnitude against the plain table: a ramp inside the table, one that starts before
    it, one beyond it (every pair keeps its frequency), no scaling."""
    from forge_engine_amd.parts.rotary import RotaryPosition, YarnRotaryPosition
    for dims, base, scaling in ((24, 20000.0, (6.0, 512, 24.0, 1.0)), (8, 100.0, (8.0, 64, 16.0, 2.0)),
                                (16, 10000.0, (2.0, 1 << 20, 1.0, 0.5)), (12, 300.0, (3.0, 16, 64.0, 32.0))):
        rot = {"dims": dims, "base": base, "scaling": dict(zip(("factor", "original", "fast", "slow"), scaling))}
        part = YarnRotaryPosition(_ctx(), head_dim=dims + 4, theta=base, rotary_dim=dims, factor=scaling[0], original=scaling[1],
                                  fast=scaling[2], slow=scaling[3])
        freq, magnitude = ku.plain.rotary_table(rot)
        assert torch.allclose(part.rotary()[0].double(), freq, rtol=1e-6) and abs(part.magnitude() - magnitude) < 1e-12
        assert part.rotary()[1] == dims
    plain_part = RotaryPosition(_ctx(), head_dim=16, theta=777.0, rotary_dim=6, precise=True)
    assert torch.allclose(plain_part.rotary()[0].double(), ku.plain.rotary_table({"dims": 6, "base": 777.0})[0], rtol=1e-6)
    assert plain_part.magnitude() == 1.0


@pytest.mark.parametrize("streams", [1, 2, 5])
def test_streams_through_a_layer(streams, monkeypatch):
    """One arrangement of several streams around sublayers that are plain functions: the update mixes the
    old streams into the new ones all at once, and the last norm reads their sum."""
    from forge_engine_amd.parts.base import Residual
    from forge_engine_amd.parts.block import HyperConnectionBlock
    from forge_engine_amd.parts.norm import LayerNorm
    kernel_refs.install(monkeypatch)
    g = torch.Generator().manual_seed(streams)
    tokens, width = 7, 10
    x0 = torch.randn(tokens, width, generator=g)
    w = {}
    for q in ("hc1", "hc2"):
        w[f"l.{q}.in"], w[f"l.{q}.out"] = torch.randn(streams, generator=g), torch.randn(streams, generator=g)
        w[f"l.{q}.mix"] = torch.eye(streams) + 0.3 * torch.randn(streams, streams, generator=g)
    for q in ("norm1", "norm2", "last"):
        w[f"l.{q}"], w[f"l.{q}.b"] = 1 + 0.1 * torch.randn(width, generator=g), 0.1 * torch.randn(width, generator=g)
    a, b = torch.randn(width, width, generator=g), torch.randn(width, width, generator=g)

    class Mixer:
        takes_stream = False

        def forward(self, x, batch, cache, writes_cache=True):
            return torch.tanh(x.float() @ a)

        def cache_needs(self):
            return None

    class FeedForward:
        takes_stream = False

        def forward(self, x, batch):
            return torch.stack([0.25 * torch.sin(x.float() @ b), 0.75 * torch.sin(x.float() @ b)])     # an update in two parts

    norms = {role: LayerNorm(_ctx(), f"l.{name}", size=width, eps=1e-5, leaf="", bias_leaf="b")
             for role, name in (("input", "norm1"), ("post_mixer", "norm2"))}
    last = LayerNorm(_ctx(), "l.last", size=width, eps=1e-5, leaf="", bias_leaf="b")
    block = HyperConnectionBlock(_ctx(), Mixer(), FeedForward(), norms, "l", streams=streams)
    for part in (block, last, *norms.values()):
        for name in part.param_specs():
            part.set_param(name, w[name])
    residual = Residual(x0.clone())
    block.forward(residual, None, None)
    block.forward(residual, None, None)       # twice: the pending update of the second sublayer meets the first norm
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    got = last.forward(residual, rows=rows)

    wd = {k: v.double() for k, v in w.items()}
    s = x0.double()[None].repeat(streams, 1, 1)
    for _ in range(2):
        s = ku.plain.hyper_sublayer(s, wd, "l.hc1", lambda u: torch.tanh(ku.plain.layer_norm(u, wd["l.norm1"], wd["l.norm1.b"], 1e-5).float() @ a).double())
        s = ku.plain.hyper_sublayer(s, wd, "l.hc2", lambda u: torch.sin(ku.plain.layer_norm(u, wd["l.norm2"], wd["l.norm2.b"], 1e-5).float() @ b).double())
    want = ku.plain.layer_norm(s.sum(0), wd["l.last"], wd["l.last.b"], 1e-5)[rows.long()]
    assert torch.allclose(got.double(), want, atol=2e-5)


@pytest.mark.parametrize("experts,top,shared", [(5, 2, 12), (3, 3, None), (1, 1, 6), (7, 1, None)])
def test_routed_experts_alone(experts, top, shared, monkeypatch):
    """The feed-forward part against the plain mixture: limits that the products reach, every expert
    chosen, one expert in all, with and without the shared one."""
    from forge_engine_amd.parts.moe import RoutedExperts
    kernel_refs.install(monkeypatch)
    g = torch.Generator().manual_seed(experts * 10 + top)
    width, inner, tokens = 16, 9, 23
    part = RoutedExperts(_ctx(), "m", hidden_size=width, experts=experts, top=top, intermediate_size=inner, limit=0.8,
                         shared_size=shared, shared_limit=0.5, names={"expert": "e{e}", "router": "router", "router_bias": "router.b"})
    w = {}
    for name, spec in part.param_specs().items():
        w[name] = torch.randn(spec.shape, generator=g) * (1.0 if "router" in name else 0.6)
        part.set_param(name, w[name].clone())
    part.finalize()
    x = torch.randn(tokens, width, generator=g)
    mlp = {"router": {"experts": experts, "top": top}, "expert": {"ff": inner, "limit": 0.8}}
    if shared:
        mlp["shared"] = {"ff": shared, "limit": 0.5}
    want = ku.plain.mixture(x.double(), {k: v.double() for k, v in w.items()}, "m", mlp)
    got = part.forward(x)
    assert got.shape[0] == top
    assert torch.allclose(got.sum(0).double(), want, atol=1e-5)
    chosen, weights = ku.plain.routing(x.double(), {k: v.double() for k, v in w.items()}, "m", top)
    assert bool((weights.sum(-1) - 1).abs().max() < 1e-12) and chosen.shape == (tokens, top)


def test_attention_alone_and_with_borrowed_keys(monkeypatch, tmp_path):
    """One-layer and two-layer models of attention alone (no feed-forward, one plain stream): the second
    layer reads the first one's keys and values with its own queries, scale and cap."""
    kernel_refs.install(monkeypatch)
    own = ku.attention(4, 2, 8, 12, 4, scale=0.6, softcap=3.0, scaling=ku.YARN)
    borrowed = ku.attention(4, 2, 8, 12, 4, scale=0.9, softcap=None, scaling=ku.YARN, kv_from=0)
    for layers in ([ku.layer(own, None)], [ku.layer(own, None), ku.layer(borrowed, None)]):
        folder = ku.write_model(ku.config(40, 24, layers), 3, tmp_path / f"attention_{len(layers)}")
        requests = ru.make_requests({"vocab_size": 40}, 2, (19, 1, 6))
        got = ru.run_trace(folder, "float32", ru.trace_portions(requests, sizes=(5, 2, 7, 3)), tmp_path / f"out_{len(layers)}",
                           block_size=4, device="cpu", on_cpu=True)
        ku.compare(got, ku.plain_logits(folder, requests), "float32")


def test_decoding_from_the_first_token(folders, tmp_path, monkeypatch):
    """Every token alone, from the first: 45 steps of one token."""
    kernel_refs.install(monkeypatch)
    requests = requests_of("A", 8, (45,))
    got = ru.run_trace(folders["A"], "float32", ru.trace_tail(requests, 10 ** 6), tmp_path, block_size=4, device="cpu", on_cpu=True)
    ku.compare(got, ku.plain_logits(folders["A"], requests), "float32")


def test_a_checkpoint_may_hold_the_norm_of_a_feed_forward_that_is_not_there(folders, tmp_path, monkeypatch):
    """A layer without a feed-forward reads no second norm and no second set of stream weights; a
    checkpoint that holds them all the same loads, and they change nothing."""
    import json
    import shutil
    from safetensors.torch import load_file, save_file
    kernel_refs.install(monkeypatch)
    folder = shutil.copytree(folders["A"], tmp_path / "more")
    weights = load_file(str(folder / "model.safetensors"))
    assert "l1.norm2" not in weights
    weights.update({"l1.norm2": torch.ones(48).bfloat16(), "l1.norm2.b": torch.ones(48).bfloat16(), "l1.hc2.in": torch.ones(3).bfloat16(),
                    "l1.hc2.out": torch.ones(3).bfloat16(), "l1.hc2.mix": torch.ones(3, 3).bfloat16()})
    save_file({n: t.contiguous() for n, t in weights.items()}, str(folder / "model.safetensors"))
    requests = requests_of("A", 5, (9,))
    got = ru.run_trace(folder, "float32", ru.trace_whole(requests), tmp_path / "out", block_size=4, device="cpu", on_cpu=True)
    ku.compare(got, ku.plain_logits(folders["A"], requests), "float32")
