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


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot", [(4, 2, 16, 24, 8), (6, 3, 128, 128, 32), (2, 2, 12, 20, 12), (3, 1, 64, 8, 0)])
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


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 16, 24), (6, 3, 128, 128), (2, 2, 12, 20)])
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


@pytest.mark.parametrize("tokens,hidden,experts,top,inner", [(1, 48, 5, 2, 20), (37, 64, 3, 1, 36), (150, 256, 8, 2, 64), (70, 40, 4, 4, 100)])
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
