"""The kernels of the output-norm layers, the short-convolution attention path and the linear
recurrences, each alone against its plain reference (tests/kernel_refs.py): sizes that are no
multiple of a tile, sequences of unequal length with empty ones between, state slots in any
order, both dtypes."""

from __future__ import annotations

import pytest
import torch

import kernel_refs as refs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from forge_engine_amd.kernels import ops as real_ops
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return real_ops


def tol(dtype):
    return dict(atol=2e-2, rtol=2e-2) if dtype == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)


def rand(gen, *shape, dtype=torch.float32, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


def layout(lengths, slots):
    """cu_q, token_seq, state_slots for sequences of the given lengths (0: an empty one)."""
    cu = [0]
    for n in lengths:
        cu.append(cu[-1] + n)
    seq = [i for i, n in enumerate(lengths) for _ in range(n)]
    return (torch.tensor(cu, dtype=torch.int32), torch.tensor(seq, dtype=torch.int32),
            torch.tensor(slots, dtype=torch.int32))


def dev(*tensors):
    return [None if t is None else t.to(DEV) for t in tensors]


LENGTHS = [(5, 0, 1, 19), (1, 1, 1), (70,), (2, 33, 0, 0)]


@pytest.mark.parametrize("x_dtype,out_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                               (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("lengths", LENGTHS)
@pytest.mark.parametrize("width,count", [(24, 1), (200, 5), (1030, 2)])
def test_token_shift(ops, x_dtype, out_dtype, lengths, width, count):
    g = torch.Generator().manual_seed(3)
    cu, seq, slots = layout(lengths, [3, 0, 5, 2][:len(lengths)])
    x = rand(g, cu[-1].item(), width, dtype=x_dtype)
    w = torch.rand(count, width, generator=g)
    state = rand(g, 7, width)
    state_ref = state.clone()
    want = refs.token_shift(x, w, state_ref, cu, seq, slots, num_seqs=len(lengths), out_dtype=out_dtype)
    xd, wd, sd, cud, seqd, slotsd = dev(x, w, state, cu, seq, slots)
    got = ops.token_shift(xd, wd, sd, cud, seqd, slotsd, num_seqs=len(lengths), out_dtype=out_dtype)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(out_dtype))
    torch.testing.assert_close(sd.cpu(), state_ref, atol=0, rtol=0)


@pytest.mark.parametrize("out_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("parts", [0, 3])
@pytest.mark.parametrize("rows,width", [(7, 24), (33, 200), (300, 2050)])
def test_rmsnorm_update(ops, out_dtype, parts, rows, width):
    g = torch.Generator().manual_seed(4)
    h = rand(g, rows, width, scale=2.0)
    update = rand(g, *((parts,) if parts else ()), rows, width, scale=5.0)
    w = 1.0 + rand(g, width, scale=0.1)
    h_ref = h.clone()
    out_ref = None if out_dtype is None else torch.empty(rows, width, dtype=out_dtype)
    refs.rmsnorm_update(h_ref, update, w, 1e-6, out_ref)
    hd, ud, wd = dev(h, update, w)
    out = None if out_dtype is None else torch.empty(rows, width, dtype=out_dtype, device=DEV)
    ops.rmsnorm_update(hd, ud, wd, 1e-6, out)
    torch.testing.assert_close(hd.cpu(), h_ref, atol=2e-5, rtol=2e-5)
    if out is not None:
        torch.testing.assert_close(out.cpu().float(), out_ref.float(), **tol(out_dtype))


@pytest.mark.parametrize("count", [1, 2, 4])
@pytest.mark.parametrize("rows,width", [(5, 40), (129, 1000)])
def test_rmsnorm_mean(ops, count, rows, width):
    g = torch.Generator().manual_seed(5)
    updates = [rand(g, *((2,) if i == 1 else ()), rows, width, scale=float(i + 1)) for i in range(count)]
    w = 1.0 + rand(g, count, width, scale=0.2)
    want = refs.rmsnorm_mean(updates, w, 1e-5, torch.empty(rows, width))
    got = ops.rmsnorm_mean(dev(*updates), w.to(DEV), 1e-5, torch.empty(rows, width, device=DEV))
    torch.testing.assert_close(got.cpu(), want, atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(3, 20), (65, 320), (10, 5000)])
def test_polynorm(ops, dtype, rows, width):
    g = torch.Generator().manual_seed(6)
    z = rand(g, rows, width, dtype=dtype, scale=1.5)
    coeff = torch.tensor([0.7, -0.4, 0.25, 0.1])
    want = refs.polynorm(z, coeff, 1e-6, torch.empty_like(z))
    got = ops.polynorm(z.to(DEV), coeff.to(DEV), 1e-6, torch.empty_like(z, device=DEV))
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))
    for shape in ((9, 40), (3, 9, 40)):
        update, row_bias = rand(g, *shape), rand(g, 40)
        torch.testing.assert_close(ops.add_bias(update.to(DEV), row_bias.to(DEV)).cpu(), refs.add_bias(update.clone(), row_bias))
    x = rand(g, 1000, dtype=dtype, scale=2.0)
    torch.testing.assert_close(ops.tanh_rows(x.to(DEV)).cpu().float(), refs.tanh_rows(x.clone()).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,shared,act,extra", [(4, 32, False, "silu", 0), (3, 64, True, "silu", 0),
                                                        (2, 100, False, "sigmoid", 1), (5, 24, False, "none", 0)])
def test_head_norm_gate(ops, dtype, heads, dim, shared, act, extra):
    g = torch.Generator().manual_seed(7)
    tokens = 37
    o = rand(g, tokens, heads, dim + extra, scale=3.0)
    weight = 1.0 + rand(g, dim if shared else heads * dim, scale=0.2)
    wide = rand(g, tokens, heads * dim + 9, dtype=dtype)
    gate = None if act == "none" else wide[:, 9:]
    floor = torch.rand(tokens, heads, generator=g) * 4.0 if extra else None
    want = refs.head_norm_gate(o, weight, gate, torch.empty(tokens, heads * dim, dtype=dtype), heads=heads, dim=dim, eps=1e-6,
                               act=act, extra=extra, floor=floor)
    wide_d = wide.to(DEV)
    got = ops.head_norm_gate(o.to(DEV), weight.to(DEV), None if gate is None else wide_d[:, 9:],
                             torch.empty(tokens, heads * dim, dtype=dtype, device=DEV), heads=heads, dim=dim, eps=1e-6,
                             act=act, extra=extra, floor=None if floor is None else floor.to(DEV))
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


def attention_case(g, dtype, lengths, before, *, q_heads, kv_heads, head_dim, value_dim, block_size):
    """Pages, tables and lengths for sequences that hold ``before[i]`` tokens and bring ``lengths[i]``."""
    ctx = [b + n for b, n in zip(before, lengths)]
    width = max(1, max(-(-c // block_size) for c in ctx))
    pages = sum(-(-c // block_size) for c in ctx) + 3
    order = torch.randperm(pages, generator=g).tolist()
    table = torch.full((len(lengths), width), -1, dtype=torch.int32)
    for i, c in enumerate(ctx):
        for b in range(-(-c // block_size)):
            table[i, b] = order.pop()
    keys = rand(g, pages, kv_heads, block_size, head_dim, dtype=dtype)
    values = rand(g, pages, kv_heads, value_dim, block_size, dtype=dtype)
    return torch.tensor(ctx, dtype=torch.int32), table, keys, values


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [
    dict(q_heads=6, kv_heads=3, head_dim=64, value_dim=64, block_size=16, taps=3, rotary_dim=32),
    dict(q_heads=3, kv_heads=3, head_dim=24, value_dim=40, block_size=4, taps=2, rotary_dim=12),
    dict(q_heads=6, kv_heads=2, head_dim=128, value_dim=32, block_size=8, taps=0, rotary_dim=0),
    dict(q_heads=2, kv_heads=1, head_dim=256, value_dim=72, block_size=16, taps=1, rotary_dim=2),
])
def test_conv_rope_norm_write(ops, dtype, sizes):
    g = torch.Generator().manual_seed(8)
    lengths, before = [5, 0, 1, 2, 30], [0, 7, 9, 14, 3]
    taps, rotary_dim = sizes["taps"], sizes["rotary_dim"]
    geometry = {k: sizes[k] for k in ("q_heads", "kv_heads", "head_dim", "value_dim")}
    cu, seq, slots = layout(lengths, [2, 4, 0, 1, 3])
    ctx, table, keys, values = attention_case(g, dtype, lengths, before, block_size=sizes["block_size"], **geometry)
    tokens = sum(lengths)
    positions = torch.tensor([b + i for b, n in zip(before, lengths) for i in range(n)], dtype=torch.int32)
    channels = (sizes["q_heads"] + sizes["kv_heads"]) * sizes["head_dim"] + sizes["kv_heads"] * sizes["value_dim"]
    wide = rand(g, tokens, channels + 17, dtype=dtype)
    qkv = wide[:, :channels]
    bias = rand(g, channels) if sizes["value_dim"] != 32 else None
    conv_w = rand(g, channels, taps) if taps else None
    state = rand(g, 6, taps - 1, channels) if taps > 1 else None
    inv_freq = (1.0 / 10000.0 ** (torch.arange(0, rotary_dim, 2).float() / rotary_dim)) if rotary_dim else None
    state_ref = None if state is None else state.clone()
    keys_ref, values_ref = keys.clone(), values.clone()
    q_ref = torch.empty(tokens, sizes["q_heads"] * sizes["head_dim"], dtype=dtype)
    refs.conv_rope_norm_write(qkv, bias, conv_w, state_ref, inv_freq, positions, seq, cu, slots, table, keys_ref, values_ref, q_ref,
                              num_seqs=len(lengths), rotary_dim=rotary_dim, unit_norm_eps=1e-6, taps=taps, **geometry)
    wide_d, conv_d, state_d, freq_d, pos_d, seq_d, cu_d, slots_d, table_d, keys_d, values_d = dev(
        wide, conv_w, state, inv_freq, positions, seq, cu, slots, table, keys, values)
    q_d = torch.empty_like(q_ref, device=DEV)
    ops.conv_rope_norm_write(wide_d[:, :channels], None if bias is None else bias.to(DEV), conv_d, state_d, freq_d, pos_d, seq_d, cu_d, slots_d, table_d, keys_d,
                             values_d, q_d, num_seqs=len(lengths), rotary_dim=rotary_dim, unit_norm_eps=1e-6, taps=taps,
                             **geometry)
    torch.testing.assert_close(q_d.cpu().float(), q_ref.float(), **tol(dtype))
    torch.testing.assert_close(keys_d.cpu().float(), keys_ref.float(), **tol(dtype))
    torch.testing.assert_close(values_d.cpu().float(), values_ref.float(), **tol(dtype))
    if taps > 1:
        torch.testing.assert_close(state_d.cpu(), state_ref, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [
    dict(q_heads=8, kv_heads=2, head_dim=64, value_dim=64, block_size=16, chunk=24, window=None, sink=True, gate=True),
    dict(q_heads=6, kv_heads=2, head_dim=128, value_dim=128, block_size=32, chunk=33, window=None, sink=True, gate=True),
    dict(q_heads=3, kv_heads=3, head_dim=24, value_dim=40, block_size=4, chunk=7, window=None, sink=True, gate=False),
    dict(q_heads=6, kv_heads=1, head_dim=128, value_dim=16, block_size=8, chunk=None, window=11, sink=False, gate=True),
    dict(q_heads=2, kv_heads=2, head_dim=200, value_dim=130, block_size=16, chunk=1000, window=None, sink=True, gate=False),
])
def test_masked_attention(ops, dtype, sizes):
    g = torch.Generator().manual_seed(9)
    lengths, before = [5, 0, 1, 1, 40], [0, 7, 48, 23, 30]
    geometry = {k: sizes[k] for k in ("q_heads", "kv_heads", "head_dim", "value_dim")}
    cu, _, _ = layout(lengths, [0] * len(lengths))
    ctx, table, keys, values = attention_case(g, dtype, lengths, before, block_size=sizes["block_size"], **geometry)
    tokens = sum(lengths)
    q = rand(g, tokens, sizes["q_heads"] * sizes["head_dim"], dtype=dtype)
    wide = rand(g, tokens, sizes["q_heads"] * sizes["value_dim"] + 5, dtype=dtype)
    sink = rand(g, sizes["q_heads"], scale=2.0) if sizes["sink"] else None
    options = dict(num_seqs=len(lengths), max_q_len=max(lengths), scale=sizes["head_dim"] ** -0.5 * 3.0,
                   window=sizes["window"], chunk=sizes["chunk"], **geometry)
    want = refs.masked_attention(q, keys, values, torch.zeros(tokens, sizes["q_heads"] * sizes["value_dim"], dtype=dtype), cu, ctx,
                                 table, sink=sink, gate=wide[:, 5:] if sizes["gate"] else None, **options)
    q_d, keys_d, values_d, cu_d, ctx_d, table_d, sink_d, wide_d = dev(q, keys, values, cu, ctx, table, sink, wide)
    got = ops.masked_attention(q_d, keys_d, values_d, torch.zeros_like(want, device=DEV), cu_d, ctx_d, table_d, sink=sink_d,
                               gate=wide_d[:, 5:] if sizes["gate"] else None, **options)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("form", ["rwkv", "gla", "mlstm", "plain"])
@pytest.mark.parametrize("heads,key_dim,value_dim", [(5, 32, 32), (2, 48, 80), (3, 20, 50), (1, 128, 16), (2, 200, 24), (3, 64, 40), (2, 136, 9)])
def test_linear_recurrence(ops, dtype, form, heads, key_dim, value_dim):
    g = torch.Generator().manual_seed(10)
    lengths = [5, 0, 1, 37, 2]
    cu, _, slots = layout(lengths, [4, 1, 0, 2, 5])
    tokens = sum(lengths)
    wide = rand(g, tokens, 2 * heads * key_dim + heads * value_dim + 3, dtype=dtype)
    q, k = wide[:, 3:3 + heads * key_dim], wide[:, 3 + heads * key_dim:3 + 2 * heads * key_dim]
    v = wide[:, 3 + 2 * heads * key_dim:]
    ones = form == "mlstm"
    columns = value_dim + (1 if ones else 0)
    state = rand(g, 7, heads, columns, key_dim)
    options = dict(num_seqs=len(lengths), max_q_len=max(lengths), heads=heads, key_dim=key_dim, value_dim=value_dim)
    extra = {}
    if form == "rwkv":
        extra = dict(decay=rand(g, tokens, heads * key_dim), decay_kind="exp_neg_exp", decay_bias=rand(g, heads * key_dim) - 1.0,
                     bonus=rand(g, heads, key_dim))
    elif form == "gla":
        extra = dict(decay=rand(g, tokens, heads * key_dim, scale=2.0), decay_kind="sigmoid_root",
                     decay_bias=rand(g, heads * key_dim), tau=7.0, q_scale=key_dim ** -0.5)
    elif form == "mlstm":
        extra = dict(head_decay=torch.rand(tokens, heads, generator=g), in_scale=torch.rand(tokens, heads, generator=g),
                     q_scale=key_dim ** -0.5, ones_column=True)
    state_ref = state.clone()
    want = refs.linear_recurrence(q, k, v, torch.zeros(tokens, heads, columns), state_ref, cu, slots, **options, **extra)
    wide_d, state_d, cu_d, slots_d = dev(wide, state, cu, slots)
    extra_d = {n: (t.to(DEV) if isinstance(t, torch.Tensor) else t) for n, t in extra.items()}
    got = ops.linear_recurrence(wide_d[:, 3:3 + heads * key_dim], wide_d[:, 3 + heads * key_dim:3 + 2 * heads * key_dim],
                                wide_d[:, 3 + 2 * heads * key_dim:], torch.zeros(tokens, heads, columns, device=DEV), state_d,
                                cu_d, slots_d, **options, **extra_d)
    torch.testing.assert_close(got.cpu(), want, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(state_d.cpu(), state_ref, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("heads", [1, 2, 5])
def test_mlstm_gate_scan(ops, heads):
    g = torch.Generator().manual_seed(11)
    lengths = [5, 0, 1, 150, 64]
    cu, _, slots = layout(lengths, [4, 1, 0, 2, 5])
    tokens = sum(lengths)
    gates = rand(g, tokens, 2 * heads, scale=6.0)
    bias = rand(g, 2 * heads)
    maximum = rand(g, 6, heads, scale=2.0)
    maximum_ref = maximum.clone()
    want = refs.mlstm_gate_scan(gates, bias, 12.0, maximum_ref, cu, slots, torch.zeros(3, tokens, heads), num_seqs=len(lengths), heads=heads)
    gates_d, bias_d, maximum_d, cu_d, slots_d = dev(gates, bias, maximum, cu, slots)
    got = ops.mlstm_gate_scan(gates_d, bias_d, 12.0, maximum_d, cu_d, slots_d, torch.zeros(3, tokens, heads, device=DEV),
                              num_seqs=len(lengths), heads=heads)
    torch.testing.assert_close(got.cpu(), want, atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(maximum_d.cpu(), maximum_ref, atol=1e-5, rtol=1e-5)
