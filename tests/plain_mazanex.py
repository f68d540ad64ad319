"""A plain, slow implementation of the Mazanex decoder: one function per mechanism, whole
sequences at once or token by token in Python loops, in float64 unless told otherwise.  It shares
no code with the package: the tests compare the engine with this.

Notation: T tokens, W model width; ``p`` is a dict of the layer's tensors by the name they carry
in the checkpoint behind the layer's prefix.
"""

from __future__ import annotations

import math

import torch

DTYPE = torch.float64


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def previous_rows(h):
    """Row t holds h[t-1]; zeros for the first token."""
    out = torch.zeros_like(h)
    out[1:] = h[:-1]
    return out


def token_shift(h, weight):
    return h + (previous_rows(h) - h) * weight


def short_convolution(u, taps_weight):
    """u [T, C], taps_weight [C, K]: y_t = sum_j w[:, j] * u_(t - K + 1 + j), zeros before the start."""
    T, C = u.shape
    K = taps_weight.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=u.dtype), u])
    y = torch.zeros_like(u)
    for j in range(K):
        y += padded[j:j + T] * taps_weight[:, j]
    return y


def rotate_half_pairs(x, positions, base, dims):
    """x [T, heads, D]: dims i and i + dims/2 (i < dims/2) turn by the angle p * base^(-2i/dims)."""
    half = dims // 2
    freq = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = positions.to(x.dtype)[:, None] * freq[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = a * cos - b * sin
    out[..., half:dims] = b * cos + a * sin
    return out


def chunked_sink_attention(q, k, v, positions, *, scale, chunk, sink):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; token i sees j <= i of its own chunk of ``chunk``
    positions; every head's softmax has one more term exp(sink_h) without a value."""
    T, H, D = q.shape
    G = k.shape[1]
    pos = positions.to(torch.long)
    seen = (pos[None, :] <= pos[:, None]) & ((pos[None, :] // chunk) == (pos[:, None] // chunk))   # [i, j]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        top = torch.maximum(s.max(-1, keepdim=True).values, sink[h])
        e = torch.exp(s - top)
        denom = e.sum(-1, keepdim=True) + torch.exp(sink[h] - top)
        out[:, h] = (e / denom) @ v[:, g]
    return out


def left_attention(h, p, cfg, eps, positions):
    H, G, D, Dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = h @ p["q"].T + p["q.b"]
    k = h @ p["k"].T + p["k.b"]
    v = h @ p["v"].T + p["v.b"]
    q = short_convolution(q, p["q.conv"]).view(T, H, D)
    k = short_convolution(k, p["k.conv"]).view(T, G, D)
    v = short_convolution(v, p["v.conv"]).view(T, G, Dv)
    rot = cfg["rot"]
    q = unit_rms(rotate_half_pairs(q, positions, rot["base"], rot["dims"]), eps)
    k = unit_rms(rotate_half_pairs(k, positions, rot["base"], rot["dims"]), eps)
    o = chunked_sink_attention(q, k, v, positions, scale=cfg["scale"], chunk=cfg["mask"]["size"], sink=p["sink"])
    o = o.reshape(T, H * Dv) * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T + p["o.b"]


def rwkv_time_mix(h, p, cfg, eps):
    H, D = cfg["heads"], cfg["dim"]
    T = h.shape[0]
    delta = previous_rows(h) - h
    mixed = {s: h + delta * p[f"mu.{s}"] for s in "rkvgw"}
    r = (mixed["r"] @ p["r"].T).view(T, H, D)
    k = (mixed["k"] @ p["k"].T).view(T, H, D)
    v = (mixed["v"] @ p["v"].T).view(T, H, D)
    gate = torch.nn.functional.silu(mixed["g"] @ p["g"].T)
    w = torch.exp(-torch.exp(torch.tanh(mixed["w"] @ p["w1"].T) @ p["w2"].T + p["w0"])).view(T, H, D)
    u = p["u"]
    S = torch.zeros(H, D, D, dtype=h.dtype)
    o = torch.zeros(T, H, D, dtype=h.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, r[t])
        S = w[t][:, :, None] * S + kv
    o = unit_rms(o, eps).reshape(T, H * D) * p["norm"] * gate
    return o @ p["o"].T


def parallel_mixer(h, p, cfg, eps, positions):
    left = left_attention(h, {n[5:]: t for n, t in p.items() if n.startswith("left.")}, cfg["left"], eps, positions)
    right = rwkv_time_mix(h, {n[6:]: t for n, t in p.items() if n.startswith("right.")}, cfg["right"], eps)
    return 0.5 * (unit_rms(left, eps) * p["left.out"] + unit_rms(right, eps) * p["right.out"])


def gla_mixer(h, p, cfg, eps):
    H, D, Dv = cfg["heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ p["k"].T).view(T, H, D)
    v = (h @ p["v"].T).view(T, H, Dv)
    z = (h @ p["a1"].T) @ p["a2"].T + p["a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / cfg["tau"])).view(T, H, D)
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = (unit_rms(o, eps) * p["norm"]).reshape(T, H * Dv) * torch.nn.functional.silu(h @ p["g"].T)
    return o @ p["o"].T


def mlstm_mixer(h, p, cfg, eps):
    H, D, Dv, cap = cfg["heads"], cfg["dim"], cfg["vdim"], cfg["gate_cap"]
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ p["k"].T).view(T, H, D)
    v = (h @ p["v"].T).view(T, H, Dv)
    gi = cap * torch.tanh((h @ p["i"].T + p["i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ p["f"].T + p["f.b"]) / cap))
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    n = torch.zeros(H, D, dtype=h.dtype)
    m = torch.zeros(H, dtype=h.dtype)
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(gf[t] + m, gi[t])
        keep = torch.exp(gf[t] + m - m_new)
        take = torch.exp(gi[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        denom = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        o[t] = torch.einsum("hkv,hk->hv", S, q[t]) / denom[:, None]
    o = unit_rms(o, eps).reshape(T, H * Dv) * p["norm"] * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T


def polynorm_feed_forward(x, p, eps):
    z = x @ p["up"].T
    a, b, c, e = p["act"]
    act = a * unit_rms(z, eps) + b * unit_rms(z ** 2, eps) + c * unit_rms(z ** 3, eps) + e
    return act @ p["down"].T


def layer_tensors(weights, index, part):
    prefix = f"l{index}.{part}."
    return {n[len(prefix):]: t for n, t in weights.items() if n.startswith(prefix)}


def forward(config, weights, tokens, dtype=DTYPE, layers_out=None):
    """Logits [T, vocab] of one whole sequence from position 0; ``layers_out`` (a list) receives
    the stream after every layer."""
    w = {n: t.to(dtype) for n, t in weights.items()}
    eps = config["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(ids))
    x = w["embed"][ids]
    for i, layer in enumerate(config["layers"]):
        h = token_shift(x, w[f"l{i}.shift"])
        p = layer_tensors(w, i, "mix")
        kind = layer["type"]
        if kind == "parallel":
            m = parallel_mixer(h, p, layer["mixer"], eps, positions)
        elif kind == "gla":
            m = gla_mixer(h, p, layer["mixer"], eps)
        elif kind == "mlstm":
            m = mlstm_mixer(h, p, layer["mixer"], eps)
        else:
            raise ValueError(kind)
        x = x + unit_rms(m, eps) * w[f"l{i}.norm1"]
        if layer.get("mlp") is not None:
            f = polynorm_feed_forward(x, layer_tensors(w, i, "mlp"), eps)
            x = x + unit_rms(f, eps) * w[f"l{i}.norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    z = unit_rms(x, eps) * w["final.norm"]
    return z @ w["head"].T
