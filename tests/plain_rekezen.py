"""A plain, slow implementation of the Rekezen decoder: one function per mechanism, whole
sequences at once, in float64 unless told otherwise.  It shares no code with the package: the
tests compare the engine with this.

Notation: T tokens, W model width, S residual streams; ``w`` maps a tensor's checkpoint name to
the tensor; ``cfg`` is the parsed config.json.
"""

from __future__ import annotations

import math

import torch

DTYPE = torch.float64


def layer_norm(x, weight, bias, eps):
    mean = x.mean(-1, keepdim=True)
    centred = x - mean
    variance = (centred * centred).mean(-1, keepdim=True)
    return centred / torch.sqrt(variance + eps) * weight + bias


def rms_over_all(x, weight, eps):
    """x [T, N]: every row divided by the root mean square over all N entries, times a weight [N]."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """The row of the pair table for every token of one sequence: the first token takes the last
    row (number ``buckets``), the others (prev * mul_prev + cur * mul_cur) mod buckets."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((int(prev) * mul_prev + int(cur) * mul_cur) % buckets)
    return torch.tensor(rows, dtype=torch.long)


def embed(tokens, w, cfg):
    x = w["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    pair = (cfg.get("embedding") or {}).get("bigram")
    if pair:
        x = x + w["bigram"][bigram_rows(list(tokens), pair["buckets"], pair["mul_prev"], pair["mul_cur"])]
    return x


def rotary_table(rot, dtype=DTYPE):
    """(frequencies [dims/2], magnitude): base^(-2i/dims), under a YaRN scaling blended with the
    frequency divided by the factor along a ramp over the pair index, and one factor on cos and sin."""
    dims, base = rot["dims"], float(rot["base"])
    half = dims // 2
    freq = [base ** (-2.0 * i / dims) for i in range(half)]
    scaling = rot.get("scaling")
    magnitude = 1.0
    if scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def turning_dim(turns):
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(turning_dim(float(scaling["fast"]))), 0)
        hi = min(math.ceil(turning_dim(float(scaling["slow"]))), dims - 1)
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            freq[i] = freq[i] / factor * ramp + freq[i] * (1.0 - ramp)
        magnitude = 0.1 * math.log(factor) + 1.0
    return torch.tensor(freq, dtype=dtype), magnitude


def rotate(x, positions, rot):
    """x [T, heads, D]: dim i < dims/2 pairs with dim i + dims/2; the rest is left alone."""
    dims = rot["dims"]
    half = dims // 2
    freq, magnitude = rotary_table(rot, x.dtype)
    angle = positions.to(x.dtype)[:, None] * freq[None, :]
    cos, sin = (torch.cos(angle) * magnitude)[:, None, :], (torch.sin(angle) * magnitude)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = a * cos - b * sin
    out[..., half:dims] = b * cos + a * sin
    return out


def keys_and_values(h, w, prefix, m, eps, positions):
    """What a layer with projections of its own puts into its cache: keys after norm and rotation, values."""
    T = h.shape[0]
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    k = rms_over_all(h @ w[f"{prefix}.k"].T, w[f"{prefix}.k.norm"], eps).reshape(T, G, D)
    k = rotate(k, positions, m["rot"])
    v = (h @ w[f"{prefix}.v"].T).reshape(T, G, Dv)
    return k, v


def capped_causal_attention(q, k, v, *, scale, softcap):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; scores scaled, then bounded by cap * tanh(s / cap)."""
    T, H, _ = q.shape
    G = k.shape[1]
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention(h, w, prefix, m, eps, positions, kv):
    """``kv``: this layer's (keys, values), its own or those of the layer it borrows from."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    q = rms_over_all(h @ w[f"{prefix}.q"].T, w[f"{prefix}.q.norm"], eps).reshape(T, H, D)
    q = rotate(q, positions, m["rot"])
    k, v = kv
    o = capped_causal_attention(q, k, v, scale=m["scale"], softcap=m.get("softcap"))
    gate = torch.sigmoid(h @ w[f"{prefix}.g"].T)            # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, -1) @ w[f"{prefix}.o"].T


def expert(h, w, prefix, limit):
    g = torch.clamp(h @ w[f"{prefix}.gate"].T, max=limit)
    u = torch.clamp(h @ w[f"{prefix}.up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[f"{prefix}.down"].T


def routing(h, w, prefix, top, margins=None):
    """(chosen experts [T, top], their weights [T, top]): the largest logits, softmax over them alone.
    ``margins`` (a list) receives, per token, how far the last chosen logit lies above the first one
    left out, as a fraction of the largest magnitude among the token's logits."""
    z = h @ w[f"{prefix}.router"].T + w[f"{prefix}.router.b"]
    best = torch.topk(z, top, dim=-1)
    if margins is not None:
        ordered = torch.sort(z, dim=-1, descending=True).values
        gap = ordered[:, top - 1] - ordered[:, top] if top < z.shape[1] else torch.full_like(ordered[:, 0], math.inf)
        margins.append(gap / z.abs().max(-1).values)
    return best.indices, torch.softmax(best.values, dim=-1)


def mixture(h, w, prefix, mlp, margins=None):
    chosen, weights = routing(h, w, prefix, mlp["router"]["top"], margins)
    out = torch.zeros(h.shape[0], w[f"{prefix}.e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, weight in zip(chosen[t].tolist(), weights[t]):
            out[t] += weight * expert(h[t:t + 1], w, f"{prefix}.e{e}", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + expert(h, w, f"{prefix}.shared", mlp["shared"]["limit"])
    return out


def hyper_sublayer(streams, w, prefix, sublayer):
    """streams [S, T, W]: the sublayer reads a weighted sum of the streams; every new stream is a
    mixture of the old ones (matrix indexed [from, to]) plus its share of the sublayer's output."""
    u = torch.einsum("s,stw->tw", w[f"{prefix}.in"], streams)
    y = sublayer(u)
    return torch.einsum("sr,stw->rtw", w[f"{prefix}.mix"], streams) + w[f"{prefix}.out"][:, None, None] * y[None]


def forward(tokens, w, cfg, dtype=DTYPE, trace=None, margins=None):
    """Logits [T, vocab] of one sequence from its first token.  ``trace`` (a list) receives the
    stream (the sum of the streams) after every layer, ``margins`` every router's margins."""
    w = {name: t.to(dtype) if t.is_floating_point() else t for name, t in w.items()}
    eps = cfg["norm"]["eps"]
    x = embed(tokens, w, cfg)
    T = x.shape[0]
    positions = torch.arange(T)
    count = cfg.get("streams")
    streams = x[None].repeat(count, 1, 1) if count else None
    cached = {}
    for index, layer in enumerate(cfg["layers"]):
        p, m = f"l{index}", layer["mixer"]

        def mixer(u):
            h = layer_norm(u, w[f"{p}.norm1"], w[f"{p}.norm1.b"], eps)
            source = m.get("kv_from")
            if source is None:
                cached[index] = keys_and_values(h, w, f"{p}.mix", m, eps, positions)
                source = index
            return attention(h, w, f"{p}.mix", m, eps, positions, cached[source])

        def feed_forward(u):
            return mixture(layer_norm(u, w[f"{p}.norm2"], w[f"{p}.norm2.b"], eps), w, f"{p}.mlp", layer["mlp"], margins)

        if streams is None:
            x = x + mixer(x)
            if layer.get("mlp"):
                x = x + feed_forward(x)
        else:
            streams = hyper_sublayer(streams, w, f"{p}.hc1", mixer)
            if layer.get("mlp"):
                streams = hyper_sublayer(streams, w, f"{p}.hc2", feed_forward)
        if trace is not None:
            trace.append(x.clone() if streams is None else streams.sum(0))
    if streams is not None:
        x = streams.sum(0)
    z = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return (z @ w["embed"].T) * cfg.get("logit_scale", 1.0)
