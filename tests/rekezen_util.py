"""Small Rekezen configurations for the tests (config.json form), model folders with random
weights, and the plain implementation's logits for them."""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import load_file

import plain_rekezen as plain


def attention(heads, kv_heads, dim, vdim, rot_dims, *, base=10000.0, scale=0.25, softcap=15.0, scaling=None, kv_from=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
             "rot": {"dims": rot_dims, "base": base}}
    if softcap is not None:
        mixer["softcap"] = softcap
    if scaling is not None:
        mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return mixer


def moe(experts, top, ff, limit, shared=None):
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared is not None:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


def layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def config(vocab, width, layers, *, streams=None, bigram=None, eps=1e-6, logit_scale=1.0):
    raw = {"architecture": "Rekezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
           "logit_scale": logit_scale}
    if streams is not None:
        raw["streams"] = streams
    if bigram is not None:
        raw["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}
    return raw


YARN = (8.0, 64, 16.0, 2.0)
# three streams; a borrowed cache two layers back; values wider than keys; a layer without a feed-forward;
# no shared expert in one layer; one chosen expert in another
SMALL_A = config(96, 48, [
    layer(attention(4, 2, 16, 24, 8, scaling=YARN), moe(5, 2, 20, 1.5, shared=(28, 2.5))),
    layer(attention(6, 3, 8, 8, 8, base=500.0, softcap=None), None),
    layer(attention(4, 2, 16, 24, 6, scale=0.4, kv_from=0, scaling=YARN), moe(3, 1, 36, 3.0)),
], streams=3, bigram=(53, 7, 11), logit_scale=0.7)
# one stream of hyper-connections; a group of one; the whole head rotated; every expert chosen
SMALL_B = config(130, 40, [
    layer(attention(2, 2, 12, 20, 12, base=200.0, scale=0.5, softcap=4.0), moe(2, 2, 24, 2.0, shared=(16, 1.0))),
    layer(attention(2, 2, 12, 20, 12, base=200.0, scale=0.3, softcap=30.0, kv_from=0), moe(4, 3, 12, 0.75)),
], streams=1, bigram=(31, 3, 0), eps=1e-5)
# no hyper-connections and no pair table: a plain residual stream
SMALL_C = config(64, 32, [
    layer(attention(2, 1, 16, 16, 4, scaling=(2.0, 32, 8.0, 1.0)), moe(4, 2, 16, 2.0, shared=(8, 2.0))),
    layer(attention(4, 1, 8, 8, 2), None),
])
# sizes that the matrix-core attention and the grouped products' full tiles take on the GPU
MEDIUM = config(320, 256, [
    layer(attention(4, 2, 128, 128, 64, scaling=YARN), moe(6, 2, 96, 2.0, shared=(64, 2.0))),
    layer(attention(4, 2, 128, 128, 64, kv_from=0, scaling=YARN), moe(6, 2, 96, 2.0)),
    layer(attention(8, 2, 64, 64, 32, softcap=25.0), moe(3, 1, 160, 4.0, shared=(128, 1.0))),
], streams=4, bigram=(211, 13, 29), logit_scale=0.5)
CONFIGS = {"A": SMALL_A, "B": SMALL_B, "C": SMALL_C}
BLOCK_SIZE = {"A": 4, "B": 8, "C": 2}


def write_model(raw: dict, seed: int, folder) -> Path:
    from forge_engine_amd.config import load_model_config
    from forge_engine_amd.weights import write_random_model

    return write_random_model(load_model_config(raw), seed, folder)


def folder_weights(folder) -> tuple[dict, dict]:
    folder = Path(folder)
    return json.loads((folder / "config.json").read_text()), load_file(str(folder / "model.safetensors"))


SAFE_MARGIN = 0.05


def plain_logits(folder, requests, only=None) -> dict:
    """(request, position) -> logits of the plain implementation, for whole requests.  The result's
    ``decided`` holds the rows whose routing is beyond doubt: in no layer does the token, or any token
    before it in its request, choose its experts by a margin that the roundings of bfloat16 could turn."""
    cfg, weights = folder_weights(folder)
    want = Rows()
    for request_id, tokens in requests.items():
        if only is not None and request_id not in only:
            continue
        margins = []
        logits = plain.forward(tokens, weights, cfg, margins=margins)
        narrow = torch.stack(margins).min(0).values < SAFE_MARGIN if margins else torch.zeros(len(tokens), dtype=torch.bool)
        doubtful = torch.cumsum(narrow.to(torch.int64), 0) > 0
        for position in range(len(tokens)):
            want[(request_id, position)] = logits[position]
            if not bool(doubtful[position]):
                want.decided.add((request_id, position))
    return want


class Rows(dict):
    def __init__(self):
        super().__init__()
        self.decided = set()


def compare(got: dict, want: Rows, dtype: str, fraction: float = 0.06, float32_factor: float = 1.0) -> float:
    """Every row the engine wrote against the plain implementation's.  float32: to 1e-5 + 1e-4 of the row's largest logit
    (times ``float32_factor`` for models made so that roundings are amplified).
    bfloat16: a row whose routing is beyond doubt to a fraction of the logits' spread; of all rows,
    four in five (a token that chooses another expert than the plain implementation, by a margin
    within bfloat16's rounding, moves its own logits and, through its keys and values, later ones)."""
    assert got, "no logits were written"
    worst, near, checked = 0.0, 0, 0
    for key, row in got.items():
        expected = want[key].to(torch.float64)
        assert bool(torch.isfinite(row).all()), f"{key}: non-finite logits"
        diff = (row.to(torch.float64) - expected).abs()
        if dtype == "float32":
            bound = float32_factor * (1e-5 + 1e-4 * float(expected.abs().max()))
            assert float(diff.max()) <= bound, f"{key}: off by {float(diff.max()):.3e}"
            worst = max(worst, float(diff.max()))
            continue
        spread = float(expected.max() - expected.min())
        within = float(diff.max()) <= fraction * spread
        near += within
        if key in want.decided:
            checked += 1
            assert within, f"{key}: off by {float(diff.max()):.3e} of a spread of {spread:.3e}"
            worst = max(worst, float(diff.max()) / spread)
    if dtype != "float32":
        assert near >= 0.8 * len(got), f"only {near} of {len(got)} rows are near the plain implementation's"
    return worst
