"""Configuration of the Rekezen decoder, from its config.json keys.

config.json names the design under ``architecture`` and gives the vocabulary (``vocab``), the model
width (``width``), the norms' epsilon (``norm.eps``), the number of residual streams of its
hyper-connections (``streams``; absent: one plain residual stream), the hashed table of token
pairs that joins the embedding (``embedding.bigram``: ``buckets``, ``mul_prev``, ``mul_cur``;
absent: none), a factor on the logits (``logit_scale``) and the list ``layers``.  Each layer entry
has a ``type`` (which mixer), the mixer's sizes and constants (``mixer``) and its feed-forward
(``mlp``: a mixture of experts, or null for none).  Every size and constant of a model comes from
here; nothing is pinned to one checkpoint.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from typing import Any, ClassVar

from .model import ConfigError, KeyReader, ModelConfig

MIXER_TYPES = ("attention",)
MLP_KINDS = ("moe",)


def _section(raw: dict, key: str, where: str) -> dict:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{where} needs an object '{key}'")
    return value


def _check_attention(raw: dict, where: str, index: int, layers: list) -> None:
    read = KeyReader(raw)
    heads, kv_heads = read.integer("heads"), read.integer("kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
    dim = read.integer("dim")
    read.integer("vdim")
    read.number("scale")
    if raw.get("softcap") is not None:
        read.number("softcap")
    rot = _section(raw, "rot", where)
    dims = KeyReader(rot).integer("dims", minimum=2)
    KeyReader(rot).number("base")
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}: rot.dims ({dims}) must be even and at most dim ({dim})")
    if rot.get("scaling") is not None:
        scaling = KeyReader(_section(rot, "scaling", where))
        for key in ("factor", "original", "fast", "slow"):
            scaling.number(key)
    source = raw.get("kv_from")
    if source is not None:
        if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < index:
            raise ConfigError(f"{where}: kv_from must name an earlier layer, got {source!r}")
        other = layers[source].get("mixer") if isinstance(layers[source], dict) else None
        if not isinstance(other, dict) or other.get("kv_from") is not None:
            raise ConfigError(f"{where}: layer {source} has no keys and values of its own to borrow")
        for key in ("kv_heads", "dim", "vdim"):
            if other.get(key) != raw.get(key):
                raise ConfigError(f"{where}: '{key}' differs from layer {source}, whose keys and values it reads")


def _check_expert(raw: dict, where: str) -> None:
    read = KeyReader(raw)
    read.integer("ff")
    read.number("limit")


def _check_mlp(mlp: Any, where: str) -> None:
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
        raise ConfigError(f"{where}: mlp must be null or of kind {' / '.join(MLP_KINDS)}")
    _check_expert(_section(mlp, "expert", where), f"{where}.expert")
    router = KeyReader(_section(mlp, "router", where))
    experts, top = router.integer("experts"), router.integer("top")
    if top > experts:
        raise ConfigError(f"{where}: router.top ({top}) exceeds router.experts ({experts})")
    if mlp.get("shared") is not None:
        _check_expert(_section(mlp, "shared", where), f"{where}.shared")


@dataclass(frozen=True)
class RekezenConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    layers_json: str                  # the list ``layers`` as JSON text (a frozen, hashable form)
    streams: int | None = None        # residual streams of the hyper-connections; None: a plain residual
    bigram_json: str = "null"         # the pair table's constants, or null
    logit_scale: float = 1.0
    eos_token_id: int | None = None

    architecture: ClassVar[str] = "Rekezen"

    @property
    def layers(self) -> list[dict]:
        return json.loads(self.layers_json)

    @property
    def bigram(self) -> dict | None:
        return json.loads(self.bigram_json)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "RekezenConfig":
        read = KeyReader(raw)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json must list the model's layers under 'layers'")
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"{where} must be an object")
            if layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"{where}: unknown mixer type {layer.get('type')!r} (known: {', '.join(MIXER_TYPES)})")
            _check_attention(_section(layer, "mixer", where), f"{where}.mixer", index, layers)
            _check_mlp(layer.get("mlp"), f"{where}.mlp")
        bigram = (raw.get("embedding") or {}).get("bigram") if isinstance(raw.get("embedding"), dict) else None
        if bigram is not None:
            pair = KeyReader(bigram if isinstance(bigram, dict) else {})
            bigram = {"buckets": pair.integer("buckets"), "mul_prev": pair.integer("mul_prev", minimum=0),
                      "mul_cur": pair.integer("mul_cur", minimum=0)}
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer, got {eos!r}")
        return cls(vocab=read.integer("vocab"), width=read.integer("width"),
                   norm_eps=KeyReader(_section(raw, "norm", "config.json")).number("eps"),
                   layers_json=json.dumps(layers, sort_keys=True),
                   streams=read.integer("streams", required=False),
                   bigram_json=json.dumps(bigram, sort_keys=True),
                   logit_scale=read.number("logit_scale", 1.0), eos_token_id=eos)

    def to_dict(self) -> dict[str, Any]:
        data = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "layers": self.layers, "logit_scale": self.logit_scale}
        if self.streams is not None:
            data["streams"] = self.streams
        if self.bigram is not None:
            data["embedding"] = {"bigram": self.bigram}
        if self.eos_token_id is not None:
            data["eos_token_id"] = self.eos_token_id
        return data
