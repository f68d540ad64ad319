"""Configuration of the Mazanex decoder, from its config.json keys.

config.json names the design under ``architecture`` and gives the vocabulary (``vocab``), the
model width (``width``), the norms' epsilon (``norm.eps``) and the list ``layers``.  Each layer
entry has a ``type`` (which mixer), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``: ``{"kind": "dense", "ff": N}``, or null for none).  Every size and
constant of a model comes from here; nothing is pinned to one checkpoint.
"""

from __future__ import annotations

import dataclasses
import json
from dataclasses import dataclass
from typing import Any, ClassVar

from .model import ConfigError, KeyReader, ModelConfig

MIXER_TYPES = ("parallel", "gla", "mlstm")


def _section(raw: dict, key: str, where: str) -> dict:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{where} needs an object '{key}'")
    return value


def _check_attention(raw: dict, where: str) -> None:
    read = KeyReader(raw)
    heads, kv_heads = read.integer("heads"), read.integer("kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
    dim = read.integer("dim")
    read.integer("vdim")
    read.integer("conv")
    read.number("scale")
    KeyReader(_section(raw, "mask", where)).integer("size")
    rot = KeyReader(_section(raw, "rot", where))
    dims = rot.integer("dims", minimum=2)
    rot.number("base")
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}: rot.dims ({dims}) must be even and at most dim ({dim})")


def _check_layer(index: int, layer: Any) -> None:
    where = f"layers[{index}]"
    if not isinstance(layer, dict):
        raise ConfigError(f"{where} must be an object")
    kind = layer.get("type")
    if kind not in MIXER_TYPES:
        raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXER_TYPES)})")
    mixer = _section(layer, "mixer", where)
    if kind == "parallel":
        _check_attention(_section(mixer, "left", where), f"{where}.mixer.left")
        right = KeyReader(_section(mixer, "right", where))
        right.integer("heads")
        right.integer("dim")
    else:
        read = KeyReader(mixer)
        read.integer("heads")
        read.integer("dim")
        read.integer("vdim")
        read.number("tau" if kind == "gla" else "gate_cap")
    mlp = layer.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
            raise ConfigError(f"{where}: mlp must be null or of kind 'dense'")
        KeyReader(mlp).integer("ff")


@dataclass(frozen=True)
class MazanexConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    layers_json: str            # the list ``layers`` as JSON text (a frozen, hashable form)
    eos_token_id: int | None = None
    tensor_shapes_json: str = "{}"   # shapes of the checkpoint's tensors, where one is at hand

    architecture: ClassVar[str] = "Mazanex"

    @property
    def layers(self) -> list[dict]:
        return json.loads(self.layers_json)

    def with_tensor_shapes(self, shapes: dict[str, tuple[int, ...]]) -> "MazanexConfig":
        """The configuration with the sizes that only the tensors' shapes give (the ranks of the
        low-rank decay projections)."""
        return dataclasses.replace(self, tensor_shapes_json=json.dumps({n: list(s) for n, s in sorted(shapes.items())}))

    def tensor_shape(self, name: str) -> tuple[int, ...] | None:
        shape = json.loads(self.tensor_shapes_json).get(name)
        return None if shape is None else tuple(shape)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "MazanexConfig":
        read = KeyReader(raw)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json must list the model's layers under 'layers'")
        for index, layer in enumerate(layers):
            _check_layer(index, layer)
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer, got {eos!r}")
        return cls(vocab=read.integer("vocab"), width=read.integer("width"),
                   norm_eps=KeyReader(_section(raw, "norm", "config.json")).number("eps"),
                   layers_json=json.dumps(layers, sort_keys=True), eos_token_id=eos)

    def to_dict(self) -> dict[str, Any]:
        data = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "layers": self.layers}
        if self.eos_token_id is not None:
            data["eos_token_id"] = self.eos_token_id
        return data
