"""Mazanex as a plan over the generic parts.

Token embedding ``embed``; layers ``l<i>`` in the order config.json lists them, each an
output-norm arrangement with token shift (``l<i>.shift``, norms ``l<i>.norm1`` / ``l<i>.norm2``)
around one of three mixers under ``l<i>.mix`` and a PolyNorm feed-forward under ``l<i>.mlp`` (or
none); final RMSNorm ``final.norm``; head ``head``.

Mixers by layer type: ``parallel`` puts chunked attention with a sink, short convolutions, an
output gate and unit-norm q/k after a partial rotation (``.left``) beside RWKV time mixing
(``.right``), each normalised with its own weight (``.left.out`` / ``.right.out``) and averaged;
``gla`` is gated linear attention; ``mlstm`` the matrix memory of xLSTM.  Low-rank sizes of the
decays are not in config.json: they are the shapes of the tensors, which the loader checks, so
the plan takes them from ``tensor_shapes`` when the checkpoint is at hand and from a default
otherwise (random weights).
"""

from __future__ import annotations

from ..config.mazanex import MazanexConfig
from ..parts.plan import LayerCall, LayerSpec, ModelPlan, PartSpec
from ..registry import register_architecture

DEFAULT_DECAY_RANK = 16

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                   "o_bias": "o.b", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "sink": "sink",
                   "gate": "g"}


def _rank(config: MazanexConfig, tensor: str, sizes: dict) -> int:
    """The inner size of a low-rank decay projection: the tensor's shape, else an optional
    ``rank`` among the mixer's sizes, else the default."""
    shape = config.tensor_shape(tensor)
    if shape is not None:
        return int(shape[0])
    return int(sizes.get("rank", DEFAULT_DECAY_RANK))


def _mixer(config: MazanexConfig, kind: str, sizes: dict, prefix: str) -> PartSpec:
    width, eps = config.width, config.norm_eps
    if kind == "parallel":
        left, right = sizes["left"], sizes["right"]
        attention = PartSpec("gqa_attention", {
            "hidden_size": width, "num_heads": left["heads"], "num_kv_heads": left["kv_heads"],
            "head_dim": left["dim"], "value_dim": left["vdim"], "bias": True, "scale": left["scale"],
            "conv_taps": left["conv"], "unit_norm_eps": eps, "chunk": left["mask"]["size"], "sink": True,
            "output_gate": True, "names": ATTENTION_NAMES,
            "position": PartSpec("rotary", {"head_dim": left["dim"], "theta": left["rot"]["base"],
                                            "rotary_dim": left["rot"]["dims"]}),
        }, f"{prefix}.left")
        time_mix = PartSpec("rwkv_time_mix", {
            "hidden_size": width, "heads": right["heads"], "dim": right["dim"], "eps": eps,
            "decay_rank": _rank(config, f"{prefix}.right.w1", right),
        }, f"{prefix}.right")
        return PartSpec("parallel_mixers", {"hidden_size": width, "eps": eps,
                                            "branches": {"left": attention, "right": time_mix}}, prefix)
    if kind == "gla":
        return PartSpec("gated_linear_attention", {
            "hidden_size": width, "heads": sizes["heads"], "dim": sizes["dim"], "value_dim": sizes["vdim"],
            "eps": eps, "tau": sizes["tau"], "decay_rank": _rank(config, f"{prefix}.a1", sizes),
        }, prefix)
    if kind == "mlstm":
        return PartSpec("mlstm", {
            "hidden_size": width, "heads": sizes["heads"], "dim": sizes["dim"], "value_dim": sizes["vdim"],
            "eps": eps, "gate_cap": sizes["gate_cap"],
        }, prefix)
    raise ValueError(f"unknown mixer type '{kind}'")


def mazanex_plan(config: MazanexConfig) -> ModelPlan:
    width, eps = config.width, config.norm_eps
    layers = []
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        mlp = layer.get("mlp")
        feed_forward = None if mlp is None else PartSpec("polynorm_mlp", {
            "hidden_size": width, "intermediate_size": mlp["ff"], "eps": eps}, f"{prefix}.mlp")
        norms = {"mixer_out": PartSpec("rms_norm_of_update", {"size": width, "eps": eps, "leaf": ""}, f"{prefix}.norm1")}
        if mlp is not None:
            norms["ff_out"] = PartSpec("rms_norm_of_update", {"size": width, "eps": eps, "leaf": ""}, f"{prefix}.norm2")
        layers.append(LayerSpec("output_norm", _mixer(config, layer["type"], layer["mixer"], f"{prefix}.mix"),
                                feed_forward, norms, {"hidden_size": width, "token_shift": True}, prefix))
    sizes = {"vocab_size": config.vocab, "hidden_size": width, "leaf": ""}
    return ModelPlan(
        hidden_size=width,
        vocab_size=config.vocab,
        embedding=PartSpec("token_embedding", dict(sizes), "embed"),
        layers=tuple(layers),
        schedule=tuple(LayerCall(index) for index in range(len(layers))),
        final_norm=PartSpec("rms_norm", {"size": width, "eps": eps, "leaf": ""}, "final.norm"),
        head=PartSpec("lm_head", dict(sizes), "head"),
        eos_token_ids=frozenset() if config.eos_token_id is None else frozenset({config.eos_token_id}),
        max_positions=None,
    )


register_architecture(MazanexConfig.architecture, MazanexConfig, mazanex_plan)
