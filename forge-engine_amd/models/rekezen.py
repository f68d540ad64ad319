"""Rekezen as a plan over the generic parts.

Embedding ``embed`` plus a hashed table of token pairs ``bigram``; layers ``l<i>`` in the order
config.json lists them, each a pre-norm arrangement over several residual streams
(hyper-connections, ``l<i>.hc1.*`` / ``l<i>.hc2.*``; one plain stream if config.json names no
``streams``) with layer norms ``l<i>.norm1`` / ``l<i>.norm2`` (bias: the same name with ``.b``),
a grouped-query attention mixer under ``l<i>.mix`` and a mixture of experts under ``l<i>.mlp`` (or
no feed-forward); final layer norm ``final.norm``; the head is the embedding table, its logits
times ``logit_scale``.

The attention normalises q and k over the whole projection, rotates the first ``rot.dims`` dims of
every head (frequencies stretched by ``rot.scaling`` if given), bounds its scores by a soft cap and
gates every head's output by one number.  A layer whose mixer names ``kv_from`` has no keys and
values of its own: its call in the schedule reads the cache slot of the layer it names.
"""

from __future__ import annotations

from ..config.rekezen import RekezenConfig
from ..parts.plan import LayerCall, LayerSpec, ModelPlan, PartSpec
from ..registry import register_architecture

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "gate": "g"}
EXPERT_NAMES = {"expert": "e{e}", "shared": "shared", "router": "router", "router_bias": "router.b",
                "gate": "gate", "up": "up", "down": "down"}


def _position(sizes: dict) -> PartSpec:
    rot = sizes["rot"]
    params = {"head_dim": sizes["dim"], "theta": rot["base"], "rotary_dim": rot["dims"]}
    scaling = rot.get("scaling")
    if scaling is None:
        return PartSpec("rotary", dict(params, precise=True))
    return PartSpec("yarn_rotary", dict(params, factor=scaling["factor"], original=scaling["original"],
                                        fast=scaling["fast"], slow=scaling["slow"]))


def _attention(config: RekezenConfig, sizes: dict, prefix: str) -> PartSpec:
    return PartSpec("gqa_attention", {
        "hidden_size": config.width, "num_heads": sizes["heads"], "num_kv_heads": sizes["kv_heads"],
        "head_dim": sizes["dim"], "value_dim": sizes["vdim"], "scale": sizes["scale"],
        "softcap": sizes.get("softcap"), "whole_norm_eps": config.norm_eps, "head_gate": True,
        "own_kv": sizes.get("kv_from") is None, "names": ATTENTION_NAMES, "position": _position(sizes),
    }, prefix)


def _feed_forward(config: RekezenConfig, mlp: dict | None, prefix: str) -> PartSpec | None:
    if mlp is None:
        return None
    shared = mlp.get("shared")
    return PartSpec("routed_experts", {
        "hidden_size": config.width, "experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
        "intermediate_size": mlp["expert"]["ff"], "limit": mlp["expert"]["limit"],
        "shared_size": None if shared is None else shared["ff"],
        "shared_limit": None if shared is None else shared["limit"], "names": EXPERT_NAMES,
    }, prefix)


def rekezen_plan(config: RekezenConfig) -> ModelPlan:
    width, eps = config.width, config.norm_eps

    def norm(name: str) -> PartSpec:
        return PartSpec("layer_norm", {"size": width, "eps": eps, "leaf": "", "bias_leaf": "b"}, name)

    layers, schedule, unread = [], [], set()
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        feed_forward = _feed_forward(config, layer.get("mlp"), f"{prefix}.mlp")
        norms = {"input": norm(f"{prefix}.norm1")}
        if feed_forward is not None:
            norms["post_mixer"] = norm(f"{prefix}.norm2")
        else:       # a checkpoint may still hold what a feed-forward's sublayer would have read
            unread |= {f"{prefix}.norm2", f"{prefix}.norm2.b", f"{prefix}.hc2.in", f"{prefix}.hc2.out", f"{prefix}.hc2.mix"}
        if config.streams is None:
            arrangement, params = "pre_norm", {}
        else:
            arrangement, params = "hyper_connections", {"streams": config.streams}
        layers.append(LayerSpec(arrangement, _attention(config, layer["mixer"], f"{prefix}.mix"), feed_forward, norms,
                                params, prefix if params else ""))
        source = layer["mixer"].get("kv_from")
        schedule.append(LayerCall(index) if source is None else LayerCall(index, cache=source, writes_cache=False))
    sizes = {"vocab_size": config.vocab, "hidden_size": width, "leaf": ""}
    pair = config.bigram
    if pair is None:
        embedding = PartSpec("token_embedding", dict(sizes), "embed")
    else:
        embedding = PartSpec("token_pair_embedding", dict(sizes, buckets=pair["buckets"], mul_prev=pair["mul_prev"],
                                                          mul_cur=pair["mul_cur"], pair_name="bigram"), "embed")
    return ModelPlan(
        hidden_size=width,
        vocab_size=config.vocab,
        embedding=embedding,
        layers=tuple(layers),
        schedule=tuple(schedule),
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", dict(sizes, tied=True, scale=config.logit_scale), "embed"),
        eos_token_ids=frozenset() if config.eos_token_id is None else frozenset({config.eos_token_id}),
        max_positions=None,
        ignorable_names=frozenset(unread),
    )


register_architecture(RekezenConfig.architecture, RekezenConfig, rekezen_plan)
