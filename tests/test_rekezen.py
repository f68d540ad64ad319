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
