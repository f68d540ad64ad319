"""Mazanex through the engine on the CPU, with the kernels' plain references patched in, against
the plain implementation (tests/plain_mazanex.py): configuration and tensor names, each mixer
alone, and that logits do not depend on how requests are cut into steps, batched, or placed in
pages and state slots.  The kernels themselves run in the GPU tests."""

from __future__ import annotations

import pytest
import torch

import kernel_refs
import mazanex_util as mu
import replay_util as ru
from forge_engine_amd.config import ConfigError, SchedulerConfig, load_model_config
from forge_engine_amd.engine import ModelRunner, StepEntry, build_engine, load_model
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.weights.random_init import declared_tensors

CONFIGS = {"A": mu.MIXED_A, "B": mu.MIXED_B}
LENGTHS = {"A": (5, 1, 14, 27), "B": (2, 9, 21, 33)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {name: mu.write_model(raw, 7, tmp_path_factory.mktemp(f"mazanex_{name}")) for name, raw in CONFIGS.items()}
    for name, raw in mu.ALONE.items():
        made[name] = mu.write_model(raw, 8, tmp_path_factory.mktemp(f"alone_{name}"))
    return made


def requests_of(name, seed, lengths):
    return ru.make_requests({"vocab_size": CONFIGS.get(name, mu.ALONE.get(name))["vocab"]}, seed, lengths)


def test_configuration_names_and_shapes():
    config = load_model_config(mu.MIXED_A)
    assert config.architecture == "Mazanex" and load_model_config(config.to_dict()) == config
    tensors = declared_tensors(config)
    for name, shape in {"embed": (96, 48), "head": (96, 48), "final.norm": (48,), "l0.shift": (48,), "l0.norm1": (48,),
                        "l0.norm2": (48,), "l0.mix.left.q": (64, 48), "l0.mix.left.q.b": (64,), "l0.mix.left.k.conv": (32, 3),
                        "l0.mix.left.v": (16, 48), "l0.mix.left.sink": (4,), "l0.mix.left.g": (32, 48), "l0.mix.left.o": (48, 32),
                        "l0.mix.left.o.b": (48,), "l0.mix.left.out": (48,), "l0.mix.right.out": (48,), "l0.mix.right.mu.w": (48,),
                        "l0.mix.right.w1": (5, 48), "l0.mix.right.w2": (48, 5), "l0.mix.right.u": (3, 16), "l0.mix.right.norm": (48,),
                        "l1.mix.a1": (5, 48), "l1.mix.a2.b": (16,), "l1.mix.norm": (24,), "l1.mix.v": (48, 48),
                        "l2.mix.i": (3, 48), "l2.mix.f.b": (3,), "l2.mix.norm": (48,), "l2.mlp.act": (4,), "l2.mlp.up": (56, 48)}.items():
        assert tuple(tensors[name].shape) == shape, name
    assert "l1.norm2" not in tensors and not any(n.startswith("l1.mlp") for n in tensors)     # a layer without a feed-forward
    for broken in ({**mu.MIXED_A, "layers": []}, {**mu.MIXED_A, "layers": [mu.layer("conv", {}, None)]},
                   {**mu.MIXED_A, "layers": [mu.layer("parallel", {"left": mu.attention(3, 2, 8, 8, 2, 4, 8), "right": {"heads": 1, "dim": 8}}, None)]},
                   {k: v for k, v in mu.MIXED_A.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            load_model_config(broken)


def test_decay_ranks_come_from_the_checkpoint(folders, tmp_path, monkeypatch):
    """The inner size of a low-rank decay projection is nowhere in config.json: a folder whose
    config lacks the optional key loads by the tensors' shapes."""
    import json
    import shutil
    kernel_refs.install(monkeypatch)
    folder = shutil.copytree(folders["A"], tmp_path / "copy")
    raw = json.loads((folder / "config.json").read_text())
    del raw["layers"][0]["mixer"]["right"]["rank"], raw["layers"][1]["mixer"]["rank"]
    (folder / "config.json").write_text(json.dumps(raw))
    _, model = load_model(folder, dtype="float32", device="cpu")
    assert model.layers[1].mixer.decay_rank == 5 and model.layers[0].mixer.branches["right"].decay_rank == 5


@pytest.mark.parametrize("name", list(mu.ALONE))
def test_each_mixer_alone(name, folders, tmp_path, monkeypatch):
    kernel_refs.install(monkeypatch)
    requests = requests_of(name, 2, (19, 1))
    got = ru.run_trace(folders[name], "float32", ru.trace_whole(requests), tmp_path, block_size=4, device="cpu", on_cpu=True)
    mu.compare(got, mu.plain_logits(folders[name], requests), "float32")


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(name, mode, folders, tmp_path, monkeypatch):
    """Whole prompts; a prompt and then token by token (across the edges of chunks and pages);
    portions down to two tokens; up to four live requests, portions beside single tokens."""
    kernel_refs.install(monkeypatch)
    requests = requests_of(name, 3, LENGTHS[name])
    trace = {"whole": ru.trace_whole, "tail": lambda r: ru.trace_tail(r, 16), "portions": ru.trace_portions,
             "mixed": lambda r: ru.trace_mixed(r, 5, max_live=3)}[mode](requests)
    got = ru.run_trace(folders[name], "float32", trace, tmp_path, block_size=mu.BLOCK_SIZE[name], device="cpu", on_cpu=True)
    mu.compare(got, mu.plain_logits(folders[name], requests), "float32")


def test_pages_and_state_slots_are_used_again(folders, tmp_path, monkeypatch):
    """Seven requests through four state slots and a pool smaller than their sum: a slot's state
    starts at zero again for the request that takes it over."""
    kernel_refs.install(monkeypatch)
    requests = requests_of("A", 4, (12, 20, 7, 16, 9, 3, 11))
    trace = ru.trace_mixed(requests, 9, max_live=4)
    assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens
    got = ru.run_trace(folders["A"], "float32", trace, tmp_path, block_size=4, device="cpu", on_cpu=True)
    mu.compare(got, mu.plain_logits(folders["A"], requests), "float32")


def test_chunked_groups_give_pages_back(folders, monkeypatch):
    """Keys before the run of positions that the next token lies in are never read again: their
    pages return to the pool while the request lives."""
    kernel_refs.install(monkeypatch)
    _, model = load_model(folders["A"], dtype="float32", device="cpu")
    runner = ModelRunner(model, block_size=2, block_capacity=16, num_state_slots=2)
    tokens = requests_of("A", 5, (40,))["r0"]
    runner.begin("r0")
    for start in range(0, 40, 5):
        runner.step([StepEntry("r0", tokens[start:start + 5], [4])])
        record = runner.cache.request("r0")
        chunk = mu.PARALLEL_P["left"]["mask"]["size"]
        assert record.first_block[0] == (start + 5) // chunk * chunk // 2
        assert sum(1 for page in record.tables[0] if page >= 0) <= 5
    runner.cache.check_invariants()
    runner.end("r0")
    assert runner.cache.allocated_pages == 0


def test_long_decoding_token_by_token(folders, tmp_path, monkeypatch):
    kernel_refs.install(monkeypatch)
    requests = requests_of("B", 6, (70,))
    got = ru.run_trace(folders["B"], "float32", ru.trace_tail(requests, 69), tmp_path, block_size=8, device="cpu", on_cpu=True)
    mu.compare(got, mu.plain_logits(folders["B"], requests), "float32")


def test_greedy_generation_through_the_scheduler(folders, monkeypatch):
    kernel_refs.install(monkeypatch)
    _, model = load_model(folders["A"], dtype="float32", device="cpu")
    engine = build_engine(model, scheduler_config=SchedulerConfig(block_size=4, block_capacity=64, token_budget=8, max_batch_size=3),
                          eos_token_ids=())
    prompts = list(requests_of("A", 11, (13, 4, 9)).values())
    ids = [engine.submit(prompt, sampling_params=SamplingParams(max_new_tokens=6)) for prompt in prompts]
    engine.run_until_idle()
    for request_id, prompt in zip(ids, prompts):
        assert list(engine.request(request_id).output_token_ids) == mu.plain_greedy(folders["A"], prompt, 6)
