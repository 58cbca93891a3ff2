"""The Dafutar decoder through the engine's configuration, loader, cache manager and step function (with the torch
stand-in for the kernel library), against the plain implementation of tests/plain/dafutar_plain.py: each mechanism in a
model of its own, whole prompts against token-by-token decoding and portions of any size, mixed batches against each
request alone, pages and state slots used again, keys far away and at page borders, and greedy generation through the
engine's own entry point."""

from __future__ import annotations

import math

import pytest
import torch

from llmserve_amd import CacheConfig, GenerationConfig, SchedulerConfig, StepEntry
from llmserve_amd.config import ConfigError, DafutarConfig
from llmserve_amd.engine import EngineCore, ModelRunner
from llmserve_amd.parts import YarnScaling, rotary_frequencies
from llmserve_amd.weights import WeightsError, load_model_folder, read_config, write_model_folder
from tests import dafutar_cases as cases
from tests.plain import dafutar_plain as plain
from tests.torch_kernels import TorchKernels


def runner_for(folder, page=4, pages=64, slots=4, dtype="float32"):
    loaded = load_model_folder(folder, dtype)
    return ModelRunner(loaded, TorchKernels(loaded.dtype), CacheConfig(block_size=page, num_blocks=pages, max_sequences=slots), use_graphs=False)


def oracle(folder, tokens):
    config, tensors = plain.read_folder(folder)
    logits, streams = plain.forward(config, tensors, tokens)
    return logits.float(), streams.float()


def close(got, want, atol=3e-4):
    torch.testing.assert_close(got.float(), want.float(), atol=atol, rtol=3e-4)


# ---------------------------------------------------------------------------- configuration and weights


def test_config_round_trip_and_refusals():
    config = DafutarConfig.from_dict(cases.MIXED)
    assert DafutarConfig.from_dict(config.to_config_json()) == config
    assert config.layers[3].mlp is None and config.layers[3].mixer.rot.scaling is None and config.loop.times == 3
    broken = dict(cases.MIXED, loop={"start": 3, "stop": 2, "times": 2})
    with pytest.raises(ConfigError):
        DafutarConfig.from_dict(broken)
    without = {key: value for key, value in cases.MIXED.items() if key != "width"}
    with pytest.raises(ConfigError, match="width"):
        DafutarConfig.from_dict(without)
    assert DafutarConfig.from_dict({key: value for key, value in cases.MIXED.items() if key != "loop"}).loop is None


def test_folder_names_and_a_random_model_folder(tmp_path):
    folder = cases.write_folder(tmp_path / "m", cases.MIXED, seed=2)
    architecture, config = read_config(folder)
    assert architecture.name == "Dafutar"
    names = set(architecture.build_spec(config).tensors())
    assert {"embed", "head", "final.norm", "final.norm.b", "loop.in", "loop.step", "l0.mix.q.conv", "l1.mix.dkv.norm", "l1.mlp.e4.down",
            "l1.mlp.shared.sg", "l2.mlp.correction", "l0.mlp.gate", "l3.norm1.b"} <= names
    assert "l3.norm2" not in names and "l2.mlp.shared.up" not in names
    loaded = load_model_folder(folder, "bfloat16")
    assert loaded.tensors["l0.mix.A_log"].dtype == torch.bfloat16
    # a folder that still holds the norm of a feed-forward that is not there is accepted, one with a stranger is not
    tensors = cases.random_tensors(cases.MIXED, 2)
    tensors["l3.norm2"] = torch.ones(32, dtype=torch.bfloat16)
    load_model_folder(cases.write_folder(tmp_path / "n", cases.MIXED, tensors=tensors))
    tensors["l3.mix.bias"] = torch.ones(32, dtype=torch.bfloat16)
    with pytest.raises(WeightsError, match="unexpected"):
        load_model_folder(cases.write_folder(tmp_path / "o", cases.MIXED, tensors=tensors))
    # the seeded random-weights mode writes the same names
    written = write_model_folder(tmp_path / "p", config, seed=4)
    assert set(plain.read_folder(written)[1]) == names


def test_yarn_frequencies():
    for dims, base, scaling in [(8, 10000.0, None), (6, 500.0, (4.0, 64, 8.0, 1.0)), (32, 10000.0, (8.0, 1024, 32.0, 1.0)), (4, 100.0, (2.0, 16, 1.0, 1.0))]:
        described = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
        want, want_magnitude = plain.rotary_frequencies(dims, base, described)
        got, magnitude = rotary_frequencies(dims, base, YarnScaling(*scaling) if scaling else None)
        torch.testing.assert_close(got.double(), want, atol=0, rtol=1e-6)
        assert math.isclose(magnitude, want_magnitude)


# ---------------------------------------------------------------------------- each mechanism in a model of its own

ALONE = {
    "latent": cases.config_of([(cases.latent(heads=3, dim=16, rot_dim=8, vdim=24, dims=4), None)]),
    "latent without scaling": cases.config_of([(cases.latent(heads=1, dim=8, rot_dim=16, vdim=8, kv_rank=16, scaling=None), None)], width=24),
    "delta": cases.config_of([(cases.delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3), None)]),
    "delta of one tap": cases.config_of([(cases.delta(heads=2, kv_heads=2, dim=8, vdim=8, conv=1), None)]),
    "delta of one head": cases.config_of([(cases.delta(heads=3, kv_heads=1, dim=24, vdim=40, conv=4), None)]),
    "dense": cases.config_of([(cases.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2), cases.dense(56))]),
    "experts": cases.config_of([(cases.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2), cases.moe(6, 3, 0.5, 12, 20))]),
    "experts, all of them, none shared": cases.config_of([(cases.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2), cases.moe(3, 3, 2.0, 8, None))]),
    "one expert a token": cases.config_of([(cases.latent(), cases.moe(7, 1, 1.0, 8, 4))]),
    "loop from the first layer": cases.config_of([(cases.delta(), cases.dense(24)), (cases.latent(), None)], loop=(0, 2, 2)),
    "loop of one pass, layers behind it": cases.config_of([(cases.latent(), None), (cases.delta(), None), (cases.delta(conv=2), cases.dense(16))], loop=(1, 2, 1)),
    "no loop": cases.config_of([(cases.latent(), cases.dense(16)), (cases.delta(), None)]),
}


@pytest.mark.parametrize("name", list(ALONE))
def test_each_mechanism_layer_by_layer(tmp_path, name):
    folder = cases.write_folder(tmp_path / "m", ALONE[name], seed=len(name))
    tokens = cases.tokens_of(19, ALONE[name]["vocab"], seed=5)
    want_logits, want_streams = oracle(folder, tokens)
    runner = runner_for(folder)
    seen = []
    runner.model.observer = lambda index, hidden, delta: seen.append(
        (hidden if delta is None else hidden + (delta if delta.ndim == 2 else delta.sum(0))).clone()
    )
    logits = runner.step([StepEntry("a", tokens, range(len(tokens)))], create_missing=True)
    assert len(seen) == want_streams.shape[0]
    for index, stream in enumerate(seen):
        close(stream, want_streams[index])
    close(logits, want_logits)


def test_the_run_order_of_a_loop():
    from llmserve_amd.models.dafutar import dafutar_spec

    spec = dafutar_spec(DafutarConfig.from_dict(cases.MIXED))
    assert [(run.layer, run.enters) for run in spec.run_order] == [
        (0, None), (1, 0), (2, None), (3, None), (1, 1), (2, None), (3, None), (1, 2), (2, None), (3, None), (4, None)]
    assert [(layer, number if first else None) for layer, number, first in plain.run_order(cases.MIXED)] == [
        (run.layer, run.enters) for run in spec.run_order]


# ---------------------------------------------------------------------------- steps, cache and state


@pytest.fixture(scope="module")
def mixed_folder(tmp_path_factory):
    return cases.write_folder(tmp_path_factory.mktemp("dafutar") / "mixed", cases.MIXED, seed=7)


@pytest.fixture(scope="module")
def sharp_folder(tmp_path_factory):
    """Attention that looks at one key, wherever it is (a large scale), and states that remember far back."""
    values = cases.config_of(
        [(cases.latent(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=16, scale=6.0), cases.dense(24)), (cases.delta(heads=2, kv_heads=1, dim=16, vdim=8, conv=4), None)],
        loop=(0, 2, 2), vocab=43, width=24,
    )
    return cases.write_folder(tmp_path_factory.mktemp("dafutar") / "sharp", values, seed=11, sharp=True)


@pytest.mark.parametrize("which", ["mixed", "sharp"])
def test_whole_then_one_by_one_then_portions(mixed_folder, sharp_folder, which):
    folder = mixed_folder if which == "mixed" else sharp_folder
    vocab = plain.read_folder(folder)[0]["vocab"]
    tokens = cases.tokens_of(150, vocab, seed=3)
    want, _ = oracle(folder, tokens)
    runner = runner_for(folder, page=8, pages=80)
    prompts = {"whole": tokens, "tail": tokens, "cut": tokens, "pairs": tokens[:40]}
    got = cases.run_steps(runner, [[("whole", 150)]], prompts)
    close(torch.stack([got[("whole", p)] for p in range(150)]), want)
    got = cases.run_steps(runner, [[("tail", 61)]] + [[("tail", 1)]] * 89, prompts)  # long decoding over page borders
    close(torch.stack([got[("tail", p)] for p in range(150)]), want)
    sizes = [7, 2, 16, 3, 2, 1, 25, 1, 14, 2, 2, 9, 33, 2, 31]
    assert sum(sizes) == 150
    got = cases.run_steps(runner, [[("cut", n)] for n in sizes], prompts)
    close(torch.stack([got[("cut", p)] for p in range(150)]), want)
    got = cases.run_steps(runner, [[("pairs", 2)]] * 20, prompts)
    close(torch.stack([got[("pairs", p)] for p in range(40)]), want[:40])
    assert runner.cache.used_pages == 0


def test_the_first_tokens_of_a_sequence(mixed_folder):
    """Prompts of one to five tokens, whole and token by token: the convolutions' zeros before the start, the empty state."""
    runner = runner_for(mixed_folder)
    for length in (1, 2, 3, 5):
        tokens = cases.tokens_of(length, 61, seed=length)
        want, _ = oracle(mixed_folder, tokens)
        got = cases.run_steps(runner, [[("w", length)]], {"w": tokens})
        close(torch.stack([got[("w", p)] for p in range(length)]), want)
        got = cases.run_steps(runner, [[("s", 1)]] * length, {"s": tokens})
        close(torch.stack([got[("s", p)] for p in range(length)]), want)


@pytest.mark.parametrize("which", ["mixed", "sharp"])
def test_mixed_batches_with_pages_and_slots_used_again(mixed_folder, sharp_folder, which):
    """Six unequal requests through three state slots and a pool that holds about half of them: portions beside
    single tokens, requests that pause for a step, slots and pages taken over from requests that ended."""
    folder = mixed_folder if which == "mixed" else sharp_folder
    vocab = plain.read_folder(folder)[0]["vocab"]
    lengths = {"a": 45, "b": 9, "c": 30, "d": 61, "e": 1, "f": 26}
    prompts = {name: cases.tokens_of(n, vocab, seed=20 + n) for name, n in lengths.items()}
    want = {name: oracle(folder, prompts[name])[0] for name in prompts}
    page = 4
    runner = runner_for(folder, page=page, pages=30, slots=3)
    generator = torch.Generator().manual_seed(5)
    done = dict.fromkeys(prompts, 0)
    waiting, live, step_number, at = list(prompts), [], 0, {}
    while waiting or live:
        while waiting and len(live) < 3 and sum(-(-lengths[n] // page) for n in live + [waiting[0]]) <= 30:
            live.append(waiting.pop(0))
        step = []
        for name in live:
            if len(live) > 1 and step_number % 5 == 3 and name == live[0]:
                continue  # left out of this step, goes on later
            left = lengths[name] - done[name]
            count = 1 if done[name] > lengths[name] // 2 else min(left, int(torch.randint(2, 13, (1,), generator=generator)))
            step.append((name, count))
            done[name] += count
        got = cases.run_steps(runner, [step], prompts, at)
        for (name, position), row in got.items():
            close(row, want[name][position])
        live = [name for name in live if done[name] < lengths[name]]
        step_number += 1
    assert runner.cache.used_pages == 0 and len(runner.cache.sequences) == 0


def test_a_slot_taken_over_starts_from_nothing(sharp_folder):
    """One slot, one request after the other: what the first left in the state and in the convolutions' inputs is gone."""
    runner = runner_for(sharp_folder, slots=1, pages=16)
    first, second = cases.tokens_of(30, 43, seed=1), cases.tokens_of(12, 43, seed=2)
    cases.run_steps(runner, [[("first", 30)]], {"first": first})
    got = cases.run_steps(runner, [[("second", 5)], [("second", 7)]], {"second": second})
    want, _ = oracle(sharp_folder, second)
    close(torch.stack([got[("second", p)] for p in range(12)]), want)


PLACES = (0, 1, 15, 16, 31, 32, 255, 256)


def far_key_case(folder_root):
    """A one-layer model of latent attention with a large scale, and two tokens (asker, key) such that a query of the
    asker 300 tokens on looks at the one key of the other kind rather than at the hundreds between: found by trying
    seeds and pairs on the plain implementation.  Returns (folder, asker, key)."""
    values = cases.config_of([(cases.latent(heads=2, dim=16, rot_dim=4, vdim=8, kv_rank=16, scale=6.0, scaling=None), None)], vocab=37, width=24)
    for seed in range(1, 40):
        folder = cases.write_folder(folder_root / f"far{seed}", values, seed=seed)
        config, tensors = plain.read_folder(folder)
        for asker in range(31, 37):
            for key in range(31, 37):
                if asker == key:
                    continue
                effects = []
                for place in PLACES:
                    tokens = [1 + (i % 30) for i in range(300)]
                    tokens[place], tokens[-1] = key, asker
                    with_key, _ = plain.forward(config, tensors, tokens)
                    tokens[place] = 30
                    without, _ = plain.forward(config, tensors, tokens)
                    effects.append(float((with_key[-1] - without[-1]).abs().max()))
                    if effects[-1] < 0.2:
                        break
                if min(effects) >= 0.2:
                    return folder, asker, key
    raise AssertionError("no seed gave a far key that matters")


def test_one_far_key_decides(tmp_path):
    """A query whose answer hangs on one key hundreds of tokens back, in a prompt's portion and decoded alone, the key at a
    page's first and last place and in the sequence's first tokens."""
    folder, asker, key = far_key_case(tmp_path)
    config, tensors = plain.read_folder(folder)
    for place in PLACES:
        tokens = [1 + (i % 30) for i in range(300)]
        tokens[place], tokens[-1] = key, asker
        want, _ = plain.forward(config, tensors, tokens)
        moved = list(tokens)
        moved[place] = 30
        other, _ = plain.forward(config, tensors, moved)
        assert float((want[-1] - other[-1]).abs().max()) > 0.05, "the far key does not matter to this query: the test tests nothing"
        runner = runner_for(folder, page=16, pages=40)
        got = cases.run_steps(runner, [[("p", 300)]], {"p": tokens})
        close(got[("p", 299)], want[-1].float())
        got = cases.run_steps(runner, [[("d", 290)]] + [[("d", 1)]] * 10, {"d": tokens})
        close(got[("d", 299)], want[-1].float())


# ---------------------------------------------------------------------------- generation


def test_greedy_generation_through_the_engine(mixed_folder):
    config, tensors = plain.read_folder(mixed_folder)
    prompts = [cases.tokens_of(n, 61, seed=40 + n) for n in (1, 6, 17, 30)]

    def generate(prompt, count):
        tokens = list(prompt)
        for _ in range(count):
            logits, _ = plain.forward(config, tensors, tokens)
            tokens.append(int(torch.argmax(logits[-1])))
        return tokens[len(prompt):]

    expected = [generate(prompt, 7) for prompt in prompts]
    runner = runner_for(mixed_folder, page=4, pages=64, slots=4)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=3, max_tokens_per_step=24), prefill_chunk_size=8)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=7)) == expected
    assert runner.cache.used_pages == 0


ONE_KIND = {
    "only the delta rule": cases.config_of([(cases.delta(), cases.moe(4, 2, 1.0, 8, 8)), (cases.delta(heads=2, kv_heads=1, dim=8, vdim=24, conv=2), None)], loop=(0, 1, 2)),
    "only latent attention": cases.config_of([(cases.latent(), cases.dense(24)), (cases.latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=12), None)]),
}


@pytest.mark.parametrize("name", list(ONE_KIND))
def test_models_of_one_kind_of_layer_through_the_scheduler(tmp_path, name):
    """A model that keeps no pages at all, and one that keeps no state: steps, and generation through the scheduler."""
    folder = cases.write_folder(tmp_path / "m", ONE_KIND[name], seed=5)
    config, tensors = plain.read_folder(folder)
    prompts = [cases.tokens_of(n, 61, seed=60 + n) for n in (3, 11, 20)]
    expected = []
    for prompt in prompts:
        tokens = list(prompt)
        for _ in range(5):
            tokens.append(int(torch.argmax(plain.forward(config, tensors, tokens)[0][-1])))
        expected.append(tokens[len(prompt):])
    runner = runner_for(folder, page=4, pages=32, slots=3)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=2, max_tokens_per_step=16), prefill_chunk_size=6)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=5)) == expected
    assert len(runner.cache.sequences) == 0


def test_the_command_line_writes_a_random_model_folder(tmp_path, capsys):
    """`llmserve random-model` goes through the registry: a Dafutar config.json gives a folder that loads and runs."""
    import json

    from llmserve_amd.cli import main

    (tmp_path / "config.json").write_text(json.dumps(cases.MIXED))
    assert main(["random-model", "--config", str(tmp_path / "config.json"), "--output", str(tmp_path / "out"), "--seed", "5", "--std", "0.2"]) == 0
    assert str(tmp_path / "out") in capsys.readouterr().out
    tokens = cases.tokens_of(12, 61, seed=2)
    want, _ = oracle(tmp_path / "out", tokens)
    runner = runner_for(tmp_path / "out")
    close(runner.step([StepEntry("a", tokens, range(12))], create_missing=True), want)
