"""The Sozavik decoder through the engine's loader, cache manager and step function (over the torch stand-in of the
kernel library, on the CPU) against the plain implementation: mechanism by mechanism, and through schedules of steps."""

from __future__ import annotations

import json

import pytest
import torch

from llmserve_amd import CacheConfig, EngineCore, GenerationConfig, ModelRunner, SchedulerConfig, StepEntry
from llmserve_amd.config import ConfigError
from llmserve_amd.config.sozavik import SozavikConfig
from llmserve_amd.weights import load_model_folder
from tests import sozavik_cases as cases
from tests.plain import sozavik_plain as plain
from tests.torch_kernels import TorchKernels


def runner_for(folder, page=4, pages=64, slots=4, dtype="float32", longest=None):
    loaded = load_model_folder(folder, dtype)
    return ModelRunner(loaded, TorchKernels(loaded.dtype), CacheConfig(block_size=page, num_blocks=pages, max_sequences=slots), use_graphs=False,
                       max_sequence_length=longest)


def oracle(folder, tokens):
    config, tensors = plain.read_folder(folder)
    logits, streams = plain.forward(config, tensors, tokens)
    return logits.float(), streams.float()


def close(got, want, atol=3e-4):
    torch.testing.assert_close(got.float(), want.float(), atol=atol, rtol=3e-4)


# ---------------------------------------------------------------------------- configuration and weights


def test_config_round_trip_and_refusals():
    config = SozavikConfig.from_dict(cases.MIXED)
    assert SozavikConfig.from_dict(config.to_config_json()) == config
    assert json.loads(json.dumps(config.to_config_json())) == cases.MIXED
    assert SozavikConfig.from_dict(cases.config_of([(cases.lightning(), None)], logit_softcap=None)).logit_softcap is None
    unmasked = cases.config_of([(cases.attention_2(), None)])
    del unmasked["layers"][0]["mixer"]["mask"]
    assert SozavikConfig.from_dict(unmasked).layers[0].mixer.window is None
    assert SozavikConfig.from_dict(SozavikConfig.from_dict(unmasked).to_config_json()) == SozavikConfig.from_dict(unmasked)
    broken = [
        cases.config_of([(cases.attention(heads=5, kv_heads=2), None)]),  # heads no multiple of kv_heads
        cases.config_of([(cases.attention(dims=26), None)]),  # more rotated dimensions than a head has
        cases.config_of([(cases.attention(dims=5), None)]),
        cases.config_of([(cases.lightning(heads=2), None)]),  # three decays for two heads
        cases.config_of([(cases.lightning(decay=(0.5, 1.5, 0.2)), None)]),
        cases.config_of([(cases.attention(), None), (cases.attention_2(vdim=24), None)]),  # mixed values of two sizes
        cases.config_of([({"type": "window", "mixer": {}}, None)]),
        cases.config_of([(cases.attention(), {"kind": "sparse", "ff": 8})]),
    ]
    missing = cases.config_of([(cases.attention(), None)])
    del missing["layers"][0]["mixer"]["scale"]
    for values in broken + [missing, {**cases.MIXED, "width": None}]:
        with pytest.raises(ConfigError):
            SozavikConfig.from_dict(values)


def test_folder_names_and_which_layers_give_and_take_values(tmp_path):
    from llmserve_amd.models.sozavik import sozavik_spec

    spec = sozavik_spec(SozavikConfig.from_dict(cases.MIXED))
    names = set(spec.tensors())
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.q.norm", "l0.mix.vmix", "l1.mix.norm", "l1.mix.g",
            "l2.mix.q.b", "l2.mix.sink", "l2.mix.g", "l2.mix.vmix", "l5.mlp.down"} <= names
    assert not {"l2.norm2", "l3.mix.vmix", "l0.mix.q.b", "l0.mix.sink", "l0.mix.g"} & names
    assert spec.tensors()["l0.mix.q.norm"].shape == (96,) and spec.tensors()["l2.mix.q.norm"].shape == (24,)
    assert spec.tensors()["l2.mix.g"].shape == (6, 40) and spec.tensors()["l1.mix.g"].shape == (72, 40) and spec.tensors()["l2.mix.vmix"].shape == ()
    assert [layer.block.mixer.values for layer in spec.layers if hasattr(layer.block.mixer, "values")] == ["give", "take", None, "take"]
    # a folder may hold the unused number of a layer that does not mix, and the norm of a feed-forward that is not there
    tensors = cases.random_tensors(cases.MIXED, 3)
    tensors["l3.mix.vmix"] = torch.tensor(0.5, dtype=torch.bfloat16)
    tensors["l2.norm2"] = torch.ones(40, dtype=torch.bfloat16)
    folder = cases.write_folder(tmp_path / "m", cases.MIXED, tensors=tensors)
    assert load_model_folder(folder, "float32").spec == spec


def test_stretched_frequencies():
    from llmserve_amd.parts import WavelengthScaling, rotary_frequencies

    for dims, base, scaling in ((10, 500.0, cases.STRETCH), (16, 10000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}),
                                (6, 50.0, {"factor": 2.5, "low": 0.5, "high": 3.0, "original": 20}), (8, 100.0, None)):
        want = plain.stretched_frequencies(dims, base, scaling)
        wanted = WavelengthScaling(*(scaling[name] for name in ("factor", "low", "high", "original"))) if scaling else None
        got, magnitude = rotary_frequencies(dims, base, wanted)
        assert magnitude == 1.0
        torch.testing.assert_close(got, want.float(), rtol=1e-6, atol=0)
    # all three regimes occur in the first case: kept, divided, and blended
    plain_f = [500.0 ** (-2.0 * i / 10) for i in range(5)]
    ratios = [float(a / b) for a, b in zip(plain.stretched_frequencies(10, 500.0, cases.STRETCH), plain_f)]
    assert ratios[0] == 1.0 and ratios[-1] == 0.25 and any(0.25 < r < 1.0 for r in ratios)


# ---------------------------------------------------------------------------- every mechanism alone

ALONE = {
    "attention": cases.config_of([(cases.attention(), None)]),
    "attention, all dimensions rotated, plain frequencies, one kv head": cases.config_of(
        [(cases.attention(heads=3, kv_heads=1, dim=16, vdim=16, dims=16, scaling=None, window=5), cases.dense(24))]),
    "attention, as many kv heads as heads, keys wider than values": cases.config_of([(cases.attention(heads=2, kv_heads=2, dim=40, vdim=8, dims=2, window=100), None)]),
    "attention_2": cases.config_of([(cases.attention_2(), cases.dense(40))]),
    "attention_2, grouped": cases.config_of([(cases.attention_2(heads=6, kv_heads=2, dim=8, vdim=24, window=4), None)], logit_softcap=None),
    "lightning": cases.config_of([(cases.lightning(), cases.dense(16))]),
    "lightning, one head, no decay": cases.config_of([(cases.lightning(heads=1, dim=24, vdim=8, decay=(1.0,)), None)]),
    "values given by attention_2 to attention": cases.config_of([(cases.attention_2(heads=4, kv_heads=2, dim=16, vdim=40), None), (cases.attention(), None)]),
    "values given by attention to both kinds": cases.config_of(
        [(cases.attention(), cases.dense(8)), (cases.lightning(), None), (cases.attention_2(), None), (cases.attention(heads=4, kv_heads=4, dim=8, vdim=20, dims=4), None)]),
    "no layer mixes values": cases.config_of([(cases.attention(v_mix=False), None), (cases.attention_2(v_mix=False), None)]),
}
ALONE["no mask"] = cases.config_of([(cases.attention(), cases.dense(16)), (cases.attention_2(), None)])
for _layer in ALONE["no mask"]["layers"]:
    del _layer["mixer"]["mask"]


@pytest.mark.parametrize("name", list(ALONE))
def test_each_mechanism_layer_by_layer(tmp_path, name):
    folder = cases.write_folder(tmp_path / "m", ALONE[name], seed=len(name))
    tokens = cases.tokens_of(37, ALONE[name]["vocab"], seed=5)
    want_logits, want_streams = oracle(folder, tokens)
    runner = runner_for(folder)
    seen = []
    runner.model.observer = lambda index, hidden, delta: seen.append(hidden.clone())
    logits = runner.step([StepEntry("a", tokens, range(len(tokens)))], create_missing=True)
    assert len(seen) == want_streams.shape[0]
    for index, stream in enumerate(seen):
        close(stream, want_streams[index])
    close(logits, want_logits)


def test_the_sink_the_cap_and_the_gate_matter(tmp_path):
    """The plain implementation without one of them gives other logits: the comparison above would see one left out."""
    values = ALONE["attention"]
    folder = cases.write_folder(tmp_path / "m", values, seed=4)
    config, tensors = plain.read_folder(folder)
    tokens = cases.tokens_of(30, values["vocab"], seed=1)
    want, _ = plain.forward(config, tensors, tokens)
    no_sink = dict(tensors, **{"l0.mix.sink": torch.full_like(tensors["l0.mix.sink"], -1e4)})
    no_gate = dict(tensors, **{"l0.mix.g": torch.zeros_like(tensors["l0.mix.g"])})
    uncapped = json.loads(json.dumps(config))
    uncapped["layers"][0]["mixer"]["softcap"] = 1e6
    for other in (plain.forward(config, no_sink, tokens)[0], plain.forward(config, no_gate, tokens)[0], plain.forward(uncapped, tensors, tokens)[0]):
        assert float((other - want).abs().max()) > 0.02


# ---------------------------------------------------------------------------- steps, cache and state


@pytest.fixture(scope="module")
def mixed_folder(tmp_path_factory):
    return cases.write_folder(tmp_path_factory.mktemp("sozavik") / "mixed", cases.MIXED, seed=7)


@pytest.fixture(scope="module")
def sharp_folder(tmp_path_factory):
    """Attention that looks at one key, wherever in its window it is, and a state that remembers far back."""
    values = cases.config_of(
        [(cases.attention(heads=2, kv_heads=1, dim=8, vdim=16, window=19, scale=1.5, softcap=40.0, dims=4), cases.dense(24)),
         (cases.lightning(heads=2, dim=16, vdim=8, decay=(0.999, 0.98)), None),
         (cases.attention_2(heads=2, kv_heads=2, dim=16, vdim=8, window=33, scale=2.0), None)],
        vocab=43, width=24,
    )
    return cases.write_folder(tmp_path_factory.mktemp("sozavik") / "sharp", values, seed=11, sharp=True)


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
    got = cases.run_steps(runner, [[("tail", 61)]] + [[("tail", 1)]] * 89, prompts)  # long decoding: windows pass over decoded tokens
    close(torch.stack([got[("tail", p)] for p in range(150)]), want)
    sizes = [7, 2, 16, 3, 2, 1, 25, 1, 14, 2, 2, 9, 33, 2, 31]
    assert sum(sizes) == 150
    got = cases.run_steps(runner, [[("cut", n)] for n in sizes], prompts)
    close(torch.stack([got[("cut", p)] for p in range(150)]), want)
    got = cases.run_steps(runner, [[("pairs", 2)]] * 20, prompts)
    close(torch.stack([got[("pairs", p)] for p in range(40)]), want[:40])
    assert runner.cache.used_pages == 0


def test_pages_behind_a_window_are_given_back(mixed_folder):
    """A long request in a pool far smaller than its length: every group keeps only its window's pages."""
    tokens = cases.tokens_of(260, 67, seed=9)
    want, _ = oracle(mixed_folder, tokens)
    runner = runner_for(mixed_folder, page=4, pages=16, longest=512)  # 64 tokens' room a group; the widest window is 30
    got = cases.run_steps(runner, [[("long", 20)]] * 11 + [[("long", 1)]] * 40, {"long": tokens})
    close(torch.stack([got[("long", p)] for p in range(260)]), want)


def test_the_first_tokens_of_a_sequence(mixed_folder):
    """Prompts of one to five tokens, whole and token by token: windows that reach before the start, the empty state."""
    runner = runner_for(mixed_folder)
    for length in (1, 2, 3, 5):
        tokens = cases.tokens_of(length, 67, seed=length)
        want, _ = oracle(mixed_folder, tokens)
        got = cases.run_steps(runner, [[("w", length)]], {"w": tokens})
        close(torch.stack([got[("w", p)] for p in range(length)]), want)
        got = cases.run_steps(runner, [[("s", 1)]] * length, {"s": tokens})
        close(torch.stack([got[("s", p)] for p in range(length)]), want)


@pytest.mark.parametrize("which", ["mixed", "sharp"])
def test_mixed_batches_with_pages_and_slots_used_again(mixed_folder, sharp_folder, which):
    """Six unequal requests through three state slots and a small pool: portions beside single tokens, requests that
    pause for a step, slots and pages taken over from requests that ended."""
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
    """One slot, one request after the other: what the first left in the state is gone."""
    runner = runner_for(sharp_folder, slots=1, pages=16)
    first, second = cases.tokens_of(30, 43, seed=1), cases.tokens_of(12, 43, seed=2)
    cases.run_steps(runner, [[("first", 30)]], {"first": first})
    got = cases.run_steps(runner, [[("second", 5)], [("second", 7)]], {"second": second})
    want, _ = oracle(sharp_folder, second)
    close(torch.stack([got[("second", p)] for p in range(12)]), want)


WINDOW = 23


def edge_case(folder_root, kind):
    """A one-layer model of window attention with large queries and keys, and two tokens (asker, key) such that the
    asker's answer hangs on the one key of the other kind wherever in its window that lies: found by trying seeds and
    pairs on the plain implementation.  Returns (folder, asker, key)."""
    mixer = cases.attention(heads=2, kv_heads=1, dim=16, vdim=8, window=WINDOW, scale=1.5, softcap=40.0, dims=4) if kind == "attention" else \
        cases.attention_2(heads=2, kv_heads=2, dim=16, vdim=8, window=WINDOW, scale=2.5)
    values = cases.config_of([(mixer, None)], vocab=37, width=24)
    for seed in range(1, 40):
        folder = cases.write_folder(folder_root / f"{kind}{seed}", values, seed=seed, sharp=True)
        config, tensors = plain.read_folder(folder)
        for asker in range(31, 37):
            for key in range(31, 37):
                if asker == key:
                    continue
                effects = []
                for distance in (1, WINDOW - 2, WINDOW - 1):
                    tokens = [1 + (i % 30) for i in range(80)]
                    tokens[79 - distance], tokens[-1] = key, asker
                    with_key, _ = plain.forward(config, tensors, tokens)
                    tokens[79 - distance] = 30
                    without, _ = plain.forward(config, tensors, tokens)
                    effects.append(float((with_key[-1] - without[-1]).abs().max()))
                    if effects[-1] < 0.2:
                        break
                if min(effects) >= 0.2:
                    return folder, asker, key
    raise AssertionError("no seed gave a key that matters at the window's edge")


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_one_key_just_inside_and_just_outside_the_window(tmp_path, kind):
    """A query whose answer hangs on one key: the key at the window's last place, one beyond it, next to the query,
    and at a page's border; in a prompt's portion and decoded alone, with pages of 4 and of 16."""
    folder, asker, key = edge_case(tmp_path, kind)
    config, tensors = plain.read_folder(folder)
    for distance in (1, WINDOW - 2, WINDOW - 1, WINDOW, WINDOW + 1, 79 - 16, 79):
        tokens = [1 + (i % 30) for i in range(80)]
        tokens[79 - distance], tokens[-1] = key, asker
        want, _ = plain.forward(config, tensors, tokens)
        moved = list(tokens)
        moved[79 - distance] = 30
        other, _ = plain.forward(config, tensors, moved)
        effect = float((want[-1] - other[-1]).abs().max())
        assert effect > 0.05 if distance < WINDOW else effect == 0.0, "the test tests nothing"
        for page in (4, 16):
            runner = runner_for(folder, page=page, pages=40)
            got = cases.run_steps(runner, [[("p", 80)]], {"p": tokens})
            close(got[("p", 79)], want[-1].float())
            got = cases.run_steps(runner, [[("d", 50)], [("d", 13)], [("d", 2)]] + [[("d", 1)]] * 15, {"d": tokens})
            close(got[("d", 79)], want[-1].float())


def test_a_token_far_back_stays_in_the_state(tmp_path):
    """Linear attention that hardly fades: the first token of 400 still decides the last one's answer."""
    values = cases.config_of([(cases.lightning(heads=2, dim=16, vdim=8, decay=(1.0, 0.9995)), None)], vocab=37, width=24)
    folder = cases.write_folder(tmp_path / "far", values, seed=2)
    config, tensors = plain.read_folder(folder)
    tokens = [1 + (i % 30) for i in range(400)]
    tokens[0] = 35
    want, _ = plain.forward(config, tensors, tokens)
    other, _ = plain.forward(config, tensors, [30] + tokens[1:])
    assert float((want[-1] - other[-1]).abs().max()) > 1e-2
    runner = runner_for(folder, page=16, pages=40)
    got = cases.run_steps(runner, [[("p", 400)]], {"p": tokens})
    close(got[("p", 399)], want[-1].float())
    got = cases.run_steps(runner, [[("d", 333)], [("d", 47)]] + [[("d", 1)]] * 20, {"d": tokens})
    close(got[("d", 399)], want[-1].float())


# ---------------------------------------------------------------------------- generation


def greedy(config, tensors, prompt, count):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(torch.argmax(plain.forward(config, tensors, tokens)[0][-1])))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_engine(mixed_folder):
    config, tensors = plain.read_folder(mixed_folder)
    prompts = [cases.tokens_of(n, 67, seed=40 + n) for n in (1, 6, 17, 30)]
    expected = [greedy(config, tensors, prompt, 7) for prompt in prompts]
    runner = runner_for(mixed_folder, page=4, pages=64, slots=4)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=3, max_tokens_per_step=24), prefill_chunk_size=8)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=7)) == expected
    assert runner.cache.used_pages == 0


ONE_KIND = {
    "only lightning": cases.config_of([(cases.lightning(), cases.dense(24)), (cases.lightning(heads=2, dim=8, vdim=24, decay=(0.9, 0.99)), None)]),
    "only attention": cases.config_of([(cases.attention(), cases.dense(24)), (cases.attention_2(), None)]),
}


@pytest.mark.parametrize("name", list(ONE_KIND))
def test_models_of_one_kind_of_layer_through_the_scheduler(tmp_path, name):
    """A model that keeps no pages at all, and one that keeps no state: generation through the scheduler."""
    folder = cases.write_folder(tmp_path / "m", ONE_KIND[name], seed=5)
    config, tensors = plain.read_folder(folder)
    prompts = [cases.tokens_of(n, 67, seed=60 + n) for n in (3, 11, 20)]
    expected = [greedy(config, tensors, prompt, 5) for prompt in prompts]
    runner = runner_for(folder, page=4, pages=32, slots=3)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=2, max_tokens_per_step=16), prefill_chunk_size=6)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=5)) == expected
    assert len(runner.cache.sequences) == 0


def test_the_command_line_writes_a_random_model_folder(tmp_path, capsys):
    """`llmserve random-model` goes through the registry: a Sozavik config.json gives a folder that loads and runs."""
    from llmserve_amd.cli import main

    (tmp_path / "config.json").write_text(json.dumps(cases.MIXED))
    assert main(["random-model", "--config", str(tmp_path / "config.json"), "--output", str(tmp_path / "out"), "--seed", "5", "--std", "0.2"]) == 0
    assert str(tmp_path / "out") in capsys.readouterr().out
    tokens = cases.tokens_of(12, 67, seed=2)
    want, _ = oracle(tmp_path / "out", tokens)
    runner = runner_for(tmp_path / "out")
    close(runner.step([StepEntry("a", tokens, range(12))], create_missing=True), want)
