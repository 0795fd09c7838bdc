"""The Katenex decoder through the engine's configuration, loader, cache manager and step function (with the torch
stand-in for the kernel library), against the plain implementation of tests/plain/katenex_plain.py: each mechanism in a
model of its own, whole prompts against token-by-token decoding and portions of any size, mixed batches against each
request alone, pages and state slots used again, keys far away and at page borders, and greedy generation through the
engine's own entry point."""

from __future__ import annotations

import json

import pytest
import torch

from llmserve_amd import CacheConfig, GenerationConfig, SchedulerConfig, StepEntry
from llmserve_amd.config import ConfigError, KatenexConfig
from llmserve_amd.engine import EngineCore, ModelRunner
from llmserve_amd.parts import LinearScaling, rotary_frequencies
from llmserve_amd.weights import WeightsError, load_model_folder, read_config, write_model_folder
from tests import katenex_cases as cases
from tests.plain import katenex_plain as plain
from tests.torch_kernels import TorchKernels


def runner_for(folder, page=4, pages=64, slots=4, dtype="float32"):
    loaded = load_model_folder(folder, dtype)
    return ModelRunner(loaded, TorchKernels(loaded.dtype), CacheConfig(block_size=page, num_blocks=pages, max_sequences=slots), use_graphs=False)


def oracle(folder, tokens):
    config, tensors = cases.read_folder(folder)
    logits, streams = plain.forward(config, tensors, tokens)
    return logits.float(), streams.float()


def close(got, want, atol=3e-4):
    torch.testing.assert_close(got.float(), want.float(), atol=atol, rtol=3e-4)


# ---------------------------------------------------------------------------- configuration and weights


def test_config_round_trip_and_refusals():
    config = KatenexConfig.from_dict(cases.MIXED)
    assert KatenexConfig.from_dict(config.to_config_json()) == config
    assert config.layers[2].mlp is None and config.layers[3].mixer.left.rot.factor is None and config.streams == 3
    assert config.layers[3].mlp.groups == 1 and config.layers[1].mlp.shared_ff is None
    for path, value in ((("layers", 0, "mlp", "router", "groups", "keep"), 5), (("layers", 1, "mixer", "left", "rot", "dims"), 7),
                        (("layers", 1, "mixer", "right", "blocks"), 3), (("layers", 0, "mlp", "router", "top"), 5)):
        broken = json.loads(json.dumps(cases.MIXED))
        target = broken
        for key in path[:-1]:
            target = target[key]
        target[path[-1]] = value
        with pytest.raises(ConfigError):
            KatenexConfig.from_dict(broken)
    plain_sum = KatenexConfig.from_dict({key: value for key, value in cases.MIXED.items() if key != "streams"})
    assert plain_sum.streams is None and "streams" not in plain_sum.to_config_json()
    assert KatenexConfig.from_dict(plain_sum.to_config_json()) == plain_sum
    without = {key: value for key, value in cases.MIXED.items() if key != "width"}
    with pytest.raises(ConfigError, match="width"):
        KatenexConfig.from_dict(without)


def test_folder_names_and_sizes_left_to_the_tensors(tmp_path):
    folder = cases.write_folder(tmp_path / "m", cases.MIXED, seed=2, drop_ranks=True)
    architecture, config = read_config(folder)
    assert architecture.name == "Katenex" and config.layers[0].mixer.decay_rank is None
    loaded = load_model_folder(folder, "bfloat16")  # the ranks of the low-rank products come from the tensors' shapes
    assert loaded.config.layers[0].mixer.decay_rank == 6 and loaded.config.layers[2].mixer.gate_rank == 7
    names = set(loaded.spec.tensors())
    assert {"embed", "head", "final.norm", "l0.mix.q.conv", "l0.mix.a1", "l0.mix.g2", "l0.mix.dt_bias", "l0.hc1.mix", "l0.hc2.in",
            "l1.mix.left.q", "l1.mix.right.ra.b", "l1.mix.right.conv.b", "l1.mix.right.lam", "l1.mlp.e7.gate", "l0.mlp.shared.gate",
            "l0.mlp.router", "l2.hc1.out"} <= names
    assert "l2.norm2" not in names and "l2.hc2.in" not in names and "l1.mlp.shared.up" not in names and "l0.mlp.correction" not in names
    assert loaded.tensors["l0.mix.A_log"].dtype == torch.bfloat16
    # a folder that still holds what belongs to a feed-forward that is not there is accepted, one with a stranger is not
    tensors = cases.random_tensors(cases.MIXED, 2)
    tensors["l2.norm2"] = torch.ones(32, dtype=torch.bfloat16)
    load_model_folder(cases.write_folder(tmp_path / "n", cases.MIXED, tensors=tensors))
    tensors["l2.mix.bias"] = torch.ones(32, dtype=torch.bfloat16)
    with pytest.raises(WeightsError, match="unexpected"):
        load_model_folder(cases.write_folder(tmp_path / "o", cases.MIXED, tensors=tensors))
    # the seeded random-weights mode writes the same names
    written = write_model_folder(tmp_path / "p", loaded.config, seed=4)
    assert set(cases.read_folder(written)[1]) == names


def test_divided_frequencies():
    got, magnitude = rotary_frequencies(6, 500.0, LinearScaling(4.0))
    want = torch.tensor([500.0 ** (-2.0 * i / 6) / 4.0 for i in range(3)], dtype=torch.float64)
    torch.testing.assert_close(got.double(), want, atol=0, rtol=1e-6)
    assert magnitude == 1.0


# ---------------------------------------------------------------------------- each mechanism in a model of its own

ALONE = {
    "delta": cases.config_of([(cases.delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3), None)]),
    "delta of one tap": cases.config_of([(cases.delta(heads=2, kv_heads=2, dim=8, vdim=8, conv=1, decay_rank=1, gate_rank=2), None)]),
    "delta of one head": cases.config_of([(cases.delta(heads=3, kv_heads=1, dim=24, vdim=40, conv=4), None)], streams=2),
    "parallel": cases.config_of([(cases.parallel(), None)]),
    "parallel, whole heads turned, plain frequencies": cases.config_of(
        [(cases.parallel(cases.attention(2, 2, 8, 16, 0.4, 8, factor=None), cases.recurrence(16, 2, 1)), None)], width=24),
    "parallel without positions, one block": cases.config_of(
        [(cases.parallel(cases.attention(6, 2, 24, 8, 0.2, 0), cases.recurrence(48, 1, 4), 1.0, 1.0), None)], streams=1),
    "experts in groups": cases.config_of([(cases.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2), cases.moe(9, 3, 0.5, 12, 20, (3, 2)))]),
    "experts, every group kept, none shared": cases.config_of([(cases.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=2), cases.moe(6, 3, 2.0, 8, None, (2, 2)))]),
    "one expert a token, no groups": cases.config_of([(cases.parallel(), cases.moe(7, 1, 1.0, 8, 4, None))], streams=4),
    "all experts": cases.config_of([(cases.delta(conv=2), cases.moe(4, 4, 1.0, 8, 12, (4, 4)))]),
    "one copy of the stream": cases.config_of([(cases.delta(), cases.moe()), (cases.parallel(), cases.moe())], streams=1, scale=1.0),
    "the plain residual sum": cases.config_of([(cases.delta(), cases.moe()), (cases.parallel(), None)], streams=None),
}


@pytest.mark.parametrize("name", list(ALONE))
def test_each_mechanism_layer_by_layer(tmp_path, name):
    folder = cases.write_folder(tmp_path / "m", ALONE[name], seed=len(name))
    tokens = cases.tokens_of(19, ALONE[name]["vocab"], seed=5)
    want_logits, want_streams = oracle(folder, tokens)
    runner = runner_for(folder)
    copies = ALONE[name].get("streams") or 1
    seen = []
    runner.model.observer = lambda index, hidden, pending: seen.append(pending.applied(hidden).view(hidden.shape[0], copies, -1).sum(1).clone())
    logits = runner.step([StepEntry("a", tokens, range(len(tokens)))], create_missing=True)
    assert len(seen) == want_streams.shape[0]
    for index, stream in enumerate(seen):
        close(stream, want_streams[index])
    close(logits, want_logits)


def test_what_the_mechanisms_change():
    """On the plain implementation: groups restrict the choice, the links between the copies, the divided frequencies,
    the decay per channel and the recurrence each change the result; so leaving one out would show above."""
    scores = torch.tensor([0.30, 0.01, 0.02, 0.25, 0.24, 0.18], dtype=torch.float64)
    assert plain.choose_experts(scores, 2, 1, 1).tolist() == [0, 3]
    assert plain.choose_experts(scores, 2, 3, 1).tolist() == [0, 1]  # only the best group of two neighbours
    assert plain.choose_experts(scores, 3, 3, 2).tolist() == [0, 3, 2]  # groups 0 and 1 (0.30 and 0.25); 4 and 5 are out
    values = cases.config_of([(cases.parallel(), cases.moe(6, 2, 1.25, 12, 20, (3, 1)))])
    tensors = {name: value.double() for name, value in cases.random_tensors(values, 3).items()}
    tokens = cases.tokens_of(24, values["vocab"], seed=1)
    want, _ = plain.forward(values, tensors, tokens)

    def changed(other_values=None, **other_tensors):
        other, _ = plain.forward(other_values or values, dict(tensors, **other_tensors), tokens)
        return float((other - want).abs().max())

    assert changed(**{"l0.hc1.mix": torch.eye(3, dtype=torch.float64)}) > 0.02
    assert changed(**{"l0.hc2.in": torch.ones(3, dtype=torch.float64)}) > 0.02
    assert changed(**{"l0.mix.right.lam": tensors["l0.mix.right.lam"] + 2.0}) > 0.02
    assert changed(**{"l0.mix.right.conv.b": torch.zeros_like(tensors["l0.mix.right.conv.b"])}) > 0.02
    plain_frequencies = json.loads(json.dumps(values))
    del plain_frequencies["layers"][0]["mixer"]["left"]["rot"]["scaling"]
    assert changed(plain_frequencies) > 0.02
    ungrouped = json.loads(json.dumps(values))
    del ungrouped["layers"][0]["mlp"]["router"]["groups"]
    assert changed(ungrouped) > 0.02
    unscaled = json.loads(json.dumps(values))
    unscaled["embedding"]["scale"] = 1.0
    assert changed(unscaled) > 0.02


# ---------------------------------------------------------------------------- steps, cache and state


@pytest.fixture(scope="module")
def mixed_folder(tmp_path_factory):
    return cases.write_folder(tmp_path_factory.mktemp("katenex") / "mixed", cases.MIXED, seed=7)


@pytest.fixture(scope="module")
def sharp_folder(tmp_path_factory):
    """Attention that looks at one key wherever it is, and states that remember far back."""
    values = cases.config_of(
        [(cases.parallel(cases.attention(2, 1, 8, 16, 2.5, 4, base=50.0, factor=4.0), cases.recurrence(24, 3, 2), 1.0, 0.7), cases.moe(4, 2, 1.0, 8, None, (2, 1))),
         (cases.delta(heads=2, kv_heads=1, dim=16, vdim=8, conv=2), None)],
        vocab=43, width=24, streams=2,
    )
    return cases.write_folder(tmp_path_factory.mktemp("katenex") / "sharp", values, seed=11, sharp=True)


@pytest.mark.parametrize("which", ["mixed", "sharp"])
def test_whole_then_one_by_one_then_portions(mixed_folder, sharp_folder, which):
    folder = mixed_folder if which == "mixed" else sharp_folder
    vocab = cases.read_folder(folder)[0]["vocab"]
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
    """Prompts of one to five tokens, whole and token by token: convolutions that reach before the start, empty states."""
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
    vocab = cases.read_folder(folder)[0]["vocab"]
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
    """One slot, one request after the other: what the first left in the states and kept inputs is gone."""
    runner = runner_for(sharp_folder, slots=1, pages=16)
    first, second = cases.tokens_of(30, 43, seed=1), cases.tokens_of(12, 43, seed=2)
    cases.run_steps(runner, [[("first", 30)]], {"first": first})
    got = cases.run_steps(runner, [[("second", 5)], [("second", 7)]], {"second": second})
    want, _ = oracle(sharp_folder, second)
    close(torch.stack([got[("second", p)] for p in range(12)]), want)


LENGTH = 300
DISTANCES = (1, 15, 16, 17, LENGTH - 1 - 16, LENGTH - 1)


def far_key_case(folder_root):
    """A one-layer model whose attention has large scores, and two tokens (asker, key) such that the asker's answer hangs on
    the one key among hundreds wherever it lies: found by trying seeds and pairs on the plain implementation."""
    mixer = cases.parallel(cases.attention(2, 1, 16, 8, 3.0, 4, base=100.0, factor=2.0), cases.recurrence(16, 2, 2), 1.0, 0.05)
    values = cases.config_of([(mixer, None)], vocab=37, width=24, streams=2)
    for seed in range(1, 40):
        folder = cases.write_folder(folder_root / f"far{seed}", values, seed=seed, sharp=True)
        config, tensors = cases.read_folder(folder)
        for asker in range(31, 37):
            for key in range(31, 37):
                if asker == key:
                    continue
                effects = []
                for distance in DISTANCES:
                    tokens = [1 + (i % 30) for i in range(LENGTH)]
                    tokens[LENGTH - 1 - distance], tokens[-1] = key, asker
                    with_key, _ = plain.forward(config, tensors, tokens)
                    tokens[LENGTH - 1 - distance] = 30
                    without, _ = plain.forward(config, tensors, tokens)
                    effects.append(float((with_key[-1] - without[-1]).abs().max()))
                    if effects[-1] < 0.2:
                        break
                if len(effects) == len(DISTANCES) and min(effects) >= 0.2:
                    return folder, asker, key
    raise AssertionError("no seed gave a key that matters from far away")


def test_one_key_far_away_and_at_page_borders(tmp_path):
    """A query whose answer hangs on one key among hundreds: next to the query, at a page's first and last place, at the
    sequence's first place; in a prompt's portion and decoded alone, with pages of 4 and of 16."""
    folder, asker, key = far_key_case(tmp_path)
    config, tensors = cases.read_folder(folder)
    for distance in DISTANCES:
        tokens = [1 + (i % 30) for i in range(LENGTH)]
        tokens[LENGTH - 1 - distance], tokens[-1] = key, asker
        want, _ = plain.forward(config, tensors, tokens)
        moved = list(tokens)
        moved[LENGTH - 1 - distance] = 30
        other, _ = plain.forward(config, tensors, moved)
        assert float((want[-1] - other[-1]).abs().max()) > 0.05, "the test tests nothing"
        for page in (4, 16):
            runner = runner_for(folder, page=page, pages=160)
            got = cases.run_steps(runner, [[("p", LENGTH)]], {"p": tokens})
            close(got[("p", LENGTH - 1)], want[-1].float())
            got = cases.run_steps(runner, [[("d", 270)], [("d", 13)], [("d", 2)]] + [[("d", 1)]] * 15, {"d": tokens})
            close(got[("d", LENGTH - 1)], want[-1].float())


@pytest.mark.parametrize("kind", ["delta", "recurrence"])
def test_a_token_far_back_stays_in_the_state(tmp_path, kind):
    """States that hardly fade: the first token of 400 still decides the last one's answer."""
    if kind == "delta":
        layers = [(cases.delta(heads=2, kv_heads=1, dim=16, vdim=8, conv=2), None)]
    else:
        layers = [(cases.parallel(cases.attention(1, 1, 8, 8, 0.01, 0), cases.recurrence(24, 2, 3), 0.01, 2.0), None)]
    values = cases.config_of(layers, vocab=37, width=24, streams=2)
    tensors = cases.random_tensors(values, 2, sharp=True)
    if kind == "delta":  # steps so small that hardly anything is forgotten or overwritten
        tensors["l0.mix.dt_bias"] = torch.full_like(tensors["l0.mix.dt_bias"], -4.0)
        tensors["l0.mix.b"] = tensors["l0.mix.b"] * 0.0
    folder = cases.write_folder(tmp_path / "far", values, tensors=tensors)
    config, tensors = cases.read_folder(folder)
    tokens = [1 + (i % 30) for i in range(400)]
    tokens[0] = 35
    want, _ = plain.forward(config, tensors, tokens)
    other, _ = plain.forward(config, tensors, [30] + tokens[1:])
    assert float((want[-1] - other[-1]).abs().max()) > 5e-3
    runner = runner_for(folder, page=16, pages=40)
    got = cases.run_steps(runner, [[("p", 400)]], {"p": tokens})
    close(got[("p", 399)], want[-1].float(), atol=5e-5)  # (a fiftieth of what the first token changes)
    got = cases.run_steps(runner, [[("d", 333)], [("d", 47)]] + [[("d", 1)]] * 20, {"d": tokens})
    close(got[("d", 399)], want[-1].float(), atol=5e-5)


# ---------------------------------------------------------------------------- generation


def greedy(config, tensors, prompt, count):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(torch.argmax(plain.forward(config, tensors, tokens)[0][-1])))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_engine(mixed_folder):
    config, tensors = cases.read_folder(mixed_folder)
    prompts = [cases.tokens_of(n, 67, seed=40 + n) for n in (1, 6, 17, 30)]
    expected = [greedy(config, tensors, prompt, 7) for prompt in prompts]
    runner = runner_for(mixed_folder, page=4, pages=64, slots=4)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=3, max_tokens_per_step=24), prefill_chunk_size=8)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=7)) == expected
    assert runner.cache.used_pages == 0


def test_a_model_without_pages_through_the_scheduler(tmp_path):
    """Only the delta rule: a model that keeps no pages at all generates through the scheduler."""
    values = cases.config_of([(cases.delta(), cases.moe()), (cases.delta(heads=2, kv_heads=2, dim=8, vdim=24, conv=2), None)])
    folder = cases.write_folder(tmp_path / "m", values, seed=5)
    config, tensors = cases.read_folder(folder)
    prompts = [cases.tokens_of(n, 67, seed=60 + n) for n in (3, 11, 20)]
    expected = [greedy(config, tensors, prompt, 5) for prompt in prompts]
    runner = runner_for(folder, page=4, pages=32, slots=3)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=2, max_tokens_per_step=16), prefill_chunk_size=6)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=5)) == expected
    assert len(runner.cache.sequences) == 0


def test_the_command_line_writes_a_random_model_folder(tmp_path, capsys):
    """`llmserve random-model` goes through the registry: a Katenex config.json gives a folder that loads and runs."""
    from llmserve_amd.cli import main

    (tmp_path / "config.json").write_text(json.dumps(cases.MIXED))
    assert main(["random-model", "--config", str(tmp_path / "config.json"), "--output", str(tmp_path / "out"), "--seed", "5", "--std", "0.2"]) == 0
    assert str(tmp_path / "out") in capsys.readouterr().out
    tokens = cases.tokens_of(12, 67, seed=2)
    want, _ = oracle(tmp_path / "out", tokens)
    runner = runner_for(tmp_path / "out")
    close(runner.step([StepEntry("a", tokens, range(12))], create_missing=True), want)
