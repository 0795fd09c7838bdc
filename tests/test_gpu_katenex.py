"""The Katenex decoder on the GPU, through the engine's runner, scheduler and trace replay, against the plain
implementation: float32 tightly, bfloat16 within what rounding allows."""

from __future__ import annotations

import pytest
import torch

from llmserve_amd import CacheConfig, GenerationConfig, SchedulerConfig
from llmserve_amd.engine import EngineCore, ModelRunner
from llmserve_amd.weights import load_model_folder
from tests import katenex_cases as cases
from tests.gpu_helpers import TraceBuilder, replay
from tests.plain import katenex_plain as plain
from tests.test_katenex import DISTANCES, LENGTH, far_key_case, greedy

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def kernels():
    from llmserve_amd.kernels import HipKernels

    return {"float32": HipKernels(torch.float32), "bfloat16": HipKernels(torch.bfloat16)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("katenex_gpu")
    sharp = cases.config_of(
        [(cases.parallel(cases.attention(2, 1, 8, 16, 2.5, 4, base=50.0, factor=4.0), cases.recurrence(24, 3, 2), 1.0, 0.7), cases.moe(4, 2, 1.0, 8, None, (2, 1))),
         (cases.delta(heads=2, kv_heads=1, dim=16, vdim=8, conv=2), None)],
        vocab=43, width=24, streams=2,
    )
    # sizes the matrix-core kernels take (heads of 64 and 128, experts in steps of 32) beside the odd ones of the other two
    wide = cases.config_of(
        [
            (cases.delta(heads=4, kv_heads=2, dim=64, vdim=128, conv=4, decay_rank=16, gate_rank=24), cases.moe(8, 2, 1.5, 64, 128, (4, 2))),
            (cases.parallel(cases.attention(8, 2, 128, 64, 0.09, 64, base=10000.0, factor=8.0), cases.recurrence(384, 6, 4), 1.1, 0.6),
             cases.moe(16, 4, 2.0, 32, 96, (4, 3))),
            (cases.delta(heads=2, kv_heads=2, dim=128, vdim=64, conv=2, decay_rank=8, gate_rank=8), None),
            (cases.parallel(cases.attention(4, 4, 64, 64, 0.125, 32, factor=None), cases.recurrence(256, 1, 3), 0.7, 1.4), cases.moe(6, 6, 1.0, 96, None, None)),
        ],
        vocab=300, width=256, streams=4,
    )
    return {
        "mixed": cases.write_folder(root / "mixed", cases.MIXED, seed=7),
        "sharp": cases.write_folder(root / "sharp", sharp, seed=11, sharp=True),
        "wide": cases.write_folder(root / "wide", wide, seed=13),
        "mixed with every expert": cases.write_folder(root / "mixed_every", cases.with_every_expert(cases.MIXED), seed=7),
        "wide with every expert": cases.write_folder(root / "wide_every", cases.with_every_expert(wide), seed=13),
    }


def runner_for(folder, kernels, dtype, page=16, pages=64, slots=4, longest=None):
    loaded = load_model_folder(folder, dtype)
    return ModelRunner(loaded, kernels[dtype], CacheConfig(block_size=page, num_blocks=pages, max_sequences=slots), max_sequence_length=longest)


def agree(got, want, dtype):
    """float32: element by element.  bfloat16: the error of a row, mean taken off, is small beside the row's own
    spread, at the median and in every row."""
    got, want = got.float(), want.float()
    if dtype == "float32":
        torch.testing.assert_close(got, want, atol=1e-3, rtol=1e-3)
        return
    error = (got - want) - (got - want).mean(-1, keepdim=True)
    spread = want - want.mean(-1, keepdim=True)
    ratio = error.pow(2).mean(-1).sqrt() / spread.pow(2).mean(-1).sqrt()
    assert float(ratio.median()) < 0.05, f"bfloat16 rows differ by {float(ratio.median()):.3f} of their spread at the median"
    assert float(ratio.max()) < 0.15, f"a bfloat16 row differs by {float(ratio.max()):.3f} of its spread"


def spread_ratio(got, want):
    got, want = got.float(), want.float()
    error = (got - want) - (got - want).mean(-1, keepdim=True)
    spread = want - want.mean(-1, keepdim=True)
    return error.pow(2).mean(-1).sqrt() / spread.pow(2).mean(-1).sqrt()


def oracle(folder, tokens):
    config, tensors = cases.read_folder(folder)
    return plain.forward(config, tensors, tokens)[0]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["mixed", "sharp", "wide"])
def test_whole_then_one_by_one_then_portions(folders, kernels, dtype, which):
    if which == "sharp" and dtype == "bfloat16":
        pytest.skip("attention that looks at one key amplifies rounding: this model is for the 32-bit run")
    folder = folders[which]
    vocab = cases.read_folder(folder)[0]["vocab"]
    tokens = cases.tokens_of(150, vocab, seed=3)
    want = oracle(folder, tokens)
    runner = runner_for(folder, kernels, dtype, page=16, pages=40)
    prompts = {"whole": tokens, "tail": tokens, "cut": tokens, "pairs": tokens[:40]}
    got = cases.run_steps(runner, [[("whole", 150)]], prompts)
    agree(torch.stack([got[("whole", p)] for p in range(150)]), want, dtype)
    got = cases.run_steps(runner, [[("tail", 61)]] + [[("tail", 1)]] * 89, prompts)
    agree(torch.stack([got[("tail", p)] for p in range(150)]), want, dtype)
    sizes = [7, 2, 16, 3, 2, 1, 25, 1, 14, 2, 2, 9, 33, 2, 31]
    got = cases.run_steps(runner, [[("cut", n)] for n in sizes], prompts)
    agree(torch.stack([got[("cut", p)] for p in range(150)]), want, dtype)
    got = cases.run_steps(runner, [[("pairs", 2)]] * 20, prompts)
    agree(torch.stack([got[("pairs", p)] for p in range(40)]), want[:40], dtype)
    assert runner.cache.used_pages == 0
    runner.close()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens_of_a_sequence(folders, kernels, dtype):
    runner = runner_for(folders["mixed"], kernels, dtype)
    for length in (1, 2, 3, 5):
        tokens = cases.tokens_of(length, 67, seed=length)
        want = oracle(folders["mixed"], tokens)
        got = cases.run_steps(runner, [[("w", length)]], {"w": tokens})
        agree(torch.stack([got[("w", p)] for p in range(length)]), want, dtype)
        got = cases.run_steps(runner, [[("s", 1)]] * length, {"s": tokens})
        agree(torch.stack([got[("s", p)] for p in range(length)]), want, dtype)
    runner.close()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("every", [False, True])
@pytest.mark.parametrize("which", ["mixed", "wide"])
def test_mixed_batches_with_pages_and_slots_used_again(folders, kernels, dtype, which, every):
    """`every`: each token uses all experts of its layer (weighted by the router all the same)."""
    folder = folders[which + (" with every expert" if every else "")]
    vocab = cases.read_folder(folder)[0]["vocab"]
    lengths = {"a": 45, "b": 9, "c": 30, "d": 61, "e": 1, "f": 26, "g": 40}
    prompts = {name: cases.tokens_of(n, vocab, seed=20 + n) for name, n in lengths.items()}
    want = {name: oracle(folder, prompts[name]) for name in prompts}
    page = 8
    runner = runner_for(folder, kernels, dtype, page=page, pages=16, slots=3)
    generator = torch.Generator().manual_seed(5)
    done = dict.fromkeys(prompts, 0)
    waiting, live, step_number, at, rows, keys = list(prompts), [], 0, {}, [], []
    while waiting or live:
        while waiting and len(live) < 3 and sum(-(-lengths[n] // page) for n in live + [waiting[0]]) <= 16:
            live.append(waiting.pop(0))
        step = []
        for name in live:
            if len(live) > 1 and step_number % 5 == 3 and name == live[0]:
                continue
            left = lengths[name] - done[name]
            count = 1 if done[name] > lengths[name] // 2 else min(left, int(torch.randint(2, 13, (1,), generator=generator)))
            step.append((name, count))
            done[name] += count
        for (name, position), row in cases.run_steps(runner, [step], prompts, at).items():
            rows.append((row, want[name][position]))
            keys.append((name, position))
        live = [name for name in live if done[name] < lengths[name]]
        step_number += 1
    assert runner.cache.used_pages == 0 and len(runner.cache.sequences) == 0
    assert runner.step_counts["replayed"] > 0  # steps of one shape came back and were replayed from their graph
    runner.close()
    got, wanted = torch.stack([row for row, _ in rows]), torch.stack([row for _, row in rows])
    if dtype == "bfloat16" and not every:
        # where rounding turns a router's close call the other way, a row (and, through the states, the rows behind it)
        # leaves the plain implementation's: only the median is held against it; the models whose tokens use every
        # expert have no such choice, and their rows agree one by one
        assert float(spread_ratio(got, wanted).median()) < 0.05
        return
    agree(got, wanted, dtype)


def test_one_key_far_away_and_at_page_borders(tmp_path, kernels):
    folder, asker, key = far_key_case(tmp_path)
    config, tensors = cases.read_folder(folder)
    for distance in DISTANCES:
        tokens = [1 + (i % 30) for i in range(LENGTH)]
        tokens[LENGTH - 1 - distance], tokens[-1] = key, asker
        want, _ = plain.forward(config, tensors, tokens)
        runner = runner_for(folder, kernels, "float32", page=16, pages=40)
        got = cases.run_steps(runner, [[("p", LENGTH)]], {"p": tokens})
        agree(got[("p", LENGTH - 1)][None], want[-1][None], "float32")
        got = cases.run_steps(runner, [[("d", 270)], [("d", 13)], [("d", 2)]] + [[("d", 1)]] * 15, {"d": tokens})
        agree(got[("d", LENGTH - 1)][None], want[-1][None], "float32")
        runner.close()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["delta", "recurrence"])
def test_a_token_far_back_stays_in_the_state(tmp_path, kernels, dtype, kind):
    if kind == "delta":
        layers = [(cases.delta(heads=2, kv_heads=1, dim=16, vdim=8, conv=2), None)]
    else:
        layers = [(cases.parallel(cases.attention(1, 1, 8, 8, 0.01, 0), cases.recurrence(24, 2, 3), 0.01, 2.0), None)]
    values = cases.config_of(layers, vocab=37, width=24, streams=2)
    tensors = cases.random_tensors(values, 2, sharp=True)
    if kind == "delta":
        tensors["l0.mix.dt_bias"] = torch.full_like(tensors["l0.mix.dt_bias"], -4.0)
        tensors["l0.mix.b"] = tensors["l0.mix.b"] * 0.0
    folder = cases.write_folder(tmp_path / "far", values, tensors=tensors)
    tokens = [1 + (i % 30) for i in range(400)]
    tokens[0] = 35
    want = oracle(folder, tokens)
    runner = runner_for(folder, kernels, dtype, page=16, pages=40)
    got = cases.run_steps(runner, [[("p", 400)]], {"p": tokens})
    agree(got[("p", 399)][None], want[-1][None], dtype)
    got = cases.run_steps(runner, [[("d", 333)], [("d", 47)]] + [[("d", 1)]] * 20, {"d": tokens})
    agree(got[("d", 399)][None], want[-1][None], dtype)
    runner.close()


def test_greedy_generation_through_the_engine(folders, kernels):
    config, tensors = cases.read_folder(folders["mixed"])
    prompts = [cases.tokens_of(n, 67, seed=40 + n) for n in (1, 6, 17, 30)]
    expected = [greedy(config, tensors, prompt, 12) for prompt in prompts]
    runner = runner_for(folders["mixed"], kernels, "float32", page=16, pages=32, slots=4)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=3, max_tokens_per_step=24), prefill_chunk_size=8)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=12)) == expected
    assert runner.cache.used_pages == 0
    runner.close()


def test_a_model_without_pages_through_the_scheduler(tmp_path, kernels):
    values = cases.config_of([(cases.delta(), cases.moe()), (cases.delta(heads=2, kv_heads=2, dim=8, vdim=24, conv=2), None)])
    folder = cases.write_folder(tmp_path / "m", values, seed=5)
    config, tensors = cases.read_folder(folder)
    prompts = [cases.tokens_of(n, 67, seed=60 + n) for n in (3, 11, 20)]
    expected = [greedy(config, tensors, prompt, 9) for prompt in prompts]
    runner = runner_for(folder, kernels, "float32", page=16, pages=16, slots=3)
    core = EngineCore(runner, SchedulerConfig(max_batch_size=2, max_tokens_per_step=16), prefill_chunk_size=6)
    assert core.generate(prompts, GenerationConfig(max_new_tokens=9)) == expected
    assert len(runner.cache.sequences) == 0
    runner.close()


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay(folders, tmp_path, dtype):
    """bin/trace_run: portions beside single tokens, a request that pauses, slots used again."""
    vocab = cases.read_folder(folders["wide"])[0]["vocab"]
    prompts = {name: cases.tokens_of(n, vocab, seed=n) for name, n in {"a": 70, "b": 23, "c": 5, "d": 33, "e": 64}.items()}
    want = {name: oracle(folders["wide"], tokens) for name, tokens in prompts.items()}
    trace = TraceBuilder()
    trace.step([("a", prompts["a"][:40]), ("b", prompts["b"][:2])])
    trace.step([("a", prompts["a"][40:41]), ("b", prompts["b"][2:20]), ("c", prompts["c"])], end=["c"])
    trace.step([("a", prompts["a"][41:42]), ("d", prompts["d"][:30])])
    trace.step([("b", prompts["b"][20:]), ("a", prompts["a"][42:70]), ("d", prompts["d"][30:31])], end=["a", "b"])
    trace.step([("d", prompts["d"][31:32]), ("e", prompts["e"])], end=["e"])
    trace.step([("d", prompts["d"][32:])], end=["d"])
    found = trace.collect(replay(folders["wide"], dtype, trace.steps, tmp_path / "out", max_tokens=256, block_size=16, vocab=vocab))
    assert len(found) == sum(len(tokens) for tokens in prompts.values())
    keys = sorted(found)
    agree(torch.stack([found[key] for key in keys]), torch.stack([want[name][position] for name, position in keys]), dtype)
