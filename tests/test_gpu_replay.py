"""The engine against the plain implementation, by trace replay: each request alone and
whole; most of it in one step and the last 32 tokens one by one; in portions of changing
size; and mixed, up to four live requests with so few pages that they are used again.
In 32-bit and in bfloat16, for tiny configurations that differ in every size and option."""
import pytest
import torch

import common

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 33, 70, 128, 40], "B": [1, 40, 97, 130, 256, 66], "C": [2, 65, 150, 31, 200]}


@pytest.fixture(scope="module")
def models():
    out = {}
    for name, cfg in common.TINY.items():
        for dtype, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
            folder = common.make_folder(cfg, seed=11 + len(out), dtype=tdt,
                                        std=common.BF16_STD if dtype == "bfloat16" else 0.15)
            reqs = common.random_requests(cfg["vocab_size"], LENGTHS[name], seed=5)
            out[(name, dtype)] = (folder, reqs, common.plain_logits(folder, reqs))
    return out


TRACES = {"whole": common.trace_whole, "tail": common.trace_tail_decode, "portions": common.trace_portions,
          "mixed": common.trace_mixed}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(models, name, dtype, mode):
    folder, reqs, want = models[(name, dtype)]
    steps, max_tokens = TRACES[mode](reqs)
    vocab = common.TINY[name]["vocab_size"]
    print(f"replay {name} {dtype} {mode}: {len(steps)} steps, max-tokens {max_tokens}", flush=True)
    outputs = common.run_trace_inprocess(folder, dtype, steps, max_tokens)
    got = common.collect(steps, outputs, vocab)
    common.assert_matches_plain(got, want, dtype, f"{name}/{dtype}/{mode}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, dtype):
    """The program itself, as a user starts it: mixed trace, files and ``done`` lines."""
    folder, reqs, want = models[("A", dtype)]
    steps, max_tokens = common.trace_mixed(reqs, seed=3)
    outputs = common.run_trace_program(folder, dtype, steps, max_tokens, common.TINY_A["vocab_size"])
    got = common.collect(steps, outputs, common.TINY_A["vocab_size"])
    common.assert_matches_plain(got, want, dtype, f"trace_run/{dtype}")


def test_float32_does_not_depend_on_cutting(models):
    """In 32-bit every kernel adds in an order that the cutting does not change: the
    logits of the four ways of running agree to the last bit."""
    import numpy as np
    folder, reqs, _ = models[("B", "float32")]
    vocab = common.TINY_B["vocab_size"]
    results = []
    for mode in ("whole", "tail", "portions", "mixed"):
        steps, max_tokens = TRACES[mode](reqs)
        results.append(common.collect(steps, common.run_trace_inprocess(folder, "float32", steps, max_tokens), vocab))
    for other in results[1:]:
        for name in reqs:
            for pos in results[0][name]:
                assert np.array_equal(results[0][name][pos], other[name][pos]), (name, pos)
