"""The bfloat16 engine against a plain model that rounds where the engine may round.

``plain.forward(..., rounding="bfloat16")`` keeps the residual stream, the sums inside a product, the softmax and the
logits unrounded and rounds what a kernel stores in bfloat16: a norm's output, q, k and v before and after the
rotation, the softmax's weights before they multiply the values, the attention's output, a branch's output, gate, up
and the activation.  Its logits are not the engine's bit for bit and cannot be: a kernel's 32-bit sums come in
another order than the plain 64-bit ones, which flips one rounding in some thousands, the matrix-core attention
rounds its weights relative to a running reference point and not to the row's maximum, and what follows a differing
rounding rounds differently in turn, so after two or three layers the two sets of rounding errors are half
independent (measured: the engine is 0.4 to 1.0 times as far from this model as this model is from the unrounded
one).  What does hold, and tightly, is the size of the error: over all logits of a replay the engine's root mean
square distance from the unrounded plain model is 0.89 to 1.02 times this model's (21 configurations, four ways of
cutting each).  An engine that rounds once more than it may (tried: the residual stream kept in bfloat16 between
the layers) comes out at 1.05 to 1.17 on the narrower models.  So the test asks for at most 1.05, in place of a
fixed tolerance that has to leave room for the widest model; the largest single error is bounded the same way.
"""
import numpy as np
import pytest
import torch

import common
import plain

pytestmark = pytest.mark.gpu

# the thirteen configurations of the search whose largest error lay above 2.5e-2 of the largest logit (by 3 to 27 %),
# and the search's first seventeen
SEEDS = [1129, 1346, 1383, 2038, 2072, 2173, 2269, 6054, 6355, 6579, 5198, 5211, 5263] + list(range(1, 18))

# three of a later search with requests of up to 200 tokens (steps of 129 to 199 rows when a request runs whole), whose
# largest error lay above the fixed bound by 12 to 36 %: the rounding model's own lies there too
LONG_SEEDS = [7095, 7168, 7221]

RMS_RATIO = 1.05
MAX_RATIO = 1.5


def distances(got, unrounded, rounding):
    """Root mean square and largest distance of the engine's logits and of the rounding model's from the unrounded
    model's, over all requests and positions."""
    e, r = [], []
    for name, ref in unrounded.items():
        ref = ref.numpy()
        assert set(got.get(name, {})) == set(range(ref.shape[0])), f"request {name}: positions missing"
        g = np.stack([got[name][p] for p in range(ref.shape[0])]).astype(np.float64)
        assert np.isfinite(g).all()
        e.append((g - ref).ravel())
        r.append((rounding[name].numpy() - ref).ravel())
    e, r = np.concatenate(e), np.concatenate(r)
    rms = lambda a: float(np.sqrt((a * a).mean()))
    return rms(e), rms(r), float(np.abs(e).max()), float(np.abs(r).max())


@pytest.mark.parametrize("seed", SEEDS + LONG_SEEDS)
def test_bfloat16_engine_errs_no_more_than_a_model_that_rounds_where_it_may(seed):
    cfg, page, lens = common.sweep_configuration(seed, lens_max=200 if seed in LONG_SEEDS else 140)
    folder = common.make_folder(cfg, seed=seed, dtype=torch.bfloat16, std=common.BF16_STD)
    reqs = common.random_requests(cfg["vocab_size"], lens, seed=seed)
    pcfg, w = plain.load_folder(folder)
    unrounded = {n: plain.forward(pcfg, w, t) for n, t in reqs.items()}
    rounding = {n: plain.forward(pcfg, w, t, rounding="bfloat16") for n, t in reqs.items()}
    traces = {"whole": common.trace_whole, "tail": common.trace_tail_decode, "portions": common.trace_portions,
              "mixed": lambda r, page: common.trace_mixed(r, seed=1, page=page)}
    for mode, make in traces.items():
        steps, max_tokens = make(reqs, page=page)
        outputs = common.run_trace_inprocess(folder, "bfloat16", steps, max_tokens, page_size=page)
        got = common.collect(steps, outputs, cfg["vocab_size"])
        e_rms, r_rms, e_max, r_max = distances(got, unrounded, rounding)
        what = f"seed {seed}, pages of {page}, {mode}: {cfg}"
        assert e_rms <= RMS_RATIO * r_rms, f"{what}: root mean square error {e_rms:.3e} against the rounding model's {r_rms:.3e}"
        assert e_max <= MAX_RATIO * r_max, f"{what}: largest error {e_max:.3e} against the rounding model's {r_max:.3e}"
