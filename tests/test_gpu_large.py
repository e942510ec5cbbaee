"""Two layers with the layer sizes of the Llama-3-8B shape (width 4096, 32 heads in 8
groups of head size 128, feed-forward 14336, vocabulary 128256): the kernels that serve
that shape (matrix-core attention for prefill and decode, the weight-streaming product,
the library product, captured decode steps) inside the whole model, against the plain
implementation, in 32-bit and in bfloat16."""
import numpy as np
import pytest
import torch

import common
import plain

pytestmark = pytest.mark.gpu

SHAPE = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=2, hidden_size=4096, num_attention_heads=32,
             num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256,
             max_position_embeddings=8192, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)


SEED = 41


def config():
    from llama_cu_amd.config import LlamaConfig
    return LlamaConfig.from_dict(SHAPE)


def host_weights():
    """The weights of seed SEED as a bfloat16 file would hold them, made on the host.  The engine
    makes its own on the GPU from the same seed (the same bits, as the kernels' tests show); with
    ``stored="bfloat16"`` the 32-bit engine gets the same values widened, so that one plain
    computation serves both compute types."""
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import DecoderModel
    from llama_cu_amd.weights import random_tensors
    return random_tensors(DecoderModel(llama_spec(config())).tensors(), SEED, dtype=torch.bfloat16, device="cpu")


def runner_for(dtype, **kw):
    from llama_cu_amd.engine.runner import ModelRunner
    return ModelRunner.from_config(config(), SEED, dtype=dtype, stored="bfloat16", **kw)


@pytest.fixture(scope="module")
def big():
    reqs = common.random_requests(SHAPE["vocab_size"], [70, 33], seed=3)
    w = host_weights()
    pcfg = plain.PlainConfig.from_dict(SHAPE)
    want = {name: plain.forward(pcfg, w, toks) for name, toks in reqs.items()}
    return {dtype: (None, reqs, want) for dtype in ("float32", "bfloat16")}


# ------------------------------------------------------------------ long contexts through the four traces
LONG = [100, 1300, 2500, 600]


def _kept(name, pos, lens):
    """The positions whose logits are compared: the first and the last 40 of a request, every 61st,
    and the ones around the places where the number of key parts of the decode kernel and the
    pages of a portion change."""
    n = lens[name]
    return pos < 3 or pos >= n - 40 or pos % 61 == 0 or pos in (511, 512, 1023, 1024, 1025, 2047, 2048)


@pytest.fixture(scope="module")
def long_requests():
    reqs = common.random_requests(SHAPE["vocab_size"], LONG, seed=8)
    lens = {k: len(v) for k, v in reqs.items()}
    keep = lambda name, pos: _kept(name, pos, lens)
    w = host_weights()
    pcfg = plain.PlainConfig.from_dict(SHAPE)
    want = {}
    for name, toks in reqs.items():
        at = [p for p in range(len(toks)) if keep(name, p)]
        print(f"plain: request {name}, {len(toks)} tokens, logits at {len(at)} positions", flush=True)
        want[name] = (at, plain.forward(pcfg, w, toks, logits_at=at))
    return reqs, keep, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_long_requests_at_full_layer_sizes_through_the_four_traces(long_requests, dtype, mode):
    """Two layers of the Llama-3-8B shape with random weights from a seed, requests of 100, 1,300,
    2,500 and 600 tokens: whole; with the last 32 tokens decoded one by one (the decode kernel cuts
    2,500 keys into parts, and its steps are replayed from a captured graph); in portions of 1 to
    700 tokens (150 and 200 among them: the widest steps of the kernel that shares the rows through LDS) (prefill over a history of up to 2,000 keys); and mixed, four live requests with a
    pool so small that pages are used again, one of them losing its pages on the way and computed
    again.  Logits at the kept positions against the plain implementation."""
    from llama_cu_amd.engine.trace import TraceReplayer
    reqs, keep, want = long_requests
    if mode == "whole":
        steps, max_tokens = common.trace_whole(reqs, keep=keep)
    elif mode == "tail":
        steps, max_tokens = common.trace_tail_decode(reqs, keep=keep)
    elif mode == "portions":
        steps, max_tokens = common.trace_portions(reqs, sizes=(300, 2, 200, 700, 17, 1, 150, 512, 64, 5), keep=keep)
    else:
        steps, max_tokens = common.trace_mixed(reqs, seed=2, tail=20, sizes=(2, 3, 17, 48, 130, 300, 640), keep=keep,
                                               preempt=0.04)
    print(f"{mode} {dtype}: {len(steps)} steps, max-tokens {max_tokens}", flush=True)
    rep = TraceReplayer(runner_for(dtype, page_size=16, max_tokens=max_tokens, max_seqs=8,
                                   max_batch_tokens=max_tokens, poison_freed=True))
    outputs = {}
    for st in steps:
        out = rep.step(st)
        if out is not None:
            outputs[st["step"]] = out
    rep.runner.cache.check()
    assert rep.runner.cache.free_pages(0) == rep.runner.num_pages
    got = common.collect(steps, outputs, SHAPE["vocab_size"])
    if mode == "mixed":
        assert rep.pages_used_again(0) > 0 and rep.mixed_steps > 0
        assert any(st.get("preempt") for st in steps)
    if mode == "tail" and dtype == "bfloat16":
        assert any(key[0] == 1 and key[1] > 1 for key in rep.runner._graphs), rep.runner._graphs.keys()   # split keys, captured
    rel = common.REL_TOL[dtype]
    for name, (at, ref) in want.items():
        ref = ref.numpy()
        scale = float(np.abs(ref).max())
        assert set(got[name]) == set(at), f"{mode}: request {name}: positions differ"
        for row, pos in enumerate(at):
            err = float(np.abs(got[name][pos].astype(np.float64) - ref[row]).max())
            assert np.isfinite(err) and err <= rel * scale, \
                f"{mode}/{dtype}: request {name}, first wrong position {pos}: error {err:.3e} > {rel * scale:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_portions_and_decoding_at_full_layer_sizes(big, dtype):
    _, reqs, want = big[dtype]
    runner = runner_for(dtype, max_tokens=512, max_seqs=4)
    names = list(reqs)
    ids = {n: i for i, n in enumerate(names)}
    got = {n: {} for n in names}
    # both requests: most of the prompt in one step (together, a mixed batch), ...
    head = {n: len(reqs[n]) - 12 for n in names}
    logits = runner.step([ids[n] for n in names], [reqs[n][:head[n]] for n in names],
                         [list(range(head[n])) for n in names]).cpu().numpy()
    row = 0
    for n in names:
        for p in range(head[n]):
            got[n][p] = logits[row]; row += 1
    # ... then the last 12 tokens one by one, both requests in every step (captured after two)
    for k in range(12):
        logits = runner.step([ids[n] for n in names], [[reqs[n][head[n] + k]] for n in names]).cpu().numpy()
        for i, n in enumerate(names):
            got[n][head[n] + k] = logits[i]
    if dtype == "bfloat16":
        assert any(key[0] == 2 for key in runner._graphs)
    common.assert_matches_plain(got, want, dtype, f"8B-sized layers/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_of_33_to_64_rows_at_full_layer_sizes(big, dtype, monkeypatch):
    """Steps of 40, 39 and 24 rows: in bfloat16 the down projection, and the output projection of the steps of 40
    and 39 rows, leave planes of partial sums to the norm that follows; the output projection of the step of 24 rows
    ends in the residual sum and the second norm's weight, and gate/up, which applies that norm's factor there, ends in
    SwiGLU: all in the kernel that shares the rows through LDS."""
    from llama_cu_amd.engine.runner import ModelRunner
    from llama_cu_amd.kernels import ops
    calls = {"planes": 0, "swiglu": 0, "add_norm": 0}
    real, real_add_norm = ops.gemm_mid, ops.gemm_mid_add_norm

    def counted(*a, **kw):
        calls["swiglu" if kw.get("swiglu") else "planes"] += 1
        return real(*a, **kw)

    def counted_add_norm(*a, **kw):
        calls["add_norm"] += 1
        return real_add_norm(*a, **kw)
    monkeypatch.setattr(ops, "gemm_mid", counted)
    monkeypatch.setattr(ops, "gemm_mid_add_norm", counted_add_norm)
    _, reqs, want = big[dtype]
    runner = runner_for(dtype, max_tokens=512, max_seqs=4)
    r0, r1 = reqs["r0"], reqs["r1"]
    got = {"r0": {}, "r1": {}}
    logits = runner.step([0], [r0[:40]], [list(range(40))]).cpu().numpy()                    # 40 rows
    for p in range(40):
        got["r0"][p] = logits[p]
    logits = runner.step([0, 1], [r0[40:58], r1[:21]], [list(range(18)), list(range(21))]).cpu().numpy()   # 39 rows
    for p in range(18):
        got["r0"][40 + p] = logits[p]
    for p in range(21):
        got["r1"][p] = logits[18 + p]
    logits = runner.step([1, 0], [r1[21:], r0[58:]], [list(range(12)), list(range(12))]).cpu().numpy()     # 24 rows
    for p in range(12):
        got["r1"][21 + p] = logits[p]
        got["r0"][58 + p] = logits[12 + p]
    layers = SHAPE["num_hidden_layers"]
    if dtype == "bfloat16":
        # the down projection of every step leaves planes, the output projection of the steps of 40 and 39 rows too (and
        # the output matrix of those steps is one plane of 32-bit sums); the output projection of the step of 24 rows ends
        # in the residual sum and the second norm's weight
        assert calls == {"planes": 5 * layers + 2, "swiglu": 3 * layers, "add_norm": layers}, calls
    else:
        assert calls == {"planes": 0, "swiglu": 0, "add_norm": 0}
    common.assert_matches_plain(got, want, dtype, f"8B-sized layers, 33 to 64 rows/{dtype}")


def _wide_steps(long_requests, monkeypatch, plan):
    """Runs ``plan`` (a list of steps, each a list of (request index, from, to)) in bfloat16 on the requests of 1,300
    and 600 tokens, compares the kept positions with the plain model and returns how often each kernel of the
    row-sharing product was called."""
    from llama_cu_amd.kernels import ops
    calls = {"planes": 0, "swiglu": 0, "qkv": 0}
    real, real_qkv = ops.gemm_mid, ops.gemm_mid_qkv_rope

    def counted(*a, **kw):
        calls["swiglu" if kw.get("swiglu") else "planes"] += 1
        return real(*a, **kw)

    def counted_qkv(*a, **kw):
        calls["qkv"] += 1
        return real_qkv(*a, **kw)
    monkeypatch.setattr(ops, "gemm_mid", counted)
    monkeypatch.setattr(ops, "gemm_mid_qkv_rope", counted_qkv)
    reqs, keep, want = long_requests
    names = [list(reqs)[1], list(reqs)[3]]          # 1,300 and 600 tokens
    runner = runner_for("bfloat16", max_tokens=1024, max_seqs=4)
    got = {n: {} for n in names}
    for step in plan:
        ids = [names[i] for i, _, _ in step]
        parts = [reqs[names[i]][lo:hi] for i, lo, hi in step]
        wanted = [[k for k in range(hi - lo) if keep(names[i], lo + k)] for i, lo, hi in step]
        logits = runner.step([i for i, _, _ in step], parts, wanted).cpu().numpy()
        row = 0
        for (i, lo, hi), w in zip(step, wanted):
            for k in w:
                got[names[i]][lo + k] = logits[row]; row += 1
    rel = common.REL_TOL["bfloat16"]
    for n in names:
        at, ref = want[n]
        ref = ref.numpy()
        scale = float(np.abs(ref).max())
        seen = 0
        for row, pos in enumerate(at):
            if pos in got[n]:
                err = float(np.abs(got[n][pos].astype(np.float64) - ref[row]).max())
                assert np.isfinite(err) and err <= rel * scale, f"request {n}, position {pos}: error {err:.3e} > {rel * scale:.3e}"
                seen += 1
        assert seen >= 3
    return calls


def test_steps_of_129_to_256_rows_at_full_layer_sizes(long_requests, monkeypatch):
    """Steps of 250, 192 (two requests) and 129 rows in bfloat16: the down projection of each, and the output
    projection up to 192 rows, leave planes of partial sums from the kernel that shares the rows through LDS (its
    ring of two buffers and three or four producer waves), gate/up with SwiGLU and q/k/v with the rotation go there
    up to 192 rows."""
    calls = _wide_steps(long_requests, monkeypatch, [[(0, 0, 250)], [(0, 250, 400), (1, 0, 42)], [(0, 400, 529)]])
    # of the two layers the last one's down projection ends in ordinary rows (the wanted rows are gathered before the
    # final norm): 1 + 0 products in the step of 250 rows, 2 + 1 in each of the others
    # (and gate/up of both layers in the steps of 192 and 129 rows)
    # (and q/k/v of both layers there)
    assert calls == {"planes": 7, "swiglu": 4, "qkv": 4}, calls


def test_steps_of_65_to_128_rows_at_full_layer_sizes(long_requests, monkeypatch):
    """Steps of 100, 128 (two requests) and 65 rows in bfloat16: q/k/v with the rotation and the cache write in the
    epilogue of the kernel that shares the rows through LDS, whose waves share each 128 k (the keys that the later
    steps read were written by it), beside its planes and its SwiGLU."""
    calls = _wide_steps(long_requests, monkeypatch, [[(0, 0, 100)], [(0, 100, 190), (1, 0, 38)], [(1, 38, 103)]])
    layers = SHAPE["num_hidden_layers"]
    assert calls["qkv"] == 3 * layers and calls["swiglu"] >= 3 * (layers - 1) and calls["planes"] >= 3, calls


_plain_rows = {}


def plain_rows_after(prompt, generated):
    """The plain model's logits at the places where the tokens of ``generated`` were chosen, given the prompt and
    the tokens chosen before (computed once per sequence: the engines under test mostly agree)."""
    key = (tuple(prompt), tuple(generated[:-1]))
    if key not in _plain_rows:
        pcfg = plain.PlainConfig.from_dict(SHAPE)
        at = list(range(len(prompt) - 1, len(prompt) - 1 + len(generated)))
        print(f"plain: {len(prompt) + len(generated) - 1} tokens, logits at {len(at)} positions", flush=True)
        _plain_rows[key] = plain.forward(pcfg, host_weights(), list(prompt) + list(generated[:-1]), logits_at=at)
    return _plain_rows[key]


@pytest.mark.parametrize("run_ahead", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_engine_generates_the_plain_models_tokens_at_full_layer_sizes(dtype, run_ahead):
    """The whole engine (scheduler, portions of prompts under a token budget, decoding with captured steps whose
    keys are cut into parts, the arg-max kernel, running ahead with the ids fed on the device, a pool so small that
    a request loses its pages and is computed again) at the layer sizes of the Llama-3-8B shape: prompts of 30,
    1,000 and 1,100 tokens, 48 greedy tokens each, so that two contexts pass 1,024 keys while decoding.  Every
    token is the plain implementation's arg-max given the same tokens before it, or one whose plain logit lies
    within the type's tolerance of the best."""
    from llama_cu_amd.engine.engine import Engine
    rng = np.random.default_rng(12)
    prompts = [[int(t) for t in rng.integers(SHAPE["vocab_size"], size=n)] for n in (30, 1000, 1100)]
    steps = 48
    # at the end the three requests hold 80 + 1,056 + 1,152 tokens' worth of pages: the pool is a little less
    engine = Engine.from_config(config(), SEED, dtype=dtype, stored="bfloat16", page_size=16, max_tokens=2256, max_seqs=4,
                                max_batch_tokens=512, prefill_chunk=384, run_ahead=run_ahead)
    got = engine.generate(prompts, max_steps=steps, ignore_eos=True)
    assert engine.sched.preemptions >= 1, "the pool was meant to be too small"
    engine.runner.cache.check()
    assert engine.runner.cache.free_pages(0) == engine.runner.num_pages
    replayed = {key: n for key, n in engine.runner.graph_replays.items() if n > 0}
    print(f"{dtype}, run_ahead={run_ahead}: {engine.steps} steps, {engine.sched.preemptions} preemptions, replays {replayed}", flush=True)
    if dtype == "bfloat16":
        assert any(key[1] > 1 for key in replayed), replayed           # decode steps with the keys cut into parts, from a graph
    exact = total = 0
    for prompt, out in zip(prompts, got):
        assert len(out) == steps
        logits = plain_rows_after(prompt, out)
        tol = common.REL_TOL[dtype] * float(logits.abs().max())
        for i, tok in enumerate(out):
            best = float(logits[i].max())
            assert float(logits[i][tok]) >= best - tol, \
                f"token {i} after a prompt of {len(prompt)}: logit {float(logits[i][tok])} against the best {best} (tolerance {tol})"
            exact += int(tok == int(torch.argmax(logits[i])))
            total += 1
    print(f"{dtype}, run_ahead={run_ahead}: {exact} of {total} tokens are the plain arg-max", flush=True)
    assert exact >= (0.97 if dtype == "float32" else 0.85) * total, (exact, total)


def test_captured_steps_of_36_requests_equal_eager_ones(big):
    """36 requests decode together: the steps replayed from a captured graph (the kernel for 33 to
    64 rows and its planes of partial sums inside it) give the bits of eager steps on every replay,
    with eager work between the replays."""
    from llama_cu_amd.engine.runner import ModelRunner
    rng = np.random.default_rng(5)
    prompts = [[int(t) for t in rng.integers(SHAPE["vocab_size"], size=3 + i % 5)] for i in range(36)]
    feeds = [[[int(t)] for t in rng.integers(SHAPE["vocab_size"], size=36)] for _ in range(6)]

    def decode(use_graphs):
        runner = runner_for("bfloat16", max_tokens=36 * 32 + 64, max_seqs=40, use_graphs=use_graphs)
        ids = list(range(36))
        runner.step(ids, prompts)
        outs = []
        for i, toks in enumerate(feeds):
            outs.append(runner.step(ids, toks).float().cpu())
            if i == 3:
                runner.step([36], [[1, 2, 3, 4, 5]])
                runner.end(36)
            torch.cuda.synchronize()
        return outs, runner

    eager, _ = decode(False)
    graphed, runner = decode(True)
    assert any(key[0] == 36 for key in runner._graphs)
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.isfinite(a).all()
        assert torch.equal(a, b), f"decode step {i} differs between eager and captured"


def test_the_engines_big_tensors_come_out_of_one_allocation():
    """Weights, their packed copies and the cache are carved out of one allocation of the driver's
    (engine.runner.reserve_in_one_piece): a fresh process builds an engine and asks torch's allocator
    in which of its segments the tensors lie."""
    import os
    import subprocess
    import sys
    script = r'''
import sys
sys.path.insert(0, %r); sys.path.insert(0, %r)
import torch
import llama_cu_amd
from test_gpu_large import runner_for
runner = runner_for("bfloat16", max_tokens=4096, max_seqs=4)
segments = [(s["address"], s["address"] + s["total_size"]) for s in torch.cuda.memory_snapshot()]
def segment_of(t):
    a = t.data_ptr()
    return [i for i, (lo, hi) in enumerate(segments) if lo <= a < hi][0]
layer = runner.model.layers[1]
big = [layer.mixer.w_qkv.plain, layer.mixer.w_qkv.packed, layer.ffn.w_gate_up.plain, layer.ffn.w_gate_up.packed,
       layer.ffn.w_down.packed, runner.model.head.weight.plain, runner.caches[0].pages, runner.caches[1].pages]
assert all(t is not None for t in big)
where = {segment_of(t) for t in big}
print("segments", len(segments), "of the big tensors", sorted(where))
assert len(where) == 1, where
''' % (common.ROOT, os.path.join(common.ROOT, "tests"))
    proc = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-500:] + proc.stderr[-1500:]
