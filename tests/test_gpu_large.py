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


@pytest.fixture(scope="module")
def big():
    out = {}
    reqs = common.random_requests(SHAPE["vocab_size"], [70, 33], seed=3)
    for dtype, tdt, std in (("float32", torch.float32, 0.02), ("bfloat16", torch.bfloat16, 0.02)):
        folder = common.make_folder(SHAPE, seed=41, dtype=tdt, std=std)
        out[dtype] = (folder, reqs, common.plain_logits(folder, reqs))
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_portions_and_decoding_at_full_layer_sizes(big, dtype):
    from llama_cu_amd.engine.runner import ModelRunner
    folder, reqs, want = big[dtype]
    runner = ModelRunner.from_folder(folder, dtype=dtype, max_tokens=512, max_seqs=4)
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
    """Steps of 40 and 39 rows: in bfloat16 the output and down projections leave planes of partial
    sums to the norm that follows, and gate/up ends in SwiGLU, in the kernel that shares the rows
    through LDS; in the step of 24 rows gate/up (with the norm's factor in its epilogue) and the down
    projection go there."""
    from llama_cu_amd.engine.runner import ModelRunner
    from llama_cu_amd.kernels import ops
    calls = {"planes": 0, "swiglu": 0}
    real = ops.gemm_mid

    def counted(*a, **kw):
        calls["swiglu" if kw.get("swiglu") else "planes"] += 1
        return real(*a, **kw)
    monkeypatch.setattr(ops, "gemm_mid", counted)
    folder, reqs, want = big[dtype]
    runner = ModelRunner.from_folder(folder, dtype=dtype, max_tokens=512, max_seqs=4)
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
        assert calls["planes"] == 5 * layers and calls["swiglu"] == 3 * layers, calls
    else:
        assert calls == {"planes": 0, "swiglu": 0}
    common.assert_matches_plain(got, want, dtype, f"8B-sized layers, 33 to 64 rows/{dtype}")


def test_captured_steps_of_36_requests_equal_eager_ones(big):
    """36 requests decode together: the steps replayed from a captured graph (the kernel for 33 to
    64 rows and its planes of partial sums inside it) give the bits of eager steps on every replay,
    with eager work between the replays."""
    from llama_cu_amd.engine.runner import ModelRunner
    folder = big["bfloat16"][0]
    rng = np.random.default_rng(5)
    prompts = [[int(t) for t in rng.integers(SHAPE["vocab_size"], size=3 + i % 5)] for i in range(36)]
    feeds = [[[int(t)] for t in rng.integers(SHAPE["vocab_size"], size=36)] for _ in range(6)]

    def decode(use_graphs):
        runner = ModelRunner.from_folder(folder, dtype="bfloat16", max_tokens=36 * 32 + 64, max_seqs=40, use_graphs=use_graphs)
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
