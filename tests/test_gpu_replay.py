"""The engine against the plain implementation, by trace replay: each request alone and
whole; most of it in one step and the last 32 tokens one by one; in portions of changing
size; and mixed, up to four live requests with so few pages that they are used again.
In 32-bit and in bfloat16, for tiny configurations that differ in every size and option."""
import pytest
import torch

import common

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 33, 70, 128, 40], "B": [1, 40, 97, 130, 256, 66], "C": [2, 65, 150, 31, 200],
           "D": [40, 100, 128, 70, 33]}
# tokens per page of the cache: each configuration has its own (A and B the ones their workloads name)
PAGE = {"A": 16, "B": 32, "C": 48, "D": 64}


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
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(models, name, dtype, mode, monkeypatch):
    folder, reqs, want = models[(name, dtype)]
    steps, max_tokens = TRACES[mode](reqs, page=PAGE[name])
    vocab = common.TINY[name]["vocab_size"]
    print(f"replay {name} {dtype} {mode}: {len(steps)} steps, max-tokens {max_tokens}, pages of {PAGE[name]}", flush=True)
    calls = []
    if name == "D" and dtype == "bfloat16":
        from llama_cu_amd.kernels import ops
        real = ops.gemm_mid
        monkeypatch.setattr(ops, "gemm_mid", lambda *a, **kw: (calls.append(a[0].shape[0]), real(*a, **kw))[1])
    stats = {}
    outputs = common.run_trace_inprocess(folder, dtype, steps, max_tokens, stats=stats, page_size=PAGE[name])
    got = common.collect(steps, outputs, vocab)
    common.assert_matches_plain(got, want, dtype, f"{name}/{dtype}/{mode}")
    if mode == "mixed":
        # the pool is so small that pages went from one request to another, and portions stood beside single tokens
        assert stats["pages_used_again"] > 0 and stats["mixed_steps"] > 0, stats
    if name == "D" and dtype == "bfloat16" and mode in ("whole", "mixed"):
        assert calls and all(32 < rows <= 128 for rows in calls), calls      # the planes of partial sums were in it


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, dtype):
    """The program itself, as a user starts it: mixed trace, files and ``done`` lines."""
    folder, reqs, want = models[("A", dtype)]
    steps, max_tokens = common.trace_mixed(reqs, seed=3)
    outputs = common.run_trace_program(folder, dtype, steps, max_tokens, common.TINY_A["vocab_size"])
    got = common.collect(steps, outputs, common.TINY_A["vocab_size"])
    common.assert_matches_plain(got, want, dtype, f"trace_run/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_with_requests_that_lose_their_pages_and_are_computed_again(models, dtype):
    """``"preempt": [name]`` in a step: the request's pages are given back, and the next step that
    names it computes all its earlier tokens again beside its new ones, in one batch with the
    other requests.  The logits are those of the plain implementation all the same."""
    folder, reqs, want = models[("B", dtype)]
    steps, max_tokens = common.trace_mixed(reqs, seed=7, preempt=0.2, page=PAGE["B"])
    assert sum(len(s.get("preempt", [])) for s in steps) >= 3
    stats = {}
    outputs = common.run_trace_inprocess(folder, dtype, steps, max_tokens, stats=stats, page_size=PAGE["B"])
    got = common.collect(steps, outputs, common.TINY_B["vocab_size"])
    common.assert_matches_plain(got, want, dtype, f"preempted/{dtype}")
    assert stats["pages_used_again"] > 0


def test_trace_run_program_with_weights_from_a_seed_and_its_own_pages(tmp_path):
    """``--random-weights SEED``: the folder holds config.json only and the weights are made on the
    GPU; the plain implementation gets the weights of the same seed made on the host.  Pages of 32
    tokens and a pool given in pages."""
    import json
    import os
    import plain
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import DecoderModel
    from llama_cu_amd.weights import random_tensors
    with open(tmp_path / "config.json", "w") as f:
        json.dump(common.TINY_B, f)
    spec = llama_spec(LlamaConfig.from_dict(common.TINY_B))
    w = random_tensors(DecoderModel(spec).tensors(), 5, dtype=torch.float32, device="cpu", std=0.02)
    reqs = common.random_requests(common.TINY_B["vocab_size"], [40, 97, 130, 66], seed=9)
    pcfg = plain.PlainConfig.from_dict(common.TINY_B)
    want = {name: plain.forward(pcfg, w, toks) for name, toks in reqs.items()}
    steps, max_tokens = common.trace_mixed(reqs, seed=4)
    outputs = common.run_trace_program(str(tmp_path), "float32", steps, max_tokens, common.TINY_B["vocab_size"],
                                       extra=["--random-weights", "5", "--page-size", "32", "--num-pages", str(max_tokens // 32),
                                              "--max-live", "4", "--poison-freed"])
    got = common.collect(steps, outputs, common.TINY_B["vocab_size"])
    common.assert_matches_plain(got, want, "float32", "trace_run --random-weights")
    assert not os.path.exists(tmp_path / "model.safetensors")


def test_float32_does_not_depend_on_cutting(models):
    """In 32-bit every kernel adds in an order that the cutting does not change: the
    logits of the four ways of running agree to the last bit."""
    import numpy as np
    folder, reqs, _ = models[("B", "float32")]
    vocab = common.TINY_B["vocab_size"]
    results = []
    for mode, page in (("whole", 32), ("tail", 16), ("portions", 64), ("mixed", 32)):     # nor on the pages' size
        steps, max_tokens = TRACES[mode](reqs, page=page)
        results.append(common.collect(steps, common.run_trace_inprocess(folder, "float32", steps, max_tokens, page_size=page), vocab))
    for other in results[1:]:
        for name in reqs:
            for pos in results[0][name]:
                assert np.array_equal(results[0][name][pos], other[name][pos]), (name, pos)


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 101, 102, 103])
def test_random_configurations_match_plain(seed):
    """Configurations drawn at random from what config.json allows: head sizes in steps of 16
    up to 256, any number of heads and groups, widths and vocabularies that are no power of
    two, both pairings of the rotation, tied and untied output; replayed whole, with a decoded
    tail, in portions and mixed, in 32-bit and in bfloat16."""
    import random
    rng = random.Random(seed)
    nkv = rng.choice([1, 2, 3, 5])
    # seeds from 100 on: widths of whole blocks of 128, for which the matrices get the copy that the decode
    # kernels stream, with intermediate sizes that are and are not whole blocks of 16
    widths, inner = ([40, 72, 88, 104, 136, 200, 264], [56, 100, 172, 232, 352]) if seed < 100 else ([128, 256], [56, 104, 128, 172])
    cfg = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=rng.choice([1, 2]),
               hidden_size=rng.choice(widths), num_attention_heads=nkv * rng.choice([1, 2, 3, 4, 7, 8]),
               num_key_value_heads=nkv, head_dim=rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 192, 256]),
               intermediate_size=rng.choice(inner), vocab_size=rng.choice([257, 301, 384, 1000, 1537]),
               max_position_embeddings=256, rope_theta=rng.choice([1e4, 5e5, 333.0]),
               rms_norm_eps=rng.choice([1e-5, 1e-6, 1e-3]), tie_word_embeddings=rng.random() < 0.5,
               rope_interleaved=rng.random() < 0.3)
    lens = [rng.randrange(1, 150) for _ in range(4)]
    page = rng.choice([16, 32, 48, 64, 128])
    for dtype, tdt, std in (("float32", torch.float32, 0.15), ("bfloat16", torch.bfloat16, common.BF16_STD)):
        folder = common.make_folder(cfg, seed=seed, dtype=tdt, std=std)
        reqs = common.random_requests(cfg["vocab_size"], lens, seed=seed)
        want = common.plain_logits(folder, reqs)
        for mode in ("whole", "tail", "portions", "mixed"):
            steps, max_tokens = TRACES[mode](reqs, page=page)
            outputs = common.run_trace_inprocess(folder, dtype, steps, max_tokens, page_size=page)
            got = common.collect(steps, outputs, cfg["vocab_size"])
            common.assert_matches_plain(got, want, dtype, f"{cfg}/pages of {page}/{dtype}/{mode}")
