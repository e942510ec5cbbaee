"""Generation through the entry points: greedy tokens equal the plain implementation's;
seeded temperature sampling equals the plain sampler drawing from the plain logits;
scheduling decisions (portions, few pages, preemption) change no token."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import common
import plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folder_a():
    return common.make_folder(common.TINY_A, seed=21, dtype=torch.float32)


@pytest.fixture(scope="module")
def folder_b():
    return common.make_folder(common.TINY_B, seed=22, dtype=torch.float32)


def test_greedy_generation_through_the_python_entry_point(folder_a):
    """Tiny A's workload: prompts of 5, 17 and 33 tokens, 16 greedy steps each."""
    import llama_cu_amd
    reqs = common.random_requests(256, [5, 17, 33], seed=1)
    cfg, w = plain.load_folder(folder_a)
    want = [plain.greedy_generate(cfg, w, p, 16) for p in reqs.values()]
    got = llama_cu_amd.generate(folder_a, list(reqs.values()), max_steps=16, dtype="float32", max_tokens=512, max_seqs=4)
    assert got == want


def test_seeded_temperature_sampling_with_portions(folder_b):
    """Tiny B's workload: prompts of 1, 40, 97 and 130 tokens in portions of 48, 24 steps
    at temperature 0.8 with a fixed seed.  The plain side draws with the same uniform
    numbers from its own logits; a token is accepted as equal, or as a near tie (the two
    candidates' cumulative weights straddle the drawn number within rounding)."""
    import llama_cu_amd
    from llama_cu_amd.engine.engine import Engine
    from llama_cu_amd.sampling import SamplingParams, uniform
    reqs = list(common.random_requests(384, [1, 40, 97, 130], seed=2).values())
    params = SamplingParams(temperature=0.8, seed=1234)
    engine = Engine.from_folder(folder_b, dtype="float32", max_tokens=1024, max_seqs=4, max_batch_tokens=64,
                                prefill_chunk=48, page_size=32)
    got = engine.generate(reqs, params, max_steps=24, ignore_eos=True)
    cfg, w = plain.load_folder(folder_b)
    for rid, (prompt, out) in enumerate(zip(reqs, got)):
        toks = list(prompt)
        assert len(out) == 24
        for tok in out:
            logits = plain.forward(cfg, w, toks)[-1]
            u = uniform(1234, rid, len(toks))
            want = plain.sample(logits, 0.8, 1.0, 10 ** 9, u)
            if tok != want:
                # a near tie: u falls within rounding of the boundary between the two
                lo = plain.sample(logits, 0.8, 1.0, 10 ** 9, max(u - 1e-5, 0.0))
                hi = plain.sample(logits, 0.8, 1.0, 10 ** 9, min(u + 1e-5, 1 - 1e-9))
                assert tok in (lo, hi), (rid, len(toks), tok, want)
            toks.append(tok)          # follow the engine's choice
    # the same seed gives the same tokens when the requests run alone (another batch)
    engine2 = Engine.from_folder(folder_b, dtype="float32", max_tokens=512, max_seqs=1, page_size=16)
    for rid, prompt in enumerate(reqs):
        rid2 = engine2.add_request(prompt, params, 24, req_id=rid, ignore_eos=True)
        out = []
        while not engine2.idle:
            out += [o.token for o in engine2.step() if o.token is not None]
        engine2.drop(rid2)
        assert out == got[rid]


def test_the_entry_point_gives_the_same_draws_on_every_call_and_is_clean_after_an_error(folder_b):
    """``llama_cu_amd.generate`` keeps the engine of a folder between calls.  A call's random draws are keyed by the
    prompt's place in the call, so the same call gives the same tokens the second time; a call that fails half
    way (a token outside the vocabulary in its second prompt) leaves nothing of itself in the engine; a folder
    that is written again is loaded again."""
    import llama_cu_amd
    from llama_cu_amd.sampling import SamplingParams
    prompts = list(common.random_requests(384, [7, 30, 12], seed=4).values())
    params = SamplingParams(temperature=0.9, top_p=0.95, seed=99)
    kw = dict(max_steps=12, dtype="float32", max_tokens=512, max_seqs=4)
    first = llama_cu_amd.generate(folder_b, prompts, params, **kw)
    engine = next(iter(llama_cu_amd._engines.values()))
    with pytest.raises(ValueError, match="outside the vocabulary"):
        llama_cu_amd.generate(folder_b, [prompts[0], [1, 2, 9999]], params, **kw)
    assert engine.idle and not engine.requests and engine.runner.cache.live_requests() == 0
    second = llama_cu_amd.generate(folder_b, prompts, params, **kw)
    assert next(iter(llama_cu_amd._engines.values())) is engine            # the same engine served all three calls
    assert second == first and len(set(map(tuple, first))) == 3
    # another order of the prompts is another set of draws for each (the key is the place in the call)
    assert llama_cu_amd.generate(folder_b, prompts[::-1], params, **kw)[::-1] != first
    # the folder written again (other weights): not the engine of before
    common.make_folder(common.TINY_B, seed=77, dtype=torch.float32, folder=folder_b)
    other = llama_cu_amd.generate(folder_b, prompts, params, **kw)
    assert next(iter(llama_cu_amd._engines.values())) is not engine and other != first
    common.make_folder(common.TINY_B, seed=22, dtype=torch.float32, folder=folder_b)      # as the fixture made it
    assert llama_cu_amd.generate(folder_b, prompts, params, **kw) == first


def test_few_pages_preemption_changes_no_token(folder_a):
    """A pool too small for all requests at once: the scheduler preempts and recomputes;
    the generated tokens are those of an ample pool."""
    from llama_cu_amd.engine.engine import Engine
    reqs = list(common.random_requests(256, [30, 45, 20, 33, 50], seed=3).values())
    ample = Engine.from_folder(folder_a, dtype="float32", max_tokens=2048, max_seqs=8)
    want = ample.generate(reqs, max_steps=40, ignore_eos=True)
    tight = Engine.from_folder(folder_a, dtype="float32", max_tokens=160, max_seqs=8, max_batch_tokens=48, prefill_chunk=16)
    got = tight.generate(reqs, max_steps=40, ignore_eos=True)
    assert tight.sched.preemptions > 0
    assert got == want
    tight.runner.cache.check()
    assert tight.runner.cache.free_pages(0) == tight.runner.num_pages


def test_long_decoding_matches_plain(folder_a):
    """100 decoded tokens after a short prompt, up to the model's context limit."""
    import llama_cu_amd
    cfg, w = plain.load_folder(folder_a)
    prompt = [7, 8, 9]
    got = llama_cu_amd.generate(folder_a, [prompt], max_steps=100, dtype="float32", max_tokens=256, max_seqs=2)[0]
    assert got == plain.greedy_generate(cfg, w, prompt, 100)


@pytest.mark.parametrize("name", ["B", "D"])
@pytest.mark.parametrize("run_ahead", [False, True])
def test_greedy_generation_in_bfloat16_through_scheduler_and_sampler(name, run_ahead):
    """The bfloat16 path through the whole engine (portions of prompts, a pool so small that a
    request is preempted and computed again, captured decode steps, the arg-max kernel): every
    generated token is the plain implementation's arg-max given the same tokens before it, or,
    where the plain implementation's two best logits lie within the bfloat16 tolerance of each
    other, one whose plain logit lies within that tolerance of the best.  Most tokens must be
    the arg-max itself."""
    from llama_cu_amd.engine.engine import Engine
    cfg_d = common.TINY[name]
    folder = common.make_folder(cfg_d, seed=31, dtype=torch.bfloat16, std=0.1)
    prompts = list(common.random_requests(cfg_d["vocab_size"], [3, 40, 77, 21, 60], seed=5).values())
    engine = Engine.from_folder(folder, dtype="bfloat16", max_tokens=256, max_seqs=4, max_batch_tokens=48, prefill_chunk=32,
                                run_ahead=run_ahead, page_size={"B": 32, "D": 64}[name])
    steps = 40
    got = engine.generate(prompts, max_steps=steps, ignore_eos=True)
    assert engine.sched.preemptions > 0                                # the pool was too small for all of them
    assert any(key[0] > 1 for key in engine.runner._graphs)            # decode steps were replayed from graphs
    engine.runner.cache.check()
    cfg, w = plain.load_folder(folder)
    exact = total = 0
    for prompt, out in zip(prompts, got):
        assert len(out) == steps
        logits = plain.forward(cfg, w, prompt + out[:-1])[len(prompt) - 1:]
        tol = common.REL_TOL["bfloat16"] * float(logits.abs().max())
        for i, tok in enumerate(out):
            best = float(logits[i].max())
            assert float(logits[i][tok]) >= best - tol, f"token {i} of a request: logit {float(logits[i][tok])} against the best {best}"
            exact += int(tok == int(torch.argmax(logits[i])))
            total += 1
    assert exact >= 0.7 * total, (exact, total)


@pytest.mark.parametrize("stored", [torch.float16, torch.float32])
def test_loading_takes_no_more_memory_than_the_weights_and_one_tensor(stored, tmp_path):
    """A folder whose file stores float16 (converted on the device) or float32 (kept) loads into one
    allocation through pinned staging: the most device memory ever held while loading is the weights
    plus one tensor as the file holds it, and the engine built on them (no second, packed copy) adds
    only its cache; its logits are the plain implementation's."""
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.engine.runner import ModelRunner
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import DecoderModel
    from llama_cu_amd.weights import load_weights, open_safetensors, write_random_model
    cfg_d = dict(common.TINY_D, hidden_size=512, intermediate_size=2048, vocab_size=4000, num_hidden_layers=3)
    cfg = LlamaConfig.from_dict(cfg_d)
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=2, dtype=stored, std=0.05)
    model = DecoderModel(llama_spec(cfg))
    compute = torch.bfloat16 if stored == torch.float16 else torch.float32
    dev = torch.device("cuda:0")
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats(dev)
    before = torch.cuda.memory_allocated(dev)
    lines = []
    t = load_weights(open_safetensors(folder), model.tensors(), compute, dev, groups=model.fused_groups(compute, dev),
                     log=lines.append)
    peak = torch.cuda.max_memory_allocated(dev) - before
    held = torch.cuda.memory_allocated(dev) - before
    elem = 2 if compute == torch.bfloat16 else 4
    weights = sum(v.numel() for v in t.values()) * elem
    largest = max(v.numel() for v in t.values()) * (2 if stored == torch.float16 else 4)
    assert weights <= held <= weights + 256 * len(t) + 4096
    assert peak <= held + largest + 4096, (peak, held, largest)
    assert "GB/s" in lines[0]
    del t
    name = "bfloat16" if compute == torch.bfloat16 else "float32"
    runner = ModelRunner.from_folder(folder, dtype=name, max_tokens=256, max_seqs=2, pack_weights=False)
    assert runner.model.layers[0].mixer.w_qkv.plain.data_ptr() == runner.model.layers[0].mixer.w_qkv.plain.untyped_storage().data_ptr() \
        or runner.model.layers[0].mixer.w_qkv.plain.storage_offset() > 0          # a view of the allocation, not a copy
    toks = list(common.random_requests(4000, [50], seed=1).values())[0]
    got = runner.step([0], [toks], [list(range(50))]).cpu()
    pcfg, pw = plain.load_folder(folder)
    want = plain.forward(pcfg, pw, toks)
    err = float((got.double() - want).abs().max())
    assert err <= common.REL_TOL[name] * float(want.abs().max())


def test_context_limit_ends_a_request(folder_a):
    from llama_cu_amd.engine.engine import Engine
    engine = Engine.from_folder(folder_a, dtype="float32", max_tokens=512, max_seqs=2)
    rid = engine.add_request(list(range(120)), max_steps=1000, ignore_eos=True)
    n = 0
    reason = None
    while not engine.idle:
        for o in engine.step():
            n += o.token is not None
            reason = o.finished or reason
    assert reason == "length" and n == 128 - 120          # max_position_embeddings of Tiny A is 128


def test_generate_command_line(folder_a):
    """``generate MODEL --max-steps N -p PROMPT`` prints the prompt, then the continuation."""
    root = common.ROOT
    proc = subprocess.run([os.path.join(root, "bin", "llama.cu_amd"), "generate", folder_a, "--max-steps", "8",
                           "-p", "Hi there", "--dtype", "float32", "--num-pages", "16", "--max-seqs", "2"],
                          capture_output=True, timeout=300)
    assert proc.returncode == 0, proc.stderr.decode()[-2000:]
    assert proc.stdout.startswith(b"Hi there")
    assert b"n toks = 8" in proc.stderr
    cfg, w = plain.load_folder(folder_a)
    want = plain.greedy_generate(cfg, w, list(b"Hi there"), 8)
    shown = bytes(t for t in want if t < 256).decode("utf-8", errors="replace")
    # the byte tokenizer shows what decodes; compare what is printable
    assert proc.stdout[len(b"Hi there"):].decode("utf-8", errors="replace").rstrip("\n").replace("�", "") == shown.replace("�", "")


def test_generate_reports_the_time_to_the_first_token_as_prefill(folder_b):
    """The report of ``generate`` as the reference counts it (llama.cu/xtask/src/generate.rs:41-52):
    prefill is the time until the first token has been received, decode the time after it.  With a
    prompt of 200 tokens in 32-bit and 3 generated tokens the prefill takes longer than a decode
    step; an engine that runs ahead and times its calls would report the opposite."""
    import io
    from llama_cu_amd import cli, text
    from llama_cu_amd.engine.engine import Engine
    prompt = list(common.random_requests(384, [200], seed=4).values())[0]
    engine = Engine.from_folder(folder_b, dtype="float32", max_tokens=512, max_seqs=2, use_graphs=False)
    engine.generate([prompt[:5]], max_steps=3, ignore_eos=True)          # everything is built and loaded
    rid = engine.add_request(prompt, max_steps=24, ignore_eos=True)
    out = io.StringIO()
    prefill, decode, ntoks = cli._stream(engine, rid, text.StreamDecoder(text.ByteTokenizer(384)), out=out)
    assert ntoks == 24
    assert prefill > 0 and decode > 0
    assert prefill > decode / 23, (prefill, decode)                      # more than one decode step


def test_chat_command_two_turns_over_stdin(folder_b):
    """``chat MODEL``: two user lines over standard input; the session's cache lives across the
    turns (llama.cu/xtask/src/chat/mod.rs:38-77), so the second answer is what the plain
    implementation generates from the whole conversation so far."""
    from llama_cu_amd import text
    root = common.ROOT
    lines = ["Hi", "And then?"]
    proc = subprocess.run([os.path.join(root, "bin", "llama.cu_amd"), "chat", folder_b, "--max-steps", "6",
                           "--dtype", "float32", "--max-tokens", "256", "--max-seqs", "2", "--page-size", "32"],
                          input="".join(l + "\n" for l in lines).encode(), capture_output=True, timeout=300)
    assert proc.returncode == 0, proc.stderr.decode()[-2000:]
    shown = proc.stdout.decode("utf-8", errors="replace")
    assert shown.count("user> ") == 3 and shown.count("assistant> ") == 2 and shown.count("=== over ===") == 2
    cfg, w = plain.load_folder(folder_b)
    template = text.load_chat_template(folder_b)
    tok = text.ByteTokenizer(384)
    context, answers = [], []
    for line in lines:
        context += tok.encode(template.render([text.user(line)]))
        reply = plain.greedy_generate(cfg, w, context, 6)
        answers.append(reply)
        context += reply
    got = shown.split("assistant> ")[1:]
    for reply, part in zip(answers, got):
        want = bytes(t for t in reply if t < 256).decode("utf-8", errors="replace").replace("�", "")
        assert part.split("\n=== over ===")[0].replace("�", "") == want


def test_smoke_entry():
    sys.path.insert(0, common.ROOT)
    import __graft_entry__
    __graft_entry__.smoke()


def test_captured_decode_steps_equal_eager_ones():
    """Decode steps replayed from a captured graph give the logits of eager steps, on
    every replay, with eager work and synchronisations between the replays, and when the
    batch's requests change places and lengths."""
    from llama_cu_amd.engine.runner import ModelRunner
    folder = common.make_folder(common.TINY_B, seed=31, dtype=torch.bfloat16, std=common.BF16_STD)
    reqs = list(common.random_requests(384, [9, 40, 33], seed=8).values())

    def decode(use_graphs):
        runner = ModelRunner.from_folder(folder, dtype="bfloat16", max_tokens=1024, max_seqs=4, use_graphs=use_graphs)
        runner.step([0, 1, 2], reqs)
        outs = []
        rng = np.random.default_rng(0)
        for i in range(12):
            toks = [[int(rng.integers(384))] for _ in range(3)]
            outs.append(runner.step([0, 1, 2], toks).float().cpu())
            if i == 6:                                    # eager work between replays: a prompt portion of another request
                runner.step([3], [[1, 2, 3, 4, 5]])
                runner.end(3)
            torch.cuda.synchronize()
        return outs, runner

    eager, _ = decode(False)
    graphed, runner = decode(True)
    assert any(key[0] == 3 for key in runner._graphs)       # the batch size was captured and replayed
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.equal(a, b), f"decode step {i} differs between eager and captured"


@pytest.mark.parametrize("name", ["B", "D"])
def test_captured_steps_with_a_prompt_portion_beside_decoding_requests_equal_eager_ones(name):
    """Steps that are not all single tokens are captured too, by their sizes: three requests decode while a fourth
    feeds five tokens of its prompt (a new request in some steps, the next portion of a long one in others, so the
    lists of the attention kernels' tasks, the contexts and the pages differ from replay to replay while the sizes
    stay).  Every replay gives the bits of the eager step, with eager work and synchronisations in between."""
    from llama_cu_amd.engine.runner import ModelRunner
    cfg = common.TINY[name]
    vocab = cfg["vocab_size"]
    folder = common.make_folder(cfg, seed=35, dtype=torch.bfloat16, std=common.BF16_STD)
    reqs = list(common.random_requests(vocab, [9, 40, 33], seed=8).values())
    rng = np.random.default_rng(1)
    plan = []
    for i in range(14):
        singles = [[int(rng.integers(vocab))] for _ in range(3)]
        portion = [int(t) for t in rng.integers(vocab, size=5)]
        plan.append((singles, portion, i % 3 == 2))               # every third step: a new request's first tokens

    def run(use_graphs):
        runner = ModelRunner.from_folder(folder, dtype="bfloat16", max_tokens=1024, max_seqs=6, use_graphs=use_graphs,
                                         page_size={"B": 32, "D": 16}[name])
        runner.step([0, 1, 2], reqs)
        outs, fresh = [], 100
        for i, (singles, portion, new) in enumerate(plan):
            if new:
                rid, fresh = fresh, fresh + 1
            else:
                rid = 3                                           # the long request goes on: its history grows by five a step
            ids, toks = [0, 1, rid, 2], [singles[0], singles[1], portion, singles[2]]
            outs.append(runner.step(ids, toks, [[0], [0], [1, 4], [0]]).float().cpu())
            if new:
                runner.end(rid)
            if i == 7:                                            # eager work between replays: another kind of step
                runner.step([50], [[1, 2, 3]])
                runner.end(50)
            torch.cuda.synchronize()
        return outs, runner

    eager, _ = run(False)
    graphed, runner = run(True)
    assert len(runner._step_graphs) == 1 and sum(runner.step_graph_replays.values()) == len(plan) - 2, runner.step_graph_replays
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.isfinite(a).all() and a.shape == (5, vocab)
        assert torch.equal(a, b), f"step {i} differs between eager and captured"


def test_the_packed_copy_of_the_weights_changes_no_logit():
    """With and without the second copy of the matrices in the decode kernels' order the
    model gives the same bits, prompt and decoding; the copy is made by default where the
    memory allows."""
    from llama_cu_amd.engine.runner import ModelRunner
    folder = common.make_folder(common.TINY_B, seed=33, dtype=torch.bfloat16, std=common.BF16_STD)
    reqs = list(common.random_requests(384, [9, 40], seed=9).values())

    def run(pack):
        runner = ModelRunner.from_folder(folder, dtype="bfloat16", max_tokens=512, max_seqs=2, pack_weights=pack)
        outs = [runner.step([0, 1], reqs).float().cpu()]
        for i in range(4):
            outs.append(runner.step([0, 1], [[3 + i], [200 - i]]).float().cpu())
        return outs, runner

    plain_outs, r0 = run(False)
    packed_outs, r1 = run(None)
    assert not r0.pack_weights and r1.pack_weights
    assert r1.model.layers[0].mixer.w_qkv.packed is not None and r0.model.layers[0].mixer.w_qkv.packed is None
    for a, b in zip(plain_outs, packed_outs):
        assert torch.equal(a, b)


def _run(engine, prompts, params=None, max_steps=20, ignore_eos=False, keep=False):
    """Tokens and finish reasons per request, through ``step()`` until idle."""
    from llama_cu_amd.sampling import GREEDY
    ids = [engine.add_request(p, params or GREEDY, max_steps, keep=keep, ignore_eos=ignore_eos) for p in prompts]
    toks = {i: [] for i in ids}
    why = {}
    while not engine.idle:
        for o in engine.step():
            if o.token is not None:
                toks[o.req].append(o.token)
            if o.finished:
                assert o.req not in why, "a request's end is reported once"
                why[o.req] = o.finished
    return ids, [toks[i] for i in ids], [why.get(i) for i in ids]


def test_running_ahead_changes_no_token_and_no_reason(folder_b):
    """The engine that launches a round before it has read the round before gives the
    tokens and finish reasons of the engine that works in turn: greedy and seeded, with
    portions, and with an end-of-sequence token that is learned a round late (what was
    computed beyond it is cut away; every page comes back)."""
    from llama_cu_amd.engine.engine import Engine
    from llama_cu_amd.sampling import SamplingParams
    prompts = list(common.random_requests(384, [3, 40, 77, 21], seed=5).values())
    kw = dict(dtype="float32", max_tokens=1024, max_seqs=4, max_batch_tokens=64, prefill_chunk=32)
    for params in (None, SamplingParams(temperature=0.9, top_p=0.95, top_k=50, seed=7)):
        in_turn = Engine.from_folder(folder_b, run_ahead=False, **kw)
        _, want, why = _run(in_turn, prompts, params, max_steps=20, ignore_eos=True)
        assert why == ["max_steps"] * 4
        ahead = Engine.from_folder(folder_b, run_ahead=True, **kw)
        _, got, why2 = _run(ahead, prompts, params, max_steps=20, ignore_eos=True)
        assert got == want and why2 == why
        # tokens that the requests generate at different steps become end-of-sequence tokens
        eos = {want[0][4], want[1][9], want[2][0]}
        a = Engine.from_folder(folder_b, run_ahead=False, **kw); a.eos = set(eos)
        b = Engine.from_folder(folder_b, run_ahead=True, **kw); b.eos = set(eos)
        _, ta, wa = _run(a, prompts, params, max_steps=20)
        _, tb, wb = _run(b, prompts, params, max_steps=20)
        assert "eos" in wa and tb == ta and wb == wa
        for e in (a, b):
            e.runner.cache.check()
            assert e.runner.cache.free_pages(0) == e.runner.num_pages


def test_a_kept_request_goes_on_after_a_late_end_of_sequence(folder_b):
    """Chat turns: a request that keeps its cache ends with an end-of-sequence token (learned
    late when running ahead) and goes on with more tokens; both engines give the same."""
    from llama_cu_amd.engine.engine import Engine
    prompt = list(common.random_requests(384, [25], seed=6).values())[0]
    kw = dict(dtype="float32", max_tokens=512, max_seqs=2)
    probe = Engine.from_folder(folder_b, run_ahead=False, **kw)
    _, first, _ = _run(probe, [prompt], max_steps=12, ignore_eos=True)
    outs = []
    for ahead in (False, True):
        e = Engine.from_folder(folder_b, run_ahead=ahead, **kw)
        e.eos = {first[0][6]}
        ids, t1, w1 = _run(e, [prompt], max_steps=12, keep=True)
        assert w1 == ["eos"] and t1[0] == first[0][:first[0].index(first[0][6]) + 1]
        assert e.runner.cache.length(ids[0]) == len(prompt) + len(t1[0]) - 1
        e.continue_request(ids[0], [11, 12, 13], max_steps=8)
        t2, w2 = [], None
        while not e.idle:
            for o in e.step():
                if o.token is not None:
                    t2.append(o.token)
                w2 = o.finished or w2
        outs.append((t1, t2, w2))
        e.drop(ids[0])
        e.runner.cache.check()
        assert e.runner.cache.free_pages(0) == e.runner.num_pages
    assert outs[0] == outs[1]
    # and the continuation is what the plain implementation generates from the whole context
    cfg, w = plain.load_folder(folder_b)
    t1, t2, _ = outs[0]
    whole = plain.greedy_generate(cfg, w, prompt + t1[0] + [11, 12, 13], len(t2))
    assert t2 == whole[:len(t2)]


def test_a_random_serving_session_changes_no_token(folder_b):
    """Requests arrive at random rounds, with random lengths, budgets and sampling, some are
    aborted on the way, the pool is so small that requests are preempted and recomputed, and
    the engine runs ahead.  Every request that was not aborted gets exactly the tokens it gets
    alone in turn with an ample pool (32-bit logits do not depend on the batch, and the random
    numbers depend on the request and the token's index only); no page or slot is lost."""
    import random
    from llama_cu_amd.engine.engine import Engine
    from llama_cu_amd.sampling import GREEDY, SamplingParams
    rng = random.Random(11)
    n_req = 14
    plan = []
    for i in range(n_req):
        prompt = [rng.randrange(384) for _ in range(rng.choice([1, 2, 17, 33, 48, 60, 60]))]
        params = GREEDY if rng.random() < 0.4 else SamplingParams(temperature=rng.choice([0.7, 1.0]), top_p=rng.choice([1.0, 0.9]),
                                                                 top_k=rng.choice([1000, 20]), seed=rng.randrange(1 << 30))
        plan.append(dict(prompt=prompt, params=params, max_steps=rng.randrange(1, 40), arrive=rng.randrange(0, 12),
                         abort_after=rng.choice([None, None, None, rng.randrange(1, 10)])))
    # alone, in turn, ample pool
    alone = Engine.from_folder(folder_b, dtype="float32", max_tokens=1024, max_seqs=1, run_ahead=False)
    want = []
    for i, r in enumerate(plan):
        rid = alone.add_request(r["prompt"], r["params"], r["max_steps"], req_id=i, ignore_eos=True)
        out = []
        while not alone.idle:
            out += [o.token for o in alone.step() if o.token is not None]
        alone.drop(rid)
        want.append(out)
    # the session: ten pages of 16 tokens; a request needs up to seven, four may be live
    eng = Engine.from_folder(folder_b, dtype="float32", max_tokens=160, max_seqs=4, max_batch_tokens=40, prefill_chunk=24,
                             run_ahead=True)
    got = {i: [] for i in range(n_req)}
    why, aborted = {}, set()
    rounds = 0
    while rounds < 12 or not eng.idle:
        for i, r in enumerate(plan):
            if r["arrive"] == rounds:
                eng.add_request(r["prompt"], r["params"], r["max_steps"], req_id=i, ignore_eos=True)
        for o in eng.step():
            if o.token is not None:
                got[o.req].append(o.token)
                r = plan[o.req]
                if r["abort_after"] is not None and len(got[o.req]) == r["abort_after"] and o.finished is None:
                    eng.abort(o.req)
                    aborted.add(o.req)
            if o.finished:
                assert o.req not in why, "a request's end is reported once"
                why[o.req] = o.finished
        rounds += 1
        assert rounds < 3000, "the session does not end"
    assert eng.sched.preemptions > 0, "the pool was meant to be too small"
    for i in range(n_req):
        if i in aborted:
            assert why[i] == "aborted" and got[i] == want[i][:len(got[i])]
        else:
            assert got[i] == want[i], f"request {i}"
            assert why[i] == "max_steps"
    for i in range(n_req):
        eng.drop(i)
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages(0) == eng.runner.num_pages and eng.runner.cache.free_slots() == 4
