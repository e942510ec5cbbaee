#!/usr/bin/python3
"""Measurement: decoded tokens a second of the Llama-3-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch through the engine (scheduler, step
function, sampling): W untimed steps, then exactly K timed ones between two
synchronisations.  The default run has the layer sizes of the Llama-3-8B shape with random
weights, a batch of 8 requests with prompts of 2,048 uniform random tokens and a context
limit of 8,192.  One JSON line comes out: decoded tokens a second (``value``), the time of
a 2,048-token prefill with its fraction of the bf16 matrix peak, the decode step's bytes
against the HBM peak, and decoding at batch 1 and 64 (``points``).

Peaks are MI355X's published ones: HBM 8 TB/s; dense matrix bf16 2.5 PFLOP/s, fp32
157.3 TFLOP/s.  The reference publishes no numbers, so ``vs_baseline`` is null.
"""
import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
MATRIX_PEAK = {"bf16": 2.5e15, "f32": 157.3e12}

# the Llama-3-8B shape
SHAPE = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=32, hidden_size=4096, num_attention_heads=32,
             num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256,
             max_position_embeddings=8192, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
# other shapes to measure the same step at (--shape): the 7B shape has a key/value head per head, a
# smaller feed-forward and vocabulary; the 70B shape is twice as wide (give it --layers: 80 layers
# of it take 141 GB)
SHAPES = {
    "llama3-8b": ("Llama-3-8B", SHAPE),
    "llama2-7b": ("Llama-2-7B", dict(SHAPE, num_key_value_heads=32, intermediate_size=11008, vocab_size=32000,
                                     max_position_embeddings=4096, rope_theta=10000.0)),
    "llama3-70b": ("Llama-3-70B", dict(SHAPE, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                                       intermediate_size=28672)),
}
PROMPT_LEN = 2048
PREFILL_TOKENS = 2048


def weight_bytes(c, elem):
    """Bytes of the weights a decode step reads once: every matrix and norm weight (of the
    embedding table only the batch's rows, which is negligible and left out)."""
    d, dh, nh, nkv, di = c.hidden_size, c.head_dim, c.num_attention_heads, c.num_key_value_heads, c.intermediate_size
    per_layer = (nh + 2 * nkv) * dh * d + d * nh * dh + 2 * di * d + d * di + 2 * d
    return (c.num_hidden_layers * per_layer + d + c.vocab_size * d) * elem


def kv_bytes_per_token(c, elem):
    return c.num_hidden_layers * 2 * c.num_key_value_heads * c.head_dim * elem


def prefill_flops(c, t, history=0):
    """Of a step that feeds ``t`` tokens of a prompt after ``history`` tokens that the cache holds."""
    d, dh, nh, nkv, di = c.hidden_size, c.head_dim, c.num_attention_heads, c.num_key_value_heads, c.intermediate_size
    per_token = 2 * ((nh + 2 * nkv) * dh * d + d * nh * dh + 2 * di * d + d * di)
    matmul = c.num_hidden_layers * per_token * t + 2 * c.vocab_size * d      # the output matrix for the last row only
    pairs = t * history + t * (t + 1) / 2                                    # causal: every key before, half of the step's own
    attention = c.num_hidden_layers * 2 * 2 * nh * dh * pairs                # QK^T and PV
    return matmul + attention


def rounds_of(prompt_len):
    """Rounds that a prompt's prefill takes (portions of PREFILL_TOKENS): earlier requests decode meanwhile."""
    return (prompt_len + PREFILL_TOKENS - 1) // PREFILL_TOKENS


def run_decode(engine, cfg, batch, steps, warmup, rng, sync, prompt_len=PROMPT_LEN):
    """Prefill ``batch`` prompts, then time ``steps`` decode steps.  Returns (seconds,
    tokens decoded in them, mean context length during the timed steps)."""
    from llama_cu_amd.sampling import GREEDY
    ids = [engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(prompt_len)], GREEDY,
                              max_steps=steps + warmup + 2 * batch * rounds_of(prompt_len) + 8, ignore_eos=True)
           for _ in range(batch)]
    # prefill rounds: until every request has produced its first token
    while any(engine.sched.info(i).generated == 0 for i in ids):
        engine.step()
    for _ in range(warmup):
        engine.step()
    import torch
    ctx0 = engine.sched.info(ids[0]).n_tokens
    sync()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    marks[0].record()
    t0 = time.perf_counter()
    produced = 0
    for k in range(steps):
        produced += sum(1 for o in engine.step() if o.token is not None)
        marks[k + 1].record()                       # on the stream, after the step's kernels
    sync()
    dt = time.perf_counter() - t0
    per_step = sorted(marks[k].elapsed_time(marks[k + 1]) for k in range(steps))
    run_decode.median_ms = per_step[len(per_step) // 2]
    ctx1 = engine.sched.info(ids[0]).n_tokens
    for i in ids:
        engine.abort(i)
        engine.drop(i)
    assert produced == batch * steps, (produced, batch, steps)
    return dt, produced, (ctx0 + ctx1) / 2.0


def run_prefill(engine, cfg, rng, sync, repeats=3, history=0):
    """Best time of one step that feeds PREFILL_TOKENS tokens of a prompt: a whole prompt, or,
    with ``history``, the portion after that many tokens (fed before, untimed)."""
    best = None
    run_prefill.whole = None                        # best time of the whole prompt, history included
    for k in range(repeats + 1):
        toks = [rng.randrange(cfg.vocab_size) for _ in range(PREFILL_TOKENS)]
        rid = 10_000 + k
        sync()
        t_all = time.perf_counter()
        for at in range(0, history, PREFILL_TOKENS):
            engine.runner.step([rid], [[rng.randrange(cfg.vocab_size) for _ in range(min(PREFILL_TOKENS, history - at))]], want=[[]])
        sync()
        t0 = time.perf_counter()
        engine.runner.step([rid], [toks])
        sync()
        t1 = time.perf_counter()
        engine.runner.end(rid)
        if k > 0:                                   # the first run warms up
            best = t1 - t0 if best is None else min(best, t1 - t0)
            run_prefill.whole = t1 - t_all if run_prefill.whole is None else min(run_prefill.whole, t1 - t_all)
    return best


def run_first_token(engine, cfg, n_requests, prompt_len, rng, sync, repeats=4):
    """Time to the first token: ``n_requests`` requests with prompts of ``prompt_len`` tokens arrive together at an
    idle engine; the time until every one of them has its first token on the host (the reference's own headline,
    llama.cu/xtask/src/generate.rs:41-52: its "prefill" is the time until the first token was received).  The best
    of ``repeats`` (the first ones build, load and capture)."""
    from llama_cu_amd.sampling import GREEDY
    best = None
    for _ in range(repeats):
        prompts = [[rng.randrange(cfg.vocab_size) for _ in range(prompt_len)] for _ in range(n_requests)]
        sync()
        t0 = time.perf_counter()
        ids = [engine.add_request(p, GREEDY, max_steps=1, ignore_eos=True) for p in prompts]
        got = 0
        while got < n_requests:
            got += sum(1 for o in engine.step() if o.token is not None)
        dt = time.perf_counter() - t0
        while not engine.idle:
            engine.step()
        for i in ids:
            engine.drop(i)
        best = dt if best is None else min(best, dt)
    return best


def run_prefill_step(engine, cfg, n_requests, prompt_len, rng, sync, repeats=4):
    """Best time of ONE step that holds the whole prompts of ``n_requests`` requests, ``prompt_len`` tokens each
    (many short tasks for the prefill attention)."""
    best = None
    for k in range(repeats):
        ids = [20_000 + k * n_requests + i for i in range(n_requests)]
        toks = [[rng.randrange(cfg.vocab_size) for _ in range(prompt_len)] for _ in ids]
        sync()
        t0 = time.perf_counter()
        engine.runner.step(ids, toks)
        sync()
        dt = time.perf_counter() - t0
        for i in ids:
            engine.runner.end(i)
        if k > 0:
            best = dt if best is None else min(best, dt)
    return best


def run_mixed(engine, cfg, n_requests, rng, sync, new_tokens=128, lo=16, hi=2048):
    """A mixed batch (the workload that goes with the Llama-2-7B shape): ``n_requests`` requests at once, prompt
    lengths uniform in [lo, hi], ``new_tokens`` greedy tokens each, through the scheduler under its
    token budget (prompt portions beside decoding requests).  Returns a dict of what was measured:
    the reference's bench prints the same (llama.cu/xtask/src/bench.rs:63-80: time to the first
    answer, tokens, time per token, steps, time per step)."""
    import torch
    from llama_cu_amd.sampling import GREEDY
    lens = [rng.randrange(lo, hi + 1) for _ in range(n_requests)]
    ids = [engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(n)], GREEDY, max_steps=new_tokens, ignore_eos=True)
           for n in lens]
    sync()
    marks = [torch.cuda.Event(enable_timing=True)]
    marks[0].record()
    t0 = time.perf_counter()
    produced = steps = 0
    first_all = first_steps = None
    while not engine.idle:
        outs = engine.step()
        steps += 1
        marks.append(torch.cuda.Event(enable_timing=True))
        marks[-1].record()
        produced += sum(1 for o in outs if o.token is not None)
        if first_all is None and all(engine.sched.info(i).generated > 0 for i in ids):
            sync()
            first_all, first_steps = time.perf_counter() - t0, steps
    sync()
    dt = time.perf_counter() - t0
    for i in ids:
        engine.drop(i)
    assert produced == n_requests * new_tokens, (produced, n_requests, new_tokens)
    per_step = [marks[k].elapsed_time(marks[k + 1]) for k in range(steps)]
    decode_steps = sorted(per_step[first_steps:]) or [0.0]
    return {"requests": n_requests, "prompt_tokens": sum(lens), "new_tokens": produced, "seconds": dt,
            "all_prompts_in_ms": first_all * 1e3, "prefill_steps": first_steps, "steps": steps,
            "decode_step_median_ms": decode_steps[len(decode_steps) // 2], "preemptions": engine.sched.preemptions}


def run_arrivals(engine, cfg, batch, steps, rng, sync, every=2, arrival_len=16, arrival_tokens=2):
    """``batch`` requests decode (after prompts of PROMPT_LEN tokens) while a new request with a prompt of
    ``arrival_len`` tokens arrives every ``every`` steps, generates ``arrival_tokens`` tokens and leaves: steps in
    which a prompt portion stands beside the decoding requests alternate with steps that only decode.  Returns what
    the engine's timeline says of the timed steps: wall time per step, the host's time per step from the plan to
    the last launch, and the fraction of the time in which the GPU had a step's work (events around each step)."""
    from llama_cu_amd.sampling import GREEDY
    total = steps + 64
    ids = [engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(PROMPT_LEN)], GREEDY, max_steps=total + 8 * batch,
                              ignore_eos=True) for _ in range(batch)]
    while any(engine.sched.info(i).generated == 0 for i in ids):
        engine.step()
    arrivals = []

    def rounds(n, timed):
        for k in range(n):
            if k % every == 0:
                arrivals.append(engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(arrival_len)], GREEDY,
                                                   max_steps=arrival_tokens, ignore_eos=True))
            engine.step()
    rounds(32, False)                                # every kind of step has come often enough to be captured, if it can be
    sync()
    engine.timeline = []
    t0 = time.perf_counter()
    rounds(steps, True)
    sync()
    dt = time.perf_counter() - t0
    line, engine.timeline = engine.timeline, None
    for i in ids:
        engine.abort(i)
        engine.drop(i)
    while not engine.idle:
        engine.step()
    for i in arrivals:
        engine.drop(i)
    busy = sum(e["first"].elapsed_time(e["last"]) for e in line)
    span = line[0]["first"].elapsed_time(line[-1]["last"])
    kinds = {}
    for e in line:
        k = kinds.setdefault((e["tokens"], e["requests"], e["graph"]), [0, 0.0, 0.0])
        k[0] += 1
        k[1] += e["host_ms"]
        k[2] += e["first"].elapsed_time(e["last"])
    return {"steps": len(line), "ms_per_step": dt / steps * 1e3, "host_ms_per_step": sum(e["host_ms"] for e in line) / len(line),
            "gpu_busy_frac": busy / span,
            "kinds": [{"tokens": t, "requests": r, "from_graph": g, "steps": n, "host_ms": h / n, "gpu_ms": u / n}
                      for (t, r, g), (n, h, u) in sorted(kinds.items())]}


def float32_copy_bytes(engine):
    """What a 32-bit copy of the engine's weights takes, with room for its small cache and activations."""
    count = sum(t.numel() for t in engine.runner.tensors.values())
    return 4 * count + (2 << 30)


def free_device_bytes():
    import torch
    torch.cuda.empty_cache()
    return torch.cuda.mem_get_info()[0]


def check_against_float32(engine, cfg, rng, sync, prompt_len=48, decode_steps=6):
    """The benchmarked bfloat16 model against the true 32-bit path with the same weights, at the benchmark's full depth:
    a prompt in one step (logits at every position) and some single-token steps after it, through both runners.  The
    32-bit path is the one that the tests hold against the plain implementation; here it says whether the bfloat16
    kernels that were just timed still compute the model.  Returns the largest difference of a logit as a fraction of
    the largest logit, the root mean square difference as a fraction of the logits' root mean square, and how many of
    the positions agree on the arg-max."""
    import torch
    from llama_cu_amd.engine.runner import ModelRunner
    ref = ModelRunner.from_config(cfg, seed=0, dtype="float32", stored="bfloat16", page_size=16, max_tokens=256, max_seqs=2,
                                  max_batch_tokens=256, one_piece=False)
    toks = [rng.randrange(cfg.vocab_size) for _ in range(prompt_len)]
    rid = 30_000
    want = list(range(prompt_len))
    a = engine.runner.step([rid], [toks], [want])
    b = ref.step([rid], [toks], [want])
    worst, scale, same, total, err2, ref2, count = 0.0, 0.0, 0, 0, 0.0, 0.0, 0
    for _ in range(decode_steps + 1):
        worst = max(worst, float((a - b).abs().max()))
        scale = max(scale, float(b.abs().max()))
        err2 += float(((a - b).double() ** 2).sum())
        ref2 += float((b.double() ** 2).sum())
        count += a.numel()
        same += int((a.argmax(-1) == b.argmax(-1)).sum())
        total += a.shape[0]
        nxt = int(b[-1].argmax())
        a = engine.runner.step([rid], [[nxt]])
        b = ref.step([rid], [[nxt]])
    sync()
    engine.runner.end(rid)
    del ref
    torch.cuda.empty_cache()
    return worst / scale, (err2 / ref2) ** 0.5, same, total


def library_product(cfg, sync, calls=400):
    """Time of the library's gate/up product of a 2,048-token prefill (the largest of a layer's four), once with
    random rows and once with rows of zeros: the same instructions on the same addresses, but zeros switch far fewer
    wires, so the difference is what the chip's power limit takes off its clock while it multiplies random numbers."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(0)
    w = (torch.randn(2 * cfg.intermediate_size, cfg.hidden_size, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(PREFILL_TOKENS, cfg.hidden_size, device="cuda", generator=g).to(torch.bfloat16)
    flops = 2.0 * PREFILL_TOKENS * cfg.hidden_size * 2 * cfg.intermediate_size
    out = {}
    for name in ("random_rows", "zero_rows"):
        if name == "zero_rows":
            x.zero_()
        best = None
        for _ in range(4):                          # the first round warms up; the clock settles within it
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(calls):
                torch.nn.functional.linear(x, w)
            b.record()
            sync()
            t = a.elapsed_time(b) / calls * 1e-3
            best = t if best is None else min(best, t)
        out[name] = {"us": round(best * 1e6, 1), "pflops": round(flops / best / 1e15, 3)}
    return out


def kernel_summary(db: str, steps: int, launches: int = 0) -> int:
    """Per-step table of kernels from the database that ``rocprofv3 --kernel-trace`` wrote for a
    run of this program: the kernels between two embedding gathers are one step of the model;
    the last ``steps`` steps are averaged (with ``launches``: the last ``steps`` steps of exactly that
    many kernel launches, to tell the kinds of steps of a mixed workload apart)."""
    import re
    import sqlite3
    con = sqlite3.connect(db)
    rows = con.execute("select name, start, end from kernels order by start").fetchall()
    marks = [i for i, r in enumerate(rows) if "embedding_gather" in r[0]]
    spans = [(a, b) for a, b in zip(marks[:-1], marks[1:]) if not launches or b - a == launches]
    if len(spans) < steps:
        kinds = sorted({b - a for a, b in zip(marks[:-1], marks[1:])})
        print(f"bench.py: {db} holds {len(spans)} such steps, fewer than the {steps} needed (launches a step: {kinds})")
        return 1
    spans = spans[-steps:]
    agg = {}
    for a, b in spans:
        for name, t0, t1 in rows[a:b]:
            short = re.sub(r"\(.*", "", name).replace("void ", "")
            short = re.sub(r"_SN_LDSB.*", "", short)[:70]
            item = agg.setdefault(short, [0, 0.0])
            item[0] += 1
            item[1] += (t1 - t0) / 1e3
    wall = sum(rows[b][1] - rows[a][1] for a, b in spans) / 1e3 / steps
    busy = sum(v[1] for v in agg.values()) / steps
    print(f"steps averaged: {steps}; wall {wall:.1f} us/step, kernels busy {busy:.1f} us/step\n")
    print("| kernel | launches/step | us/step | avg us | % of busy |")
    print("|---|---|---|---|---|")
    for name, (n, t) in sorted(agg.items(), key=lambda kv: -kv[1][1]):
        print(f"| `{name}` | {n / steps:.0f} | {t / steps:.1f} | {t / n:.1f} | {100 * t / steps / busy:.1f} |")
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="llama3-8b", help="the layer sizes (default: the Llama-3-8B shape)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN,
                    help="tokens of each request's prompt (other context lengths than the default run's; the context "
                         "limit grows with it)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--page-size", type=int, default=16, help="tokens in a page of the cache (a multiple of 16)")
    ap.add_argument("--workload", choices=["decode", "mixed", "arrivals"], default="decode",
                    help="decode: --batch requests decode together after prompts of --prompt-len (the default); mixed: "
                         "--batch requests at once with prompt lengths uniform in [16, 2048], 128 tokens each, through the "
                         "scheduler (the workload that goes with --shape llama2-7b --batch 64); arrivals: --batch requests "
                         "decode while a prompt of 16 tokens arrives every second step (host time and the GPU's busy "
                         "fraction per kind of step)")
    ap.add_argument("--no-points", action="store_true", help="skip decoding at batch 1 and 64, the prefill and the check")
    ap.add_argument("--no-check", action="store_true",
                    help="skip the comparison of the benchmarked model's logits with the 32-bit path's (same weights, all layers)")
    ap.add_argument("--points", choices=["default", "all"], default="default",
                    help="all: beside decoding at batch 1 and 64 also the time to the first token at 1 and 8 requests for "
                         "prompts of 16, 128, 512 and 8192 tokens, one prefill step of 16 prompts of 128 tokens and of 64 of "
                         "32, and decoding at 256 requests over 512 keys")
    ap.add_argument("--only-prefill", action="store_true", help="time the 2048-token prefill alone (for profiles)")
    ap.add_argument("--prefill-history", type=int, default=0,
                    help="with --only-prefill: time the 2048 tokens that follow this many tokens of the same prompt")
    ap.add_argument("--library-product", action="store_true",
                    help="time the library's gate/up product of 2048 rows with random rows and with rows of zeros, and exit")
    ap.add_argument("--kernel-summary", metavar="DB", help="print the per-step kernel table of a rocprofv3 database and exit")
    ap.add_argument("--summary-steps", type=int, default=8)
    ap.add_argument("--summary-launches", type=int, default=0,
                    help="with --kernel-summary: only steps of exactly this many kernel launches (0: all)")
    args = ap.parse_args()
    if args.kernel_summary:
        return kernel_summary(args.kernel_summary, args.summary_steps, args.summary_launches)
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported (no multi-GPU path)")
        return 2

    import torch
    import llama_cu_amd  # noqa: F401
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.engine.engine import Engine

    shape_name, shape = SHAPES[args.shape]
    shape = dict(shape)
    full_layers = shape["num_hidden_layers"]
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    grow = args.steps + args.warmup + 2 * max(args.batch, 64) * rounds_of(args.prompt_len) + 64
    need_ctx = max(args.prompt_len + grow + 64, args.prefill_history + PREFILL_TOKENS, 8192 + 64 if args.points == "all" else 0)
    while shape["max_position_embeddings"] < need_ctx:
        shape["max_position_embeddings"] *= 2
    cfg = LlamaConfig.from_dict(shape)
    dt_name = "bf16" if args.dtype == "bfloat16" else "f32"
    elem = 2 if args.dtype == "bfloat16" else 4
    rng = random.Random(0)
    sync = torch.cuda.synchronize
    page = args.page_size
    if args.library_product:
        print(json.dumps({"library_product": library_product(cfg, sync), "rows": PREFILL_TOKENS,
                          "in": cfg.hidden_size, "out": 2 * cfg.intermediate_size, "dtype": "bf16"}))
        return 0
    all_points = args.points == "all" and not args.no_points
    biggest = max(args.batch, 1 if (args.no_points or args.only_prefill or args.workload != "decode") else (256 if all_points else 64))
    # a request decodes while later ones still prefill: room for that too
    per_req = max(args.prompt_len, PROMPT_LEN) + grow
    engine = Engine.from_config(cfg, seed=0, dtype=args.dtype, page_size=page,
                                max_tokens=biggest * ((per_req + page - 1) // page * page) + args.prefill_history + PREFILL_TOKENS + page,
                                max_seqs=biggest + 2, max_batch_tokens=max(PREFILL_TOKENS, biggest), prefill_chunk=PREFILL_TOKENS)

    if args.workload == "arrivals":
        a = run_arrivals(engine, cfg, args.batch, args.steps, rng, sync)
        print(json.dumps({"metric": f"ms a step ({shape_name} shape, {args.batch} requests decode, a prompt of 16 tokens arrives "
                                    f"every second step)", "value": round(a["ms_per_step"], 4), "unit": "ms", "n_gpus": 1,
                          "steps": a["steps"], "higher_is_better": False, "dtype": dt_name, "data": "synthetic",
                          "host_ms_per_step": round(a["host_ms_per_step"], 3), "gpu_busy_frac": round(a["gpu_busy_frac"], 4),
                          "kinds": [{k: (round(v, 3) if isinstance(v, float) else v) for k, v in kind.items()} for kind in a["kinds"]]}),
              flush=True)
        return 0
    if args.workload == "mixed":
        run_mixed(engine, cfg, min(args.batch, 8), rng, sync, new_tokens=8)          # builds, loads and captures
        m = run_mixed(engine, cfg, args.batch, rng, sync)
        print(json.dumps({
            "metric": f"generated tok/s ({shape_name} shape, mixed batch: {args.batch} requests at once, prompts uniform in "
                      f"[16, 2048], 128 tokens each)", "value": round(m["new_tokens"] / m["seconds"], 1), "unit": "tok/s",
            "n_gpus": 1, "steps": m["steps"], "warmup": 0, "ms_per_step": round(m["seconds"] / m["steps"] * 1e3, 3),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dt_name, "data": "synthetic",
            "config": {"model": f"{shape_name} shape, random weights", "global_batch": args.batch, "parallelism": "none (1 GPU)",
                       "layers": cfg.num_hidden_layers, "layers_of_shape": full_layers, "kv_heads": cfg.num_key_value_heads,
                       "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size, "page_size": page,
                       "token_budget": PREFILL_TOKENS, "sampling": "greedy"},
            "mixed": {k: (round(v, 3) if isinstance(v, float) else v) for k, v in m.items()},
            "total_tok_s": round((m["prompt_tokens"] + m["new_tokens"]) / m["seconds"], 1)}), flush=True)
        return 0
    if args.only_prefill:
        pt = run_prefill(engine, cfg, rng, sync, repeats=args.steps, history=args.prefill_history)
        flops = prefill_flops(cfg, PREFILL_TOKENS, args.prefill_history)
        print(json.dumps({"prefill": {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS, "ms": round(pt * 1e3, 3),
                                      "frac": round(flops / pt / MATRIX_PEAK[dt_name], 4), "history": args.prefill_history,
                                      "whole_prompt_tokens": args.prefill_history + PREFILL_TOKENS,
                                      "whole_prompt_ms": round(run_prefill.whole * 1e3, 2)}}))
        return 0
    seconds, produced, mean_ctx = run_decode(engine, cfg, args.batch, args.steps, args.warmup, rng, sync, args.prompt_len)
    ms_per_step = seconds / args.steps * 1e3
    median_ms = run_decode.median_ms                # of the steps' times on the GPU (events), beside the mean of the wall time
    value = produced / seconds
    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / (seconds / args.steps)
    line = {
        "metric": f"decode tok/s ({shape_name} shape, prompts of {args.prompt_len} tokens)", "value": round(value, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_median": round(median_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dt_name, "data": "synthetic",
        "config": {"model": f"{shape_name} shape, random weights", "global_batch": args.batch, "seq_len": args.prompt_len,
                   "parallelism": "none (1 GPU)", "context": cfg.max_position_embeddings,
                   "layers": cfg.num_hidden_layers, "layers_of_shape": full_layers, "hidden_size": cfg.hidden_size,
                   "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps, "page_size": page,
                   "sampling": "greedy"},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    if not args.no_points:
        pt = run_prefill(engine, cfg, rng, sync)
        flops = prefill_flops(cfg, PREFILL_TOKENS)
        line["prefill"] = {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS, "ms": round(pt * 1e3, 3),
                           "frac": round(flops / pt / MATRIX_PEAK[dt_name], 4)}
        points = {}
        for b in (1, 64):
            s, p, _ = run_decode(engine, cfg, b, max(16, args.steps // 4), 4, rng, sync)
            points[f"decode_b{b}"] = round(p / s, 2)
        if all_points:
            s, p, _ = run_decode(engine, cfg, 256, max(16, args.steps // 4), 4, rng, sync, prompt_len=512)
            points["decode_b256_ctx512"] = round(p / s, 2)
            for b in (1, 8):
                for n in (16, 128, 512, 8192):
                    points[f"first_token_ms_b{b}_prompt{n}"] = round(run_first_token(engine, cfg, b, n, rng, sync) * 1e3, 3)
            for b, n in ((16, 128), (64, 32)):
                t = run_prefill_step(engine, cfg, b, n, rng, sync)
                points[f"prefill_step_ms_{b}x{n}"] = round(t * 1e3, 3)
        line["points"] = points
        need = float32_copy_bytes(engine)
        free = free_device_bytes()
        if not args.no_check and args.dtype == "bfloat16" and need > free:
            # the 32-bit model would not fit beside the benchmarked one (all layers of the largest shape): said, not hidden
            line["check"] = {"against": "float32 path, same weights, all layers", "skipped":
                             f"the 32-bit copy of the weights takes {need / 1e9:.0f} GB, {free / 1e9:.0f} GB are free", "ok": None}
        elif not args.no_check and args.dtype == "bfloat16":
            rel, rms, same, total = check_against_float32(engine, cfg, rng, sync)
            # bfloat16 rounding through all layers moves the logits by a few hundredths of their size (measured:
            # root mean square 0.04 of the logits' own, largest 0.05 of the largest); a kernel that computes
            # something else moves them by their size
            line["check"] = {"against": "float32 path, same weights, all layers", "positions": total,
                             "rms_error_of_rms_logit": round(rms, 5), "max_error_of_largest_logit": round(rel, 5),
                             "same_argmax": same, "ok": bool(rms < 0.1 and rel < 0.2)}
    print(json.dumps(line), flush=True)
    if "check" in line and line["check"]["ok"] is False:
        print("bench.py: the benchmarked model's logits differ from the 32-bit path's", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
