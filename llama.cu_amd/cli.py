"""The command line, in the manner of the reference's ``xtask``
(llama.cu/xtask/src/main.rs:25-73): ``generate MODEL [--max-steps N] [-p PROMPT] [-t]`` and
``chat MODEL [--max-steps N]``.  ``--gpus``, ``--no-cuda-graph``, ``--tui`` and the
``service`` and ``bench`` subcommands are not here: one GPU, no server.  Added: the
compute type and the sampling options.
"""
from __future__ import annotations

import argparse
import sys
import time
from typing import List, Optional


def _base(p: argparse.ArgumentParser) -> None:
    p.add_argument("model", metavar="MODEL", help="model folder (config.json, model.safetensors[, tokenizer.json]); with "
                   "--random-weights a folder that holds config.json, or a config.json itself, is enough")
    p.add_argument("--max-steps", type=int, default=1000, help="most tokens to generate (default 1000)")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                   help="make the weights from SEED on the GPU instead of reading model.safetensors")
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--top-k", type=int, default=None)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--page-size", type=int, default=16, help="tokens per page of the cache (default 16)")
    p.add_argument("--num-pages", type=int, default=None, help="pages in the cache pool (default: from free memory)")
    p.add_argument("--max-tokens", type=int, default=None, help="size of the cache pool in tokens, instead of --num-pages")
    p.add_argument("--max-seqs", type=int, default=4, help="most requests that run at a time (default 4)")
    _plugin_option(p)


def model_folder(path: str) -> str:
    """The folder of MODEL: MODEL itself, or the folder of a config.json that was named."""
    import os
    return os.path.dirname(os.path.abspath(path)) if os.path.isfile(path) else path


def _plugin_option(p) -> None:
    p.add_argument("--plugin", action="append", default=[], metavar="MODULE",
                   help="import MODULE first (a module of yours that registers an architecture or parts); may be given "
                        "several times; the environment variable LLAMA_CU_AMD_PLUGINS names modules too")


def _engine(args):
    from . import models  # noqa: F401  (registers the architectures)
    from . import text
    from .config import load_config
    from .engine.engine import Engine
    from .sampling import SamplingParams, TOP_K_ALL
    kw = dict(page_size=args.page_size, max_seqs=args.max_seqs)
    if args.num_pages:
        kw["num_pages"] = args.num_pages
    elif args.max_tokens:
        kw["max_tokens"] = args.max_tokens
    folder = model_folder(args.model)
    t0 = time.time()
    if args.random_weights is not None:
        _, cfg = load_config(folder)
        engine = Engine.from_config(cfg, args.random_weights, dtype=args.dtype, **kw)
    else:
        engine = Engine.from_folder(folder, dtype=args.dtype, **kw)
    print(f"[info] model ready in {time.time() - t0:.2f} s", file=sys.stderr)
    params = SamplingParams(args.temperature, args.top_p, args.top_k or TOP_K_ALL, args.seed)
    tok = text.load_tokenizer(folder, engine.runner.spec.vocab_size)
    return engine, params, tok, folder


def _stream(engine, rid: int, decoder, out=sys.stdout):
    """Run rounds until request ``rid`` ends; print its text as it comes.  Returns (prefill,
    decode, tokens) as the reference counts them (llama.cu/xtask/src/generate.rs:41-52): prefill
    is the time until the first token has been received, decode all the time after that.  The
    engine runs ahead, so a call of ``step`` returns the tokens of the round before the one it
    launches; the clock therefore runs over calls, not per call."""
    start = time.time()
    first_at = None
    ntoks = 0
    while True:
        results = engine.step()
        done = False
        for o in results:
            if o.req != rid:
                continue
            if o.token is not None:
                if first_at is None:
                    first_at = time.time()
                ntoks += 1
                out.write(decoder.push(o.token))
                out.flush()
            done = done or o.finished is not None
        if done or engine.idle:
            end = time.time()
            if first_at is None:
                first_at = end
            return first_at - start, end - first_at, ntoks


def generate(args) -> int:
    """llama.cu/xtask/src/generate.rs:16-69: echo the prompt, stream the continuation, then
    report prefill time, decode time, tokens, time per token and tokens per second."""
    from . import text
    engine, params, tok, folder = _engine(args)
    prompt = args.prompt if args.prompt is not None else "Once upon a time,"
    sys.stdout.write(prompt)
    sys.stdout.flush()
    if args.use_template:
        prompt = text.load_chat_template(folder).render([text.user(prompt)])
    rid = engine.add_request(tok.encode(prompt), params, args.max_steps)
    prefill, decode, ntoks = _stream(engine, rid, text.StreamDecoder(tok))
    print()
    print(f"[info] prefill = {prefill * 1e3:.2f} ms, decode = {decode * 1e3:.2f} ms", file=sys.stderr)
    if ntoks > 0 and decode > 0:
        per = decode / ntoks              # as the reference: over all tokens, the first included (generate.rs:63)
        print(f"[info] n toks = {ntoks}, perf: {per * 1e3:.3f} ms/tok, {1 / per:.1f} tok/s", file=sys.stderr)
    return 0


def chat(args) -> int:
    """llama.cu/xtask/src/chat/mod.rs:38-77: one session whose cache lives across turns."""
    from . import text
    engine, params, tok, folder = _engine(args)
    template = text.load_chat_template(folder)
    rid: Optional[int] = None
    while True:
        line = ""
        while not line:
            sys.stdout.write("user> ")
            sys.stdout.flush()
            raw = sys.stdin.readline()
            if not raw:
                print()
                return 0
            line = raw.rstrip("\n")
        tokens = tok.encode(template.render([text.user(line)]))
        if rid is None:
            rid = engine.add_request(tokens, params, args.max_steps, keep=True)
        else:
            engine.continue_request(rid, tokens, args.max_steps)
        sys.stdout.write("assistant> ")
        sys.stdout.flush()
        _stream(engine, rid, text.StreamDecoder(tok))
        print()
        print("=== over ===")
        if engine.sched.info(rid).reason == "length":
            print("[info] the context is full; starting a new session", file=sys.stderr)
            engine.drop(rid)
            rid = None


def random_model(args) -> int:
    """Write a model folder with random weights from a configuration and a seed (the reference
    has no such mode; without files to download this is how a model of a given shape is had)."""
    import json

    import torch

    from . import models  # noqa: F401  (registers the architectures)
    from .config import architecture_of
    from .weights import write_random_model
    with open(args.config) as f:
        data = json.load(f)
    config = architecture_of(data, args.config).config_from_dict(data)
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    folder = write_random_model(args.folder, config, args.seed, dtype=dtype, std=args.std)
    print(f"[info] wrote {folder}/config.json and model.safetensors (seed {args.seed}, {args.dtype})", file=sys.stderr)
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="llama.cu_amd")
    sub = ap.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="text generation")
    _base(g)
    g.add_argument("-p", "--prompt", default=None)
    g.add_argument("-t", "--use-template", action="store_true")
    g.set_defaults(func=generate)
    c = sub.add_parser("chat", help="chat in console")
    _base(c)
    c.set_defaults(func=chat)
    r = sub.add_parser("random-model", help="write a model folder with random weights")
    r.add_argument("config", metavar="CONFIG", help="a config.json of a registered architecture")
    r.add_argument("folder", metavar="FOLDER", help="where config.json and model.safetensors are written")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16", help="type of the stored matrices")
    r.add_argument("--std", type=float, default=0.02, help="standard deviation of the matrices' entries")
    _plugin_option(r)
    r.set_defaults(func=random_model)
    args = ap.parse_args(argv)
    from .config import load_plugins
    load_plugins(args.plugin)
    return args.func(args)
