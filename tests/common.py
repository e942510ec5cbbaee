"""Shared by the tests: the tiny configurations, model folders in temporary places,
builders of traces, and the comparison with the plain implementation."""
from __future__ import annotations

import json
import os
import random
import subprocess
import sys
import tempfile
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

import plain

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# Tiny configurations of the architecture that differ in every size and option.
TINY_A = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=2, hidden_size=64, num_attention_heads=4,
              num_key_value_heads=4, head_dim=16, intermediate_size=172, vocab_size=256,
              max_position_embeddings=128, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
TINY_B = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=3, hidden_size=128, num_attention_heads=4,
              num_key_value_heads=1, head_dim=32, intermediate_size=352, vocab_size=384,
              max_position_embeddings=256, rope_theta=500000.0, rms_norm_eps=1e-6, tie_word_embeddings=True)
# no size a power of two, head_dim * heads != hidden_size, groups of 3, neighbour pairing, a large epsilon
TINY_C = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=1, hidden_size=80, num_attention_heads=6,
              num_key_value_heads=2, head_dim=48, intermediate_size=100, vocab_size=301,
              max_position_embeddings=200, rope_theta=777.0, rms_norm_eps=1e-3, tie_word_embeddings=False,
              rope_interleaved=True)
# sizes that the kernel for 17 to 128 rows takes (K a multiple of 128, a feed-forward wide enough to be cut over
# K): whole steps and mixed steps of 33 to 128 rows leave planes of partial sums to the next norm
TINY_D = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=2, hidden_size=256, num_attention_heads=4,
              num_key_value_heads=2, head_dim=64, intermediate_size=1024, vocab_size=500,
              max_position_embeddings=256, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}


def make_folder(cfg_dict: dict, seed: int, dtype: torch.dtype, std: float = 0.15, folder: Optional[str] = None) -> str:
    """A model folder with random weights, written by the test's own generator (so the
    engine's writer is not what the comparison rests on)."""
    folder = folder or tempfile.mkdtemp(prefix="lcu_model_")
    pcfg = plain.PlainConfig.from_dict(cfg_dict)
    w = plain.random_weights(pcfg, seed, std=std)
    w = {k: v.to(dtype) for k, v in w.items()}
    sys.path.insert(0, ROOT)
    from llama_cu_amd.weights import write_safetensors
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg_dict, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), w)
    return folder


def random_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def plain_logits(folder: str, reqs: Dict[str, List[int]]) -> Dict[str, torch.Tensor]:
    cfg, w = plain.load_folder(folder)
    return {name: plain.forward(cfg, w, toks) for name, toks in reqs.items()}


# ----------------------------------------------------------------------------- traces
def ceil64(n: int, page: int = 16) -> int:
    """What a request of ``n`` tokens counts for in ``--max-tokens``: ``n`` rounded up to a multiple of 64, or to
    whole pages where that is more (pages that do not divide 64)."""
    return max((n + 63) // 64 * 64, (n + page - 1) // page * page)


def _want(name, first, n, keep):
    """The places among tokens first .. first + n - 1 of request ``name`` whose logits are wanted:
    all, or those whose position ``keep(name, position)`` accepts."""
    return [k for k in range(n) if keep is None or keep(name, first + k)]


def trace_whole(reqs, keep=None, page=16):
    """Each request alone and whole: one step with all its tokens, all logits wanted."""
    steps = []
    for name, toks in reqs.items():
        steps.append({"step": len(steps), "entries": [{"id": name, "tokens": toks, "want": _want(name, 0, len(toks), keep)}],
                      "end": [name]})
    return steps, max(ceil64(len(t), page) for t in reqs.values())


def trace_tail_decode(reqs, tail=32, keep=None, page=16):
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for name, toks in reqs.items():
        head = max(len(toks) - tail, 0)
        if head:
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": toks[:head], "want": _want(name, 0, head, keep)}],
                          "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": [toks[i]], "want": _want(name, i, 1, keep)}],
                          "end": [name] if i == len(toks) - 1 else []})
    return steps, max(ceil64(len(t), page) for t in reqs.values())


def trace_portions(reqs, sizes=(7, 2, 16, 3, 48, 2, 1, 33, 5, 2), keep=None, page=16):
    """Portions of changing size, down to two tokens (and one), across page edges."""
    steps = []
    k = 0
    for name, toks in reqs.items():
        fed = 0
        while fed < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - fed)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": toks[fed:fed + n], "want": _want(name, fed, n, keep)}],
                          "end": [name] if fed + n == len(toks) else []})
            fed += n
    return steps, max(ceil64(len(t), page) for t in reqs.values())


def trace_mixed(reqs, seed=0, max_live=4, tail=12, sizes=(2, 2, 3, 5, 7, 16, 17, 31, 48), keep=None, preempt=0.0, page=16):
    """Up to ``max_live`` requests at a time: portions of some beside single tokens of
    others; requests sit steps out; finished requests' pages go to the next ones.  ``page``: the
    tokens of a page of the engine that will replay it (for the count of tokens only).  ``preempt``:
    the chance per step that one live request loses its pages (it is computed again when it next
    appears).  Returns the steps and the smallest ``--max-tokens`` that holds them."""
    rng = random.Random(seed)
    pending = list(reqs.items())
    live: Dict[str, int] = {}
    steps = []
    need = 0
    while pending or live:
        while pending and len(live) < max_live and (not live or rng.random() < 0.6):
            name, _ = pending.pop(0)
            live[name] = 0
        entries, end = [], []
        names = list(live)
        for name in names:
            toks, fed = reqs[name], live[name]
            remaining = len(toks) - fed
            if len(names) > 1 and rng.random() < 0.25:
                continue                                   # sits this step out
            if remaining <= tail:
                n = 1
            else:
                n = min(remaining - tail, rng.choice(list(sizes)))
            entries.append({"id": name, "tokens": toks[fed:fed + n], "want": _want(name, fed, n, keep)})
            live[name] = fed + n
        if not entries:
            name = names[0]
            toks, fed = reqs[name], live[name]
            entries.append({"id": name, "tokens": toks[fed:fed + 1], "want": _want(name, fed, 1, keep)})
            live[name] = fed + 1
        need = max(need, sum(ceil64(v, page) for v in live.values()))
        for name in list(live):
            if live[name] == len(reqs[name]):
                end.append(name)
                del live[name]
        step = {"step": len(steps), "entries": entries, "end": end}
        if preempt and live and rng.random() < preempt:
            step["preempt"] = [rng.choice(sorted(live))]
        steps.append(step)
    return steps, need


def collect(steps, outputs: Dict[int, np.ndarray], vocab: int) -> Dict[str, Dict[int, np.ndarray]]:
    """Logits by request and position from the per-step outputs of a replay."""
    fed: Dict[str, int] = {}
    got: Dict[str, Dict[int, np.ndarray]] = {}
    for st in steps:
        out = outputs.get(st["step"])
        row = 0
        for e in st["entries"]:
            base = fed.get(e["id"], 0)
            for k in e.get("want", []):
                got.setdefault(e["id"], {})[base + k] = out[row]
                row += 1
            fed[e["id"]] = base + len(e["tokens"])
        if out is not None:
            assert out.shape == (row, vocab), (out.shape, row, vocab)
    return got


def run_trace_inprocess(folder: str, dtype: str, steps, max_tokens: int, stats: Optional[dict] = None, **kw) -> Dict[int, np.ndarray]:
    """Replay in this process.  Pages that are given back are filled with NaN, so a read of memory
    that no live request owns shows.  ``stats``: takes ``pages_used_again`` (pages that more than
    one request held) and ``mixed_steps`` (steps with a portion of several tokens beside a single
    token)."""
    sys.path.insert(0, ROOT)
    import llama_cu_amd  # noqa: F401
    from llama_cu_amd.engine.trace import TraceReplayer
    rep = TraceReplayer.open(folder, dtype, max_tokens, poison_freed=True, **kw)
    outputs = {}
    for st in steps:
        out = rep.step(st)
        if out is not None:
            outputs[st["step"]] = out
    rep.runner.cache.check()
    assert rep.runner.cache.live_requests() == 0
    assert rep.runner.cache.free_pages(0) == rep.runner.num_pages
    if stats is not None:
        stats["pages_used_again"] = rep.pages_used_again(0)
        stats["mixed_steps"] = rep.mixed_steps
    return outputs


def run_trace_program(folder: str, dtype: str, steps, max_tokens: int, vocab: int, extra: Sequence[str] = (),
                      env: Optional[dict] = None) -> Dict[int, np.ndarray]:
    """Through ``bin/trace_run`` as a user runs it."""
    out_dir = tempfile.mkdtemp(prefix="lcu_trace_")
    text = "".join(json.dumps(s) + "\n" for s in steps)
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out_dir,
                           "--max-tokens", str(max_tokens)] + list(extra), input=text, capture_output=True, text=True, timeout=600,
                          env=env)
    assert proc.returncode == 0, proc.stderr[-2000:]
    done = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {s['step']}" for s in steps]
    outputs = {}
    for s in steps:
        p = os.path.join(out_dir, f"{s['step']}.f32")
        if os.path.exists(p):
            outputs[s["step"]] = np.fromfile(p, dtype="<f4").reshape(-1, vocab)
    return outputs


# Tolerances, as a fraction of the largest logit of the sequence, from the formats'
# precision: float32 rounds at 6e-8 and sums a few hundred terms.  bfloat16 activations
# round at 2^-8 = 4e-3 some forty times on the way through a tiny model; as independent
# errors that is 4e-3 * sqrt(40) = 2.5e-2.  That model of the error holds while the softmax
# is not sharp, so bfloat16 folders are made with a smaller weight scale (BF16_STD) than
# float32 ones: with sharp scores a rounding of a score by 4e-3 * |score| moves the
# softmax by several percent, and the comparison would measure the model's sensitivity,
# not the engine.  Sharp scores are covered in 32-bit and by the kernels' own tests.
REL_TOL = {"float32": 1e-4, "bfloat16": 2.5e-2}
BF16_STD = 0.06


def assert_matches_plain(got: Dict[str, Dict[int, np.ndarray]], want: Dict[str, torch.Tensor], dtype: str, what: str):
    rel = REL_TOL[dtype]
    for name, logits in want.items():
        ref = logits.numpy()
        scale = float(np.abs(ref).max())
        assert set(got.get(name, {})) == set(range(ref.shape[0])), f"{what}: request {name}: positions missing"
        for pos in range(ref.shape[0]):
            err = float(np.abs(got[name][pos].astype(np.float64) - ref[pos]).max())
            assert np.isfinite(err) and err <= rel * scale, \
                f"{what}: request {name}, first wrong position {pos} of {ref.shape[0]}: error {err:.3e} > {rel * scale:.3e}"


# ----------------------------------------------------------------------------- a plugin
# A module of a user's, as a file outside the package: an architecture of its own (the Llama layout, but the layer
# that config.json's "mean_layer" names mixes with a running mean of its inputs, whose state of fixed size lives in
# the engine's state slots) with a part of its own.  Named with --plugin or in LLAMA_CU_AMD_PLUGINS.
TOY_PLUGIN = '''
import dataclasses

import torch

from llama_cu_amd import register_architecture, register_part
from llama_cu_amd.config import LlamaConfig
from llama_cu_amd.models.llama import llama_spec
from llama_cu_amd.parts import Part, PartSpec, SlotState, TensorSpec


class RunningMean(Part):
    def __init__(self, hidden_size):
        self.d = hidden_size

    def tensors(self):
        return {"mix.weight": TensorSpec((self.d, self.d))}

    def cache_need(self):
        return SlotState((self.d,), torch.float32)

    def load(self, tensors, build):
        self.w = tensors["mix.weight"].float()

    def forward(self, h, step, cache):
        out = torch.empty_like(h)
        start = 0
        for r, n in enumerate(step.q_lens):
            slot = step.state_slots[r]
            first = step.ctx_lens[r] - n
            if first == 0:
                cache.state[slot].zero_()
            sums = cache.state[slot] + torch.cumsum(h[start:start + n].float(), 0)
            counts = torch.arange(first + 1, first + n + 1, device=h.device, dtype=torch.float32)[:, None]
            out[start:start + n] = ((sums / counts) @ self.w.T).to(h.dtype)
            cache.state[slot] = sums[-1]
            start += n
        return out


@dataclasses.dataclass(frozen=True)
class ToyMeanConfig:
    base: LlamaConfig
    mean_layer: int

    @staticmethod
    def from_dict(d):
        d = dict(d)
        mean_layer = int(d.pop("mean_layer"))
        d["architectures"] = ["LlamaForCausalLM"]
        base = LlamaConfig.from_dict(d)
        if not 0 <= mean_layer < base.num_hidden_layers:
            raise ValueError("mean_layer names no layer")
        return ToyMeanConfig(base, mean_layer)

    def to_dict(self):
        return dict(self.base.to_dict(), architectures=["ToyMeanForCausalLM"], mean_layer=self.mean_layer)


def toy_mean_spec(cfg):
    spec = llama_spec(cfg.base)
    spec.layers[cfg.mean_layer].params["mixer"] = PartSpec("running_mean", {"hidden_size": cfg.base.hidden_size}, "toy")
    return spec


register_part("mixer", "running_mean", RunningMean, replace=True)
register_architecture("ToyMeanForCausalLM", ToyMeanConfig.from_dict, toy_mean_spec, replace=True)
'''


def write_toy_plugin(folder: str, name: str = "lcu_toy_plugin") -> Tuple[str, dict]:
    """Writes the module into ``folder``; returns its name and an environment in which a child process finds it."""
    with open(os.path.join(folder, name + ".py"), "w") as f:
        f.write(TOY_PLUGIN)
    env = dict(os.environ)
    env["PYTHONPATH"] = folder + os.pathsep + env.get("PYTHONPATH", "")
    return name, env


# ----------------------------------------------------------------------------- a sweep of configurations
def sweep_configuration(seed: int, lens_max: int = 140):
    """A configuration, a page size and request lengths drawn from ``seed``: the generator of a search for wrong
    logits over some 1,700 seeds.  Among them are the widest and deepest models that tests replay (width up to
    512, three layers), where bfloat16 rounding adds up to the most."""
    rng = random.Random(seed * 7919)
    mfma = rng.random() < 0.6
    nkv = rng.choice([1, 2, 3, 4, 8])
    g = rng.choice([1, 2, 4, 8, 16]) if mfma else rng.choice([1, 2, 3, 5, 7])
    dh = rng.choice([32, 64, 96, 128]) if mfma else rng.choice([16, 48, 80, 112, 144, 256])
    cfg = dict(architectures=["LlamaForCausalLM"], num_hidden_layers=rng.choice([1, 2, 3]),
               hidden_size=rng.choice([64, 72, 128, 136, 192, 256, 320, 384, 512, 8 * rng.randrange(5, 40)]),
               num_attention_heads=nkv * g, num_key_value_heads=nkv, head_dim=dh,
               intermediate_size=rng.choice([56, 128, 172, 352, 2 * rng.randrange(4, 300), 16 * rng.randrange(1, 40),
                                             8 * rng.randrange(1, 80)]),
               vocab_size=rng.choice([257, 384, 1000, 16 * rng.randrange(4, 80), rng.randrange(50, 1500)]),
               max_position_embeddings=512, rope_theta=rng.choice([1e4, 5e5]),
               rms_norm_eps=rng.choice([1e-5, 1e-6]), tie_word_embeddings=rng.random() < 0.5,
               rope_interleaved=rng.random() < 0.2)
    page = rng.choice([16, 32, 48, 64, 128])
    lens = [rng.randrange(1, lens_max) for _ in range(rng.choice([2, 3, 4]))]
    return cfg, page, lens
