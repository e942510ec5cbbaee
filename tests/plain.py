"""A plain, slow implementation of the Llama dense decoder.

Written from the formulas of the reference (YdrMaster/llama.cu); every function
cites the file and lines it follows.  Whole sequences, no cache, one function
for each part, float64 unless a formula fixes 32-bit (the rotation angles).  It
shares no code with the engine: it imports nothing from the package.

Paths are relative to the reference's root.
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

F64 = torch.float64


def rounded(x: torch.Tensor, rounding: Optional[str]) -> torch.Tensor:
    """``x`` as a tensor of the type ``rounding`` holds it (None: as it is; "bfloat16": rounded to 32-bit, as
    a kernel's accumulator holds it, and then to bfloat16, as the kernel stores it)."""
    if rounding is None:
        return x
    if rounding != "bfloat16":
        raise ValueError(f"rounding {rounding!r}: None or 'bfloat16'")
    return x.to(torch.float32).to(torch.bfloat16).to(F64)


# --------------------------------------------------------------------------- parts


def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """``out[i, :] = table[ids[i], :]``: a row copy, no scale and no position term.

    llama.cu/src/op/embedding.cuh:6-8; no position table: llama.cu/src/model/mod.rs:91-99
    (``wpe: None``).
    """
    return torch.stack([table[int(i)] for i in ids]).to(F64)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``y = x * rsqrt(sum(x^2)/d + eps) * w``; the weight multiplies as it is (no 1+w).

    llama.cu/src/op/rms_norm.cuh:21-29 (sum of squares, divided by the width, plus
    epsilon, rsqrt, then rms * x * w).
    """
    x = x.to(F64)
    d = x.shape[-1]
    acc = (x * x).sum(dim=-1, keepdim=True)
    rms = 1.0 / torch.sqrt(acc / d + eps)
    return rms * x * w.to(F64)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``y = x @ w.T`` with ``w`` stored ``[out, in]``; Llama has no bias.

    llama.cu/src/op/linear.rs:85-89 (the weight is passed transposed);
    no bias for the ``llama`` architecture: llama.cu/src/model/mod.rs:62-64.
    """
    return x.to(F64) @ w.to(F64).T


def rope_tables(n_pos: int, head_dim: int, theta: float):
    """Sine and cosine tables ``[n_pos, head_dim/2]``.

    llama.cu/src/model/mod.rs:200-209: in 32-bit, ``freq_i = theta^(-(2i/dh))``, the angle
    is ``pos as f32 * freq_i``, then sine and cosine of that angle.  The 32-bit product
    is part of the formula (at large positions it differs from a 64-bit angle), so it
    is kept; the sine and cosine of that 32-bit angle are taken in 64-bit.
    """
    half = head_dim // 2
    i = np.arange(half, dtype=np.float32)
    expo = -(np.float32(2.0) * i / np.float32(head_dim))
    freq = np.power(np.float32(theta), expo.astype(np.float32)).astype(np.float32)
    pos = np.arange(n_pos, dtype=np.float32)
    ang = (pos[:, None] * freq[None, :]).astype(np.float32)
    ang64 = ang.astype(np.float64)
    return torch.from_numpy(np.sin(ang64)), torch.from_numpy(np.cos(ang64))


def rope(x: torch.Tensor, pos: Sequence[int], sin: torch.Tensor, cos: torch.Tensor,
         pairing: str) -> torch.Tensor:
    """Rotate every head of ``x [n, heads, dh]`` by the angle of its token's position.

    llama.cu/src/op/rope.cuh:26-34: a pair ``(a, b)`` becomes
    ``(a*cos - b*sin, a*sin + b*cos)``.  The reference pairs neighbours
    ``(x[2i], x[2i+1])`` (``pairing="adjacent"``) because its files hold q/k rows in that
    order; tensors under the names of config.json's ecosystem hold them so that the
    pairs are ``(x[i], x[i+dh/2])`` (``pairing="half"``).  The two differ by a fixed
    reordering of the rows of the q and k projections and by nothing else.
    """
    x = x.to(F64)
    n, heads, dh = x.shape
    half = dh // 2
    out = torch.empty_like(x)
    # pair i is (x[2i], x[2i+1]) or (x[i], x[i + half])
    ia = [2 * i if pairing == "adjacent" else i for i in range(half)]
    ib = [2 * i + 1 if pairing == "adjacent" else i + half for i in range(half)]
    for t in range(n):
        s = sin[int(pos[t])]
        c = cos[int(pos[t])]
        a = x[t][:, ia]                    # [heads, half]: the first element of every pair
        b = x[t][:, ib]
        out[t][:, ia] = a * c - b * s
        out[t][:, ib] = a * s + b * c
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
              first_pos: int = 0, window: Optional[int] = None, rounding: Optional[str] = None) -> torch.Tensor:
    """Causal attention of the queries ``q [nq, nh, dh]`` over the keys ``k, v [nk, nkvh, dh]``.

    The call contract is llama.cu/src/exec/step.rs:162-178: causal mask with the
    request's position as offset, so the query at absolute position ``p`` sees keys
    ``0..p``.  Query ``t`` stands at ``first_pos + t``; key ``j`` stands at ``j``.  The
    operator itself lies outside the reference's tree; taken as usual: head ``h`` reads
    the key/value head ``h // (nh/nkvh)``, scores are scaled by ``scale``
    (``dh**-0.5`` for Llama), softmax over the visible keys.  ``window`` (not used by
    Llama) limits a query to the last ``window`` keys, itself included.  ``rounding``: the
    weights ``exp(s - max)`` are rounded to that type before they multiply the values, and the
    sum that divides them is that of the unrounded weights.
    """
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    nq, nh, dh = q.shape
    nk, nkvh, _ = k.shape
    g = nh // nkvh
    out = torch.zeros(nq, nh, dh, dtype=F64)
    for t in range(nq):
        p = first_pos + t
        lo = 0 if window is None else max(0, p - window + 1)
        for h in range(nh):
            kv = h // g
            s = (k[lo:p + 1, kv, :] @ q[t, h, :]) * scale
            s = s - s.max()
            e = torch.exp(s)
            if rounding is None:
                a = e / e.sum()
                out[t, h, :] = a @ v[lo:p + 1, kv, :]
            else:
                out[t, h, :] = (rounded(e, rounding) @ v[lo:p + 1, kv, :]) / e.sum()
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``gate * sigmoid(gate) * up`` with ``sigmoid(z) = 1 / (1 + exp(-z))``.

    llama.cu/src/op/swiglu.cuh:1-3,17-19.
    """
    gate, up = gate.to(F64), up.to(F64)
    return gate * (1.0 / (1.0 + torch.exp(-gate))) * up


# --------------------------------------------------------------------------- model


@dataclass
class PlainConfig:
    """The sizes and constants of one Llama model (the keys of its config.json)."""
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rope_theta: float = 1e4          # default: llama.cu/src/model/mod.rs:54
    rms_norm_eps: float = 1e-5       # default: llama.cu/src/model/mod.rs:77
    tie_word_embeddings: bool = False
    rope_pairing: str = "half"
    # not Llama's: used by tests of the parts' generality
    window: Optional[int] = None
    run_order: Optional[List[int]] = None

    @staticmethod
    def from_dict(d: dict) -> "PlainConfig":
        nh = d["num_attention_heads"]
        return PlainConfig(
            num_hidden_layers=d["num_hidden_layers"], hidden_size=d["hidden_size"],
            num_attention_heads=nh,
            num_key_value_heads=d.get("num_key_value_heads", nh),
            head_dim=d.get("head_dim", d["hidden_size"] // nh),
            intermediate_size=d["intermediate_size"], vocab_size=d["vocab_size"],
            max_position_embeddings=d["max_position_embeddings"],
            rope_theta=d.get("rope_theta", 1e4), rms_norm_eps=d.get("rms_norm_eps", 1e-5),
            tie_word_embeddings=d.get("tie_word_embeddings", False),
            rope_pairing="adjacent" if d.get("rope_interleaved", False) else "half")


def attention_block(cfg: PlainConfig, w: Dict[str, torch.Tensor], prefix: str, x1: torch.Tensor,
                    pos: Sequence[int], sin, cos, shared_kv=None, keep_kv: Optional[list] = None,
                    rounding: Optional[str] = None) -> torch.Tensor:
    """q, k, v projections, rotation of q and k, causal attention, output projection,
for one whole sequence: ``pos`` (the positions the rotation uses) may start anywhere,
the mask only counts places in the sequence.

    Weights and shapes: llama.cu/src/model/mod.rs:111-130 (the reference's file holds
    q, k and v as one matrix with rows q, then k, then v; here they are three).
    Rotation of q and k, not v: llama.cu/src/model/mod.rs:120-124.
    """
    n = x1.shape[0]
    nh, nkvh, dh = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    R = lambda t: rounded(t, rounding)
    q = R(linear(x1, w[prefix + "self_attn.q_proj.weight"])).view(n, nh, dh)
    q = R(rope(q, pos, sin, cos, cfg.rope_pairing))
    if shared_kv is not None:          # not Llama's: a layer that reads the keys and values another one made
        k, v = shared_kv
    else:
        k = R(linear(x1, w[prefix + "self_attn.k_proj.weight"])).view(n, nkvh, dh)
        v = R(linear(x1, w[prefix + "self_attn.v_proj.weight"])).view(n, nkvh, dh)
        k = R(rope(k, pos, sin, cos, cfg.rope_pairing))
    if keep_kv is not None:
        keep_kv.append((k, v))
    o = R(attention(q, k, v, dh ** -0.5, first_pos=0, window=cfg.window, rounding=rounding))
    return R(linear(o.reshape(n, nh * dh), w[prefix + "self_attn.o_proj.weight"]))


def feed_forward(w: Dict[str, torch.Tensor], prefix: str, x2: torch.Tensor, rounding: Optional[str] = None) -> torch.Tensor:
    """``down(swiglu(gate(x), up(x)))``: llama.cu/src/model/mod.rs:140-154 (gate rows
    first, then up, in the reference's one matrix; here two)."""
    R = lambda t: rounded(t, rounding)
    gate = R(linear(x2, w[prefix + "mlp.gate_proj.weight"]))
    up = R(linear(x2, w[prefix + "mlp.up_proj.weight"]))
    return R(linear(R(swiglu(gate, up)), w[prefix + "mlp.down_proj.weight"]))


def forward(cfg: PlainConfig, w: Dict[str, torch.Tensor], tokens: Sequence[int],
            logits_at: Optional[Sequence[int]] = None, rounding: Optional[str] = None,
            states: Optional[list] = None) -> torch.Tensor:
    """Logits ``[n, vocab]`` at every position of one whole sequence that starts at 0
    (``logits_at``: at these positions only, ``[len(logits_at), vocab]``: the output selects
    its rows before the final norm, llama.cu/src/exec/output_head.rs:74-78).

    Block: ``x += attn(norm1(x)); x += ffn(norm2(x))``
    (llama.cu/src/model/mod.rs:100-157: ``TransformerBlk::new(norm, attention, norm, mlp)``,
    the residual is added in the output and down projections: llama.cu/src/op/linear.rs:35-62).
    Output: final norm, then the output matrix, which is the embedding table when the
    file holds none (llama.cu/src/model/mod.rs:83-88,158-168; llama.cu/src/exec/output_head.rs:80-100).

    ``rounding="bfloat16"``: the model of an engine that keeps its activations in bfloat16, as the reference keeps
    them in float16 (llama.cu/src/model/mod.rs:78: the activations' type is the matrices'): what a norm, a
    projection, the rotation, the attention and the activation function give is rounded to that type where it is
    stored, the softmax's weights before they multiply the values; sums inside a product, the residual stream
    and the logits are not.  ``states``: a list that takes the residual stream ``[n, d]`` before every entry of
    the run order and after the last.
    """
    n = len(tokens)
    pos = list(range(n))
    sin, cos = rope_tables(max(n, 1), cfg.head_dim, cfg.rope_theta)
    x = embedding(w["model.embed_tokens.weight"], tokens)
    # Llama runs its layers once each, in order; tests of the parts' generality may name a
    # layer twice, or as (layer, j) let it read the keys and values that entry j made
    order = cfg.run_order if cfg.run_order is not None else list(range(cfg.num_hidden_layers))
    kept = []
    for entry in order:
        layer, cache_of = entry if isinstance(entry, tuple) else (entry, None)
        p = f"model.layers.{layer}."
        if states is not None:
            states.append(x.clone())
        x1 = rounded(rms_norm(x, w[p + "input_layernorm.weight"], cfg.rms_norm_eps), rounding)
        made = []
        x = x + attention_block(cfg, w, p, x1, pos, sin, cos,
                                shared_kv=kept[cache_of] if cache_of is not None else None, keep_kv=made, rounding=rounding)
        kept.append(made[0] if cache_of is None else None)
        x2 = rounded(rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps), rounding)
        x = x + feed_forward(w, p, x2, rounding=rounding)
    if states is not None:
        states.append(x.clone())
    if logits_at is not None:
        x = x[list(logits_at)]
    y = rounded(rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps), rounding)
    head = w["model.embed_tokens.weight"] if (cfg.tie_word_embeddings or "lm_head.weight" not in w) \
        else w["lm_head.weight"]
    return linear(y, head)


# --------------------------------------------------------------------------- sampling


def sample(logits: torch.Tensor, temperature: float, top_p: float, top_k: int, u: float) -> int:
    """One token from one row of logits.

    Greedy when ``temperature == 0`` or ``top_k == 1``
    (llama.cu/src/op/random_sample/mod.rs:80-82): the largest logit, the lowest index
    among equals.  Otherwise llama.cu/src/op/random_sample/sample.cuh:186-207 and :71-87:
    sort descending (stable), ``w_0 = 1``, ``w_i = exp((l_i - l_0)/T)``, inclusive
    prefix sums ``c``, ``p = u * min(top_p * c[n-1], c[top_k-1])``, the first ``i`` with
    ``c[i] >= p``; the answer is that entry's index before sorting.
    """
    logits = logits.to(F64)
    n = logits.numel()
    if temperature == 0 or top_k == 1:
        return int(torch.argmax(logits))          # first maximal index
    order = torch.sort(logits, descending=True, stable=True).indices
    srt = logits[order]
    wgt = torch.exp((srt - srt[0]) / temperature)
    wgt[0] = 1.0
    c = torch.cumsum(wgt, 0)
    k = min(top_k, n)
    p = u * min(top_p * float(c[n - 1]), float(c[k - 1]))
    i = int(torch.nonzero(c >= p)[0])
    return int(order[i])


def greedy_generate(cfg: PlainConfig, w: Dict[str, torch.Tensor], prompt: Sequence[int],
                    steps: int) -> List[int]:
    """``steps`` greedy tokens after ``prompt``, each from a whole forward pass."""
    toks = list(prompt)
    out = []
    for _ in range(steps):
        nxt = int(torch.argmax(forward(cfg, w, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out


# --------------------------------------------------------------------------- files


def random_weights(cfg: PlainConfig, seed: int, std: float = 0.02) -> Dict[str, torch.Tensor]:
    """Random weights under the tensor names of a Llama model folder (the test's own
    generator: matrices N(0, std), norm weights 1 + N(0, std))."""
    g = torch.Generator().manual_seed(seed)
    d, dh = cfg.hidden_size, cfg.head_dim
    nh, nkvh, di = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.intermediate_size
    w: Dict[str, torch.Tensor] = {}

    def mat(name, rows, cols):
        w[name] = torch.randn(rows, cols, generator=g, dtype=torch.float32) * std

    def vec(name, size):
        w[name] = 1.0 + torch.randn(size, generator=g, dtype=torch.float32) * std

    mat("model.embed_tokens.weight", cfg.vocab_size, d)
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        vec(p + "input_layernorm.weight", d)
        mat(p + "self_attn.q_proj.weight", nh * dh, d)
        mat(p + "self_attn.k_proj.weight", nkvh * dh, d)
        mat(p + "self_attn.v_proj.weight", nkvh * dh, d)
        mat(p + "self_attn.o_proj.weight", d, nh * dh)
        vec(p + "post_attention_layernorm.weight", d)
        mat(p + "mlp.gate_proj.weight", di, d)
        mat(p + "mlp.up_proj.weight", di, d)
        mat(p + "mlp.down_proj.weight", d, di)
    vec("model.norm.weight", d)
    if not cfg.tie_word_embeddings:
        mat("lm_head.weight", cfg.vocab_size, d)
    return w


_ST_DTYPES = {"F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2),
              "I32": (torch.int32, 4), "F64": (torch.float64, 8)}


def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """A safetensors file read by its published layout: 8 bytes of little-endian header
    length, a JSON header ``{name: {dtype, shape, data_offsets}}``, then the raw data."""
    with open(path, "rb") as f:
        raw = f.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    base = 8 + hlen
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        dt, _ = _ST_DTYPES[info["dtype"]]
        a, b = info["data_offsets"]
        buf = bytearray(raw[base + a: base + b])
        t = torch.frombuffer(buf, dtype=dt) if b > a else torch.empty(0, dtype=dt)
        out[name] = t.view(*info["shape"]).clone()
    return out


def load_folder(folder: str):
    """(PlainConfig, weights) of a model folder (config.json, model.safetensors)."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = PlainConfig.from_dict(json.load(f))
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))
