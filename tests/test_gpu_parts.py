"""Each part of a layer alone against its plain formula, and the generality of the
composition: a run order that names a layer twice and lets a layer read another's cache,
a window with pages of its own, and a toy mixer with per-request state that is defined
here, registered, built and stepped without a change to the framework."""
import copy
import os

import pytest
import torch

import common
import plain
from test_gpu_kernels import Batch, close, rnd

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def build_ctx(dtype, page=16, max_pos=512):
    from llama_cu_amd.parts import BuildContext
    return BuildContext(DT[dtype], torch.device("cuda:0"), max_pos, page)


def random_part_tensors(part, seed, dtype, std=0.2):
    from llama_cu_amd.weights import random_tensors
    return random_tensors(part.tensors(), seed, dtype=DT[dtype], std=std, device="cuda")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_part(dtype):
    from llama_cu_amd.parts import PartSpec, make_part
    part = make_part("norm", PartSpec("rmsnorm", {"size": 100, "eps": 1e-3}))
    t = random_part_tensors(part, 1, dtype)
    part.load(t, build_ctx(dtype))
    x = rnd(7, 100, seed=1, scale=0.02)
    delta = rnd(7, 100, seed=2, scale=0.02).to(DT[dtype])
    xg = x.cuda()
    y = part.forward(xg, delta.cuda())
    want_x = x.double() + delta.double()
    close(xg, want_x, "float32")
    close(y, plain.rms_norm(want_x, t["weight"].cpu(), 1e-3), dtype)
    assert y.dtype == DT[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_part(dtype):
    from llama_cu_amd.parts import PartSpec, make_part
    for n in (3, 70):                                   # few rows (the fused kernel) and many
        part = make_part("ffn", PartSpec("swiglu", {"hidden_size": 48, "intermediate_size": 100}))
        t = random_part_tensors(part, 2, dtype)
        part.load(dict(t), build_ctx(dtype))
        h = rnd(n, 48, seed=3).to(DT[dtype])
        w = {"L.mlp." + k: v.cpu() for k, v in t.items()}
        close(part.forward(h.cuda()), plain.feed_forward(w, "L.", h), dtype)


@pytest.mark.parametrize("inner,packed", [(56, False), (24, False), (96, True), (352, True)])
def test_feed_forward_whose_width_allows_a_packed_copy_but_whose_halves_may_not(inner, packed):
    """A width of whole blocks of 128: the matrices may get a copy in the order the decode kernel streams.
    Gate and up are one matrix of 2 x inner rows, which is whole blocks of 16 rows for inner = 56 too, but
    its halves are not: such a matrix must stay unpacked (the kernel pairs row i of the one half with row i
    of the other, block by block), and every number of rows must give the plain formula's result."""
    from llama_cu_amd.parts import PartSpec, make_part
    part = make_part("ffn", PartSpec("swiglu", {"hidden_size": 128, "intermediate_size": inner}))
    t = random_part_tensors(part, 4, "bfloat16", std=0.05)
    part.load(dict(t), build_ctx("bfloat16"))
    assert (part.w_gate_up.packed is not None) == packed
    w = {"L.mlp." + k: v.cpu() for k, v in t.items()}
    for n in (1, 8, 20, 70, 200):
        h = rnd(n, 128, seed=n).to(torch.bfloat16)
        close(part.forward(h.cuda()), plain.feed_forward(w, "L.", h), "bfloat16", f"{n} rows")


@pytest.mark.parametrize("pack", [True, False])
def test_feed_forward_with_rows_of_zeros_for_the_library(monkeypatch, pack):
    """Where the library's product is faster with more output features, each half of the plain
    gate/up matrix gets rows of zeros; the copy that the decode kernels stream does not, and what
    the zeros give is left out before the down projection: few rows, 17 to 128 and many rows give
    what the plain formula gives."""
    import llama_cu_amd.parts.ffn as ffn
    from llama_cu_amd.parts import BuildContext, PartSpec, make_part
    monkeypatch.setattr(ffn, "library_friendly_rows", lambda di, d, device: di + 96)
    part = make_part("ffn", PartSpec("swiglu", {"hidden_size": 128, "intermediate_size": 8288}))
    t = random_part_tensors(part, 2, "bfloat16", std=0.05)
    part.load(dict(t), BuildContext(torch.bfloat16, torch.device("cuda:0"), 512, 16, pack))
    assert part.w_gate_up.plain.shape == (2 * (8288 + 96), 128)
    assert (part.w_gate_up.packed is not None) == pack and (not pack or part.w_gate_up.packed.shape == (2 * 8288, 128))
    w = {"L.mlp." + k: v.cpu() for k, v in t.items()}
    for n in (3, 20, 70, 200):
        h = rnd(n, 128, seed=n).to(torch.bfloat16)
        got = part.forward(h.cuda())
        assert got.shape == (n, 128)
        close(got, plain.feed_forward(w, "L.", h), "bfloat16", f"{n} rows")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("interleaved", [False, True])
def test_attention_mixer_part_whole_prompt_then_decode(dtype, interleaved):
    """The mixer alone: a whole prompt, then two single tokens from its cache, against the
    plain attention block on the whole sequence."""
    from llama_cu_amd.engine.runner import LayerCache
    from llama_cu_amd.parts import PartSpec, make_part
    d, nh, nkv, dh, page = 80, 6, 2, 32, 16
    pos_spec = PartSpec("rotary", {"head_dim": dh, "theta": 777.0, "max_positions": 64, "interleaved": interleaved})
    part = make_part("mixer", PartSpec("attention", {"hidden_size": d, "heads": nh, "kv_heads": nkv, "head_dim": dh,
                                                     "position": pos_spec}))
    t = random_part_tensors(part, 3, dtype)
    part.load(dict(t), build_ctx(dtype, page, 64))
    cfg = plain.PlainConfig(1, d, nh, nkv, dh, 1, 1, 64, rope_theta=777.0, rope_pairing="adjacent" if interleaved else "half")
    w = {"L.self_attn." + k: v.cpu() for k, v in t.items()}
    n = 21
    h = rnd(n, d, seed=4).to(DT[dtype])
    sin, cos = plain.rope_tables(64, dh, 777.0)
    want = plain.attention_block(cfg, w, "L.", h, list(range(n)), sin, cos)
    cache = LayerCache(group=0, pages=torch.zeros(4, 2, nkv * dh * page, dtype=DT[dtype], device="cuda"))
    table = [2, 0, 3]

    def step(q_len, ctx_len):
        s = Batch([q_len], [ctx_len], [table], 4).step
        first = ctx_len - q_len
        s.positions = torch.arange(first, ctx_len, dtype=torch.int32).cuda()
        s.slot_maps = [torch.tensor([table[p // page] * page + p % page for p in range(first, ctx_len)], dtype=torch.int32).cuda()]
        return s

    got = [part.forward(h[:n - 2].cuda(), step(n - 2, n - 2), cache)]
    got.append(part.forward(h[n - 2:n - 1].cuda(), step(1, n - 1), cache))
    got.append(part.forward(h[n - 1:].cuda(), step(1, n), cache))
    close(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_and_output_parts(dtype):
    from llama_cu_amd.parts import PartSpec, make_part
    emb = make_part("embedding", PartSpec("tokens", {"vocab_size": 301, "hidden_size": 40}))
    t = random_part_tensors(emb, 5, dtype)
    emb.load(dict(t), build_ctx(dtype))
    ids = torch.tensor([300, 0, 17], dtype=torch.int32)
    x = emb.forward(ids.cuda())
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), t["weight"].cpu().float()[ids.long()])
    for tied in (True, False):
        head = make_part("head", PartSpec("linear", {"vocab_size": 301, "hidden_size": 40, "tied": tied}))
        own = random_part_tensors(emb, 6, dtype)
        head.load({} if tied else {"weight": own["weight"]}, build_ctx(dtype), table=emb.weight)
        y = rnd(3, 40, seed=7).to(DT[dtype])
        logits = head.forward(y.cuda())
        assert logits.dtype == torch.float32
        close(logits, plain.linear(y, (t if tied else own)["weight"].cpu()), dtype)


# ----------------------------------------------------------------------------- whole models from custom layouts
def runner_for(spec, seed, dtype, std=0.15, **kw):
    from llama_cu_amd.engine.runner import ModelRunner
    from llama_cu_amd.parts import DecoderModel
    from llama_cu_amd.weights import random_tensors
    tensors = random_tensors(DecoderModel(spec).tensors(), seed, dtype=DT[dtype], std=std, device="cuda")
    kw.setdefault("max_tokens", 1024)
    return ModelRunner(spec, dict(tensors), dtype, **kw), {k: v.cpu() for k, v in tensors.items()}


def run_cut(runner, toks, sizes, rid=0):
    """Feed ``toks`` in portions of the given sizes; logits at every position."""
    out, fed, i = [], 0, 0
    while fed < len(toks):
        n = min(sizes[i % len(sizes)], len(toks) - fed)
        i += 1
        out.append(runner.step([rid], [toks[fed:fed + n]], [list(range(n))]).cpu())
        fed += n
    runner.end(rid)
    return torch.cat(out)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_run_order_names_a_layer_twice_and_shares_a_cache(dtype):
    """Run order: layer 0, layer 1, layer 0 again (with a cache of its own), then layer 2,
    which has no key and value projections and reads the cache of the second entry."""
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import RunEntry
    cfg_d = dict(common.TINY_A, num_hidden_layers=3)
    spec = llama_spec(LlamaConfig.from_dict(cfg_d))
    spec.layers[2].params["mixer"].params["shares_kv"] = True
    spec.run_order = [RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(2, cache_of=1)]
    std = 0.15 if dtype == "float32" else common.BF16_STD
    runner, w = runner_for(spec, 3, dtype, std=std)
    assert "model.layers.2.self_attn.k_proj.weight" not in w
    assert runner.caches[3].pages is runner.caches[1].pages and not runner.caches[3].writes
    assert runner.caches[2].pages is not runner.caches[0].pages
    toks = common.random_requests(256, [90], 4)["r0"]
    pcfg = plain.PlainConfig.from_dict(cfg_d)
    pcfg.run_order = [0, 1, 0, (2, 1)]
    want = plain.forward(pcfg, w, toks)
    for sizes in ([90], [58, 1, 1, 7, 2, 16]):
        got = run_cut(runner, toks, sizes)
        err = float((got.double() - want).abs().max()) / float(want.abs().max())
        assert err <= common.REL_TOL[dtype], (sizes, err)
    with pytest.raises(ValueError, match="before"):
        from llama_cu_amd.parts import DecoderModel
        bad = copy.copy(spec)
        bad.run_order = [RunEntry(0, cache_of=1), RunEntry(1)]
        DecoderModel(bad)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_with_pages_of_its_own(dtype):
    """Layer 0 attends to all keys, layer 1 to the last 24: two groups of pages; the
    window's group gives pages back as the window passes them, and the logits are those of
    the plain implementation with the same window."""
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.models.llama import llama_spec
    cfg_d = dict(common.TINY_B, num_hidden_layers=2, head_dim=64, num_attention_heads=2, num_key_value_heads=1)
    spec = llama_spec(LlamaConfig.from_dict(cfg_d))
    spec.layers[1].params["mixer"].params["window"] = 24
    std = 0.15 if dtype == "float32" else common.BF16_STD
    runner, w = runner_for(spec, 5, dtype, std=std, max_tokens=256)
    assert [g.window for g in runner.groups] == [0, 24]
    assert runner.caches[0].group == 0 and runner.caches[1].group == 1
    toks = common.random_requests(384, [150], 6)["r0"]
    # the plain model with a window in layer 1 only
    pcfg = plain.PlainConfig.from_dict(cfg_d)
    sin, cos = plain.rope_tables(150, pcfg.head_dim, pcfg.rope_theta)
    x = plain.embedding(w["model.embed_tokens.weight"], toks)
    for layer, window in ((0, None), (1, 24)):
        p = f"model.layers.{layer}."
        pcfg.window = window
        x = x + plain.attention_block(pcfg, w, p, plain.rms_norm(x, w[p + "input_layernorm.weight"], pcfg.rms_norm_eps),
                                      list(range(150)), sin, cos)
        x = x + plain.feed_forward(w, p, plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], pcfg.rms_norm_eps))
    want = plain.linear(plain.rms_norm(x, w["model.norm.weight"], pcfg.rms_norm_eps), w["model.embed_tokens.weight"])
    for sizes in ([150], [100, 1, 1, 1, 30, 2], [1]):
        out, fed, i = [], 0, 0
        while fed < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - fed)
            i += 1
            out.append(runner.step([7], [toks[fed:fed + n]], [list(range(n))]).cpu())
            fed += n
            held = [p for p in runner.cache.table(7, 1) if p >= 0]
            assert len(held) <= (24 + 15) // 16 + 1             # the window's group holds a window's worth of pages
            assert all(p >= 0 for p in runner.cache.table(7, 0))
        runner.end(7)
        got = torch.cat(out)
        err = float((got.double() - want).abs().max()) / float(want.abs().max())
        assert err <= common.REL_TOL[dtype], (sizes, err)
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_with_pages_of_its_own_size(dtype):
    """Layer 1 asks for pages of 32 tokens while the engine's are 16: its keys and values get a pool of
    their own, with its own block table, and the logits are those of the plain implementation; a mixed
    replay gives all pages of both pools back."""
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.engine.trace import TraceReplayer
    from llama_cu_amd.models.llama import llama_spec
    cfg_d = dict(common.TINY_B, num_hidden_layers=2, head_dim=64, num_attention_heads=2, num_key_value_heads=1)
    spec = llama_spec(LlamaConfig.from_dict(cfg_d))
    spec.layers[1].params["mixer"].params["page_size"] = 32
    std = 0.15 if dtype == "float32" else common.BF16_STD
    reqs = common.random_requests(384, [70, 33, 120, 9], 4)
    steps, max_tokens = common.trace_mixed(reqs, seed=1, max_live=3)
    runner, w = runner_for(spec, 6, dtype, std=std, max_tokens=max_tokens, max_seqs=4, max_batch_tokens=max_tokens, page_size=16)
    assert [(g.page_size, g.num_pages) for g in runner.groups] == [(16, max_tokens // 16), (32, max_tokens // 32)]
    assert runner.caches[0].pages.shape[2] == 64 * 16 and runner.caches[1].pages.shape[2] == 64 * 32
    pcfg = plain.PlainConfig.from_dict(cfg_d)
    want = {name: plain.forward(pcfg, w, toks) for name, toks in reqs.items()}
    rep = TraceReplayer(runner)
    outputs = {}
    for st in steps:
        out = rep.step(st)
        if out is not None:
            outputs[st["step"]] = out
    common.assert_matches_plain(common.collect(steps, outputs, 384), want, dtype, "pages of 16 and 32")
    runner.cache.check()
    assert [runner.cache.free_pages(g) for g in range(2)] == [max_tokens // 16, max_tokens // 32]


# ----------------------------------------------------------------------------- a toy mixer with state of its own
def toy_mean_direct(cfg_d, w, toks):
    """The logits of the toy model whose layer 1 mixes with a running mean (layer 0 is a Llama layer), computed
    directly from the plain implementation's functions."""
    pcfg = plain.PlainConfig.from_dict(cfg_d)
    sin, cos = plain.rope_tables(len(toks), 16, pcfg.rope_theta)
    x = plain.embedding(w["model.embed_tokens.weight"], toks)
    p = "model.layers.0."
    x = x + plain.attention_block(pcfg, w, p, plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5), list(range(len(toks))), sin, cos)
    x = x + plain.feed_forward(w, p, plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5))
    p = "model.layers.1."
    h = plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
    mean = torch.cumsum(h, 0) / torch.arange(1, len(toks) + 1, dtype=torch.float64)[:, None]
    x = x + mean @ w[p + "toy.mix.weight"].double().T
    x = x + plain.feed_forward(w, p, plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5))
    return plain.linear(plain.rms_norm(x, w["model.norm.weight"], 1e-5), w["lm_head.weight"])


def test_a_toy_mixer_with_state_is_registered_built_and_stepped():
    """The mixer ``running_mean`` is defined here: its output at a token is a matrix times
    the mean of its inputs up to that token.  Its state per request (the running sum, of
    fixed size) lives in the engine's state slots.  It is registered, laid into a model
    beside an attention layer, and stepped whole, in portions, token by token and mixed
    with other requests whose slots are used again; all agree with a direct computation."""
    import llama_cu_amd
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import Part, PartSpec, SlotState, TensorSpec, register_part

    class RunningMean(Part):
        def __init__(self, hidden_size):
            self.d = hidden_size

        def tensors(self):
            return {"mix.weight": TensorSpec((self.d, self.d))}

        def cache_need(self):
            return SlotState((self.d,), torch.float32)

        def load(self, tensors, build):
            self.w = tensors["mix.weight"].float()
            self.dtype = build.dtype

        def forward(self, h, step, cache):
            out = torch.empty_like(h)
            start = 0
            for r, n in enumerate(step.q_lens):
                slot = step.state_slots[r]
                first = step.ctx_lens[r] - n
                if first == 0:
                    cache.state[slot].zero_()                     # a new request in this slot
                sums = cache.state[slot] + torch.cumsum(h[start:start + n].float(), 0)
                counts = torch.arange(first + 1, first + n + 1, device=h.device, dtype=torch.float32)[:, None]
                out[start:start + n] = ((sums / counts) @ self.w.T).to(h.dtype)
                cache.state[slot] = sums[-1]
                start += n
            return out

    register_part("mixer", "running_mean", RunningMean, replace=True)
    cfg_d = dict(common.TINY_A)
    cfg = LlamaConfig.from_dict(cfg_d)
    spec = llama_spec(cfg)
    spec.layers[1].params["mixer"] = PartSpec("running_mean", {"hidden_size": 64}, "toy")
    runner, w = runner_for(spec, 9, "float32", max_tokens=512, max_seqs=3)
    assert "model.layers.1.toy.mix.weight" in w and "model.layers.1.self_attn.q_proj.weight" not in w
    assert runner.caches[1].state.shape == (3, 64) and runner.caches[1].pages is None
    assert not runner.use_graphs                # the toy reads lengths on the host: its steps are not captured

    def direct(toks):
        return toy_mean_direct(cfg_d, w, toks)

    reqs = common.random_requests(256, [40, 9, 77, 30, 5], 12)
    want = {k: direct(v) for k, v in reqs.items()}
    for mode in (common.trace_whole, common.trace_portions, common.trace_tail_decode, lambda r: common.trace_mixed(r, max_live=3)):
        steps, _ = mode(reqs)
        ids, outputs = {}, {}
        for st in steps:
            es = st["entries"]
            logits = runner.step([ids.setdefault(e["id"], len(ids)) for e in es], [e["tokens"] for e in es], [e["want"] for e in es])
            outputs[st["step"]] = logits.cpu().numpy()
            for name in st["end"]:
                runner.end(ids[name])
        got = common.collect(steps, outputs, 256)
        common.assert_matches_plain(got, want, "float32", "toy mixer")
    runner.cache.check()
    assert runner.cache.free_slots() == 3


def test_a_toy_routed_feed_forward_and_a_toy_position_encoding_are_registered_and_stepped():
    """Two more parts defined here and not in the package.  ``pick_one``: a feed-forward that
    routes each token to the one of its experts whose router score is largest (the score in
    32-bit) and scales the expert's output by the softmax weight of that score.  ``key_shift``:
    a position encoding that is no rotation: it adds ``sin(pos / 7)`` times a learned vector to
    every query and key head before the cache write.  Layer 0 gets the position encoding and
    keeps SwiGLU, layer 1 keeps the rotation and gets the routed feed-forward; the model is
    stepped whole, in portions, token by token and mixed, and agrees with a direct computation."""
    import llama_cu_amd
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import Part, PartSpec, TensorSpec, register_part

    class PickOne(Part):
        graph_safe = True

        def __init__(self, hidden_size, inner, experts):
            self.d, self.di, self.e = hidden_size, inner, experts

        def tensors(self):
            return {"router.weight": TensorSpec((self.e, self.d)), "w_in": TensorSpec((self.e * self.di, self.d)),
                    "w_out": TensorSpec((self.e * self.d, self.di))}

        def load(self, tensors, build):
            self.router = tensors["router.weight"].float()
            self.w_in = tensors["w_in"].float().view(self.e, self.di, self.d)
            self.w_out = tensors["w_out"].float().view(self.e, self.d, self.di)
            self.dtype = build.dtype

        def forward(self, h):
            x = h.float()
            scores = torch.softmax(x @ self.router.T, dim=-1)                    # router in 32-bit
            weight, which = scores.max(dim=-1)
            inner = torch.relu(torch.einsum("nd,nid->ni", x, self.w_in[which]))
            return (torch.einsum("ni,ndi->nd", inner, self.w_out[which]) * weight[:, None]).to(self.dtype)

    class KeyShift(Part):
        graph_safe = True

        def __init__(self, head_dim):
            self.dh = head_dim

        def tensors(self):
            return {}

        def load(self, tensors, build):
            g = torch.Generator().manual_seed(77)
            self.vec = (torch.randn(self.dh, generator=g) * 0.5).to(build.device)

        def rotary_tables(self):
            return None

        def apply(self, qkv, positions, heads, kv_heads, head_dim):
            n = qkv.shape[0]
            shift = torch.sin(positions.float() / 7.0)[:, None, None] * self.vec[None, None, :]
            qk = qkv[:, :(heads + kv_heads) * head_dim].view(n, heads + kv_heads, head_dim)
            qk += shift.to(qkv.dtype)

    register_part("ffn", "pick_one", PickOne, replace=True)
    register_part("position", "key_shift", KeyShift, replace=True)
    cfg_d = dict(common.TINY_A)
    cfg = LlamaConfig.from_dict(cfg_d)
    spec = llama_spec(cfg)
    spec.layers[0].params["mixer"].params["position"] = PartSpec("key_shift", {"head_dim": 16})
    spec.layers[1].params["ffn"] = PartSpec("pick_one", {"hidden_size": 64, "inner": 40, "experts": 3}, "moe")
    runner, w = runner_for(spec, 13, "float32", max_tokens=512, max_seqs=3)
    assert "model.layers.1.moe.router.weight" in w and "model.layers.1.mlp.gate_proj.weight" not in w
    vec = runner.model.layers[0].mixer.position.vec.double().cpu()

    def direct(toks):
        pcfg = plain.PlainConfig.from_dict(cfg_d)
        n = len(toks)
        pos = list(range(n))
        sin, cos = plain.rope_tables(n, 16, pcfg.rope_theta)
        x = plain.embedding(w["model.embed_tokens.weight"], toks)
        # layer 0: attention whose queries and keys are shifted, not rotated
        p = "model.layers.0."
        h = plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
        shift = torch.sin(torch.tensor(pos, dtype=torch.float32) / 7.0).double()[:, None, None] * vec[None, None, :]
        q = plain.linear(h, w[p + "self_attn.q_proj.weight"]).view(n, 4, 16) + shift
        k = plain.linear(h, w[p + "self_attn.k_proj.weight"]).view(n, 4, 16) + shift
        v = plain.linear(h, w[p + "self_attn.v_proj.weight"]).view(n, 4, 16)
        o = plain.attention(q, k, v, 16 ** -0.5, first_pos=0, window=None)
        x = x + plain.linear(o.reshape(n, 64), w[p + "self_attn.o_proj.weight"])
        x = x + plain.feed_forward(w, p, plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5))
        # layer 1: Llama's attention, then the routed feed-forward
        p = "model.layers.1."
        x = x + plain.attention_block(pcfg, w, p, plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5), pos, sin, cos)
        h = plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
        scores = torch.softmax(h @ w[p + "moe.router.weight"].double().T, dim=-1)
        weight, which = scores.max(dim=-1)
        w_in = w[p + "moe.w_in"].double().view(3, 40, 64)
        w_out = w[p + "moe.w_out"].double().view(3, 64, 40)
        out = torch.stack([w_out[e] @ torch.relu(w_in[e] @ h[t]) * weight[t] for t, e in enumerate(which.tolist())])
        x = x + out
        return plain.linear(plain.rms_norm(x, w["model.norm.weight"], 1e-5), w["lm_head.weight"]), scores

    reqs = common.random_requests(256, [40, 9, 77, 30], 14)
    want = {}
    for name, toks in reqs.items():
        logits, scores = direct(toks)
        top2 = scores.topk(2, dim=-1).values
        # a token whose two best experts are nearly tied may go either way in 32-bit: none here
        assert float((top2[:, 0] - top2[:, 1]).min()) > 1e-4, "choose another seed: a routing tie"
        want[name] = logits
    for mode in (common.trace_whole, common.trace_portions, common.trace_tail_decode, lambda r: common.trace_mixed(r, max_live=3)):
        steps, _ = mode(reqs)
        ids, outputs = {}, {}
        for st in steps:
            es = st["entries"]
            logits = runner.step([ids.setdefault(e["id"], len(ids)) for e in es], [e["tokens"] for e in es], [e["want"] for e in es])
            outputs[st["step"]] = logits.cpu().numpy()
            for name in st["end"]:
                runner.end(ids[name])
        got = common.collect(steps, outputs, 256)
        common.assert_matches_plain(got, want, "float32", "toy parts")
    runner.cache.check()


def test_a_toy_position_encoding_that_is_a_bias_inside_the_scores():
    """A third kind of position encoding, defined here and not in the package: nothing is done to
    queries and keys; instead every head adds ``slope[h] * (key position - query position)`` to its
    scaled scores (the part hands the slopes to the mixer through ``score_slopes()``).  Layer 0 gets
    it, layer 1 keeps the rotation; whole, in portions, token by token and mixed against a direct
    computation.  With slopes this steep the far keys hardly count: a kernel that left the bias out
    would be far off."""
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import Part, PartSpec, register_part

    class DistanceBias(Part):
        graph_safe = True

        def __init__(self, heads):
            self.heads = heads

        def tensors(self):
            return {}

        def load(self, tensors, build):
            self.slopes = torch.tensor([2.0 ** -(h + 1) for h in range(self.heads)], dtype=torch.float32, device=build.device)

        def rotary_tables(self):
            return None

        def apply(self, qkv, positions, heads, kv_heads, head_dim):
            pass

        def score_slopes(self):
            return self.slopes

    register_part("position", "distance_bias", DistanceBias, replace=True)
    cfg_d = dict(common.TINY_A)
    cfg = LlamaConfig.from_dict(cfg_d)
    spec = llama_spec(cfg)
    spec.layers[0].params["mixer"].params["position"] = PartSpec("distance_bias", {"heads": cfg.num_attention_heads})
    runner, w = runner_for(spec, 17, "float32", max_tokens=512, max_seqs=3)
    nh, nkv, dh = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim

    def direct(toks):
        pcfg = plain.PlainConfig.from_dict(cfg_d)
        n = len(toks)
        pos = list(range(n))
        sin, cos = plain.rope_tables(n, dh, pcfg.rope_theta)
        x = plain.embedding(w["model.embed_tokens.weight"], toks)
        p = "model.layers.0."
        h = plain.rms_norm(x, w[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        q = plain.linear(h, w[p + "self_attn.q_proj.weight"]).view(n, nh, dh).double()
        k = plain.linear(h, w[p + "self_attn.k_proj.weight"]).view(n, nkv, dh).double()
        v = plain.linear(h, w[p + "self_attn.v_proj.weight"]).view(n, nkv, dh).double()
        dist = (torch.arange(n)[None, :] - torch.arange(n)[:, None]).double()          # key position - query position
        o = torch.empty(n, nh, dh, dtype=torch.float64)
        for hd in range(nh):
            sc = q[:, hd] @ k[:, hd // (nh // nkv)].T * dh ** -0.5 + 2.0 ** -(hd + 1) * dist
            sc = sc.masked_fill(dist > 0, float("-inf"))
            o[:, hd] = torch.softmax(sc, dim=-1) @ v[:, hd // (nh // nkv)]
        x = x + plain.linear(o.reshape(n, nh * dh), w[p + "self_attn.o_proj.weight"])
        x = x + plain.feed_forward(w, p, plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps))
        p = "model.layers.1."
        x = x + plain.attention_block(pcfg, w, p, plain.rms_norm(x, w[p + "input_layernorm.weight"], cfg.rms_norm_eps), pos, sin, cos)
        x = x + plain.feed_forward(w, p, plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps))
        return plain.linear(plain.rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps), w["lm_head.weight"])

    reqs = common.random_requests(256, [40, 9, 77, 30], 15)
    want = {name: direct(toks) for name, toks in reqs.items()}
    for mode in (common.trace_whole, common.trace_portions, common.trace_tail_decode, lambda r: common.trace_mixed(r, max_live=3)):
        steps, _ = mode(reqs)
        ids, outputs = {}, {}
        for st in steps:
            es = st["entries"]
            logits = runner.step([ids.setdefault(e["id"], len(ids)) for e in es], [e["tokens"] for e in es], [e["want"] for e in es])
            outputs[st["step"]] = logits.cpu().numpy()
            for name in st["end"]:
                runner.end(ids[name])
        got = common.collect(steps, outputs, 256)
        common.assert_matches_plain(got, want, "float32", "distance bias")
    runner.cache.check()


def _engine_turns(engine, prompt, eos, more, steps, seen=None):
    """A kept request: one turn until the end-of-sequence token, then a turn with ``more``.  ``seen``: takes what
    the request has computed and which pages it holds between the turns."""
    from llama_cu_amd.sampling import GREEDY
    engine.eos = {eos} if eos is not None else set()
    rid = engine.add_request(prompt, GREEDY, steps, keep=True, ignore_eos=eos is None)
    turns = []
    for turn in range(2):
        toks, why = [], None
        while not engine.idle:
            for o in engine.step():
                if o.token is not None:
                    toks.append(o.token)
                why = o.finished or why
        turns.append((toks, why))
        if turn == 0:
            if seen is not None:
                seen["computed"] = engine.sched.info(rid).computed
                seen["pages"] = [len(engine.runner.cache.table(rid, g)) for g in range(len(engine.runner.groups))]
            engine.continue_request(rid, more, steps)
    engine.drop(rid)
    engine.runner.cache.check()
    assert engine.runner.cache.free_slots() == engine.runner.max_seqs
    assert all(engine.runner.cache.free_pages(g) == engine.runner.num_pages for g in range(len(engine.runner.groups)))
    return turns


@pytest.mark.parametrize("kind", ["state", "window"])
def test_an_end_learned_late_with_a_cache_that_cannot_be_cut_back(kind):
    """A toy mixer that folds every token into a state of fixed size, and an attention layer whose
    window of 4 tokens gives a page back with every fourth token, each in layer 1 of Tiny A, through
    the engine that runs ahead: when the end-of-sequence token is learned, one token more has gone
    into the state (or the window has passed a page that the shorter request would see).  The kept
    request's next turn must continue as if that token had never been computed: the tokens of the
    engine that runs ahead equal those of the engine that works in turn, and both equal a request
    that is given the whole context at once."""
    import llama_cu_amd
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.engine.engine import Engine
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import Part, PartSpec, SlotState, TensorSpec, register_part

    class DecayingSum(Part):
        """state <- 0.5 state + h; out = state @ W (a state that cannot be cut back)."""
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
                if step.ctx_lens[r] - n == 0:
                    cache.state[slot].zero_()
                st = cache.state[slot].clone()
                for i in range(n):
                    st = 0.5 * st + h[start + i].float()
                    out[start + i] = (st @ self.w.T).to(h.dtype)
                cache.state[slot] = st
                start += n
            return out

    register_part("mixer", "decaying_sum", DecayingSum, replace=True)
    spec = llama_spec(LlamaConfig.from_dict(dict(common.TINY_A)))
    if kind == "state":
        spec.layers[1].params["mixer"] = PartSpec("decaying_sum", {"hidden_size": 64}, "toy")
    else:
        spec.layers[1].params["mixer"].params["window"] = 4
    prompt = list(common.random_requests(256, [9], seed=3).values())[0]
    more = [7, 8, 9]

    def engine(run_ahead):
        runner, _ = runner_for(spec, 4, "float32", max_tokens=256, max_seqs=2, page_size=8)
        assert runner.can_truncate == (kind == "window")
        return Engine(runner, run_ahead=run_ahead)

    probe = _engine_turns(engine(False), prompt, None, more, 10)[0][0]
    assert len(probe) == 10
    # every place of the end-of-sequence token among the first tokens: with pages of 8 and a window
    # of 4 some of them fall on the step that gives a page back
    for at in range(1, 8):
        eos = probe[at]
        if eos in probe[:at]:
            continue
        want = _engine_turns(engine(False), prompt, eos, more, 10)
        assert want[0] == (probe[:at + 1], "eos")
        e = engine(True)
        seen = {}
        got = _engine_turns(e, prompt, eos, more, 10, seen)
        assert got == want, f"end-of-sequence token at {at}"
        held = len(prompt) + at                  # tokens before the end-of-sequence token
        if kind == "window":
            # the window keeps its pages a token longer than the next query needs, so the one token computed
            # beyond the end is cut away and nothing is computed again
            assert seen["computed"] == held, seen
        else:
            # the state cannot be cut back: the request starts again at its first token, but the pages of the
            # layer that has pages stayed its own
            assert seen["computed"] == 0 and seen["pages"] == [(held + 7) // 8], seen
        # the second turn is what a fresh request with the whole context generates
        fresh = engine(False)
        whole = fresh.generate([prompt + probe[:at + 1] + more], max_steps=len(want[1][0]), ignore_eos=True)[0]
        stop = want[1][0].index(eos) + 1 if eos in want[1][0] else len(want[1][0])
        assert want[1][0][:stop] == whole[:stop]


def test_an_architecture_of_a_module_outside_the_package_through_the_programs(tmp_path):
    """A whole architecture with a part of its own, defined in a module that is no file of the package and named
    with --plugin: ``random-model`` writes its folder, ``bin/trace_run`` replays a mixed trace on it (config.json's
    architecture picks the model, as everywhere) and agrees with a direct computation, ``generate`` generates."""
    import json
    import subprocess
    from llama_cu_amd.weights.safetensors_io import open_safetensors
    name, env = common.write_toy_plugin(str(tmp_path))
    cfg_d = dict(common.TINY_A)
    (tmp_path / "config.json").write_text(json.dumps(dict(cfg_d, architectures=["ToyMeanForCausalLM"], mean_layer=1)))
    tool = os.path.join(common.ROOT, "bin", "llama.cu_amd")
    folder = str(tmp_path / "model")
    made = subprocess.run([tool, "random-model", str(tmp_path / "config.json"), folder, "--plugin", name, "--dtype", "float32", "--std", "0.15",
                           "--seed", "4"], capture_output=True, text=True, env=env, timeout=300)
    assert made.returncode == 0, made.stderr[-2000:]
    w = {n: f.tensor(n).double() for f in open_safetensors(folder) for n in f.names()}
    reqs = common.random_requests(256, [40, 9, 77, 30], 21)
    want = {k: toy_mean_direct(cfg_d, w, v) for k, v in reqs.items()}
    steps, _ = common.trace_mixed(reqs, max_live=3)
    outputs = common.run_trace_program(folder, "float32", steps, 256, 256, extra=["--plugin", name, "--max-live", "3"], env=env)
    common.assert_matches_plain(common.collect(steps, outputs, 256), want, "float32", "architecture of a plugin")
    gen = subprocess.run([tool, "generate", folder, "--plugin", name, "--dtype", "float32", "--max-steps", "6", "-p", "ab"],
                         capture_output=True, text=True, env=env, timeout=300)
    assert gen.returncode == 0 and "n toks = " in gen.stderr + gen.stdout, (gen.stdout + gen.stderr)[-2000:]
