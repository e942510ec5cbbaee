"""Each kernel alone against a plain formula, at other sizes than the engine's tiny
models use: widths and vocabularies that are no power of two, head sizes in steps of 16,
odd group sizes, pages of several sizes, windows, and inputs made so that a fault shows
(one key far back that dominates, poisoned memory where nothing may be read)."""
import math
import random

import numpy as np
import pytest
import torch

import plain

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def close(got, want, dtype, what=""):
    want = want.double()
    scale = float(want.abs().max()) + 1e-30
    err = float((got.double().cpu() - want).abs().max())
    assert math.isfinite(err) and err <= TOL[dtype] * scale, f"{what}: error {err:.3e} vs scale {scale:.3e}"


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


# ------------------------------------------------------------------ rows
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,d,vocab", [(1, 8, 3), (7, 100, 301), (33, 4096, 1000)])
def test_embedding_gather(dtype, n, d, vocab):
    from llama_cu_amd.kernels import ops
    table = rnd(vocab, d, seed=n).to(DT[dtype])
    ids = torch.randint(0, vocab, (n,), dtype=torch.int32)
    out = torch.empty(n, d, dtype=torch.float32, device="cuda")
    ops.embedding_gather(table.cuda(), ids.cuda(), out)
    assert torch.equal(out.cpu(), plain.embedding(table.float(), ids.tolist()).float())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,d,eps", [(1, 16, 1e-5), (5, 172, 1e-6), (3, 4096, 1e-5), (2, 5000, 1e-2)])
@pytest.mark.parametrize("w32", [False, True])
def test_rmsnorm_with_residual_sum(dtype, n, d, eps, w32):
    from llama_cu_amd.kernels import ops
    x = rnd(n, d, seed=1, scale=0.05)
    delta = rnd(n, d, seed=2, scale=0.05).to(DT[dtype])
    w = (1 + rnd(d, seed=3, scale=0.1)).to(torch.float32 if w32 else DT[dtype])
    xg = x.cuda()
    out = torch.empty(n, d, dtype=DT[dtype], device="cuda")
    ops.rmsnorm(xg, w.cuda(), eps, out, delta=delta.cuda())
    xs = x.double() + delta.double()
    close(xg, xs, "float32", "residual sum")            # the sum is 32-bit on both paths
    close(out, plain.rms_norm(xs, w, eps), dtype, "norm")
    out2 = torch.empty_like(out)
    ops.rmsnorm(xg, w.cuda(), eps, out2)                   # no delta: x unchanged
    close(out2, plain.rms_norm(xs, w, eps), dtype, "norm without delta")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,di", [(1, 8), (3, 172), (17, 14336)])
def test_swiglu(dtype, n, di):
    from llama_cu_amd.kernels import ops
    gu = rnd(n, 2 * di, seed=di, scale=3.0).to(DT[dtype])
    out = ops.swiglu(gu.cuda())
    close(out, plain.swiglu(gu[:, :di], gu[:, di:]), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gather_rows_and_residual_add(dtype):
    from llama_cu_amd.kernels import ops
    x = rnd(9, 70, seed=4).to(DT[dtype])
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    assert torch.equal(ops.gather_rows(x.cuda(), rows.cuda()).cpu(), x[rows.long()])
    r = rnd(9, 70, seed=5)
    rg = r.cuda()
    ops.residual_add(rg, x.cuda())
    close(rg, r.double() + x.double(), "float32")


# ------------------------------------------------------------------ matrix products
@pytest.mark.parametrize("a_t,w_t,o_t", [("float32", "float32", "float32"), ("bfloat16", "bfloat16", "bfloat16"),
                                         ("bfloat16", "bfloat16", "float32"), ("bfloat16", "float32", "bfloat16")])
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 172, 64), (65, 301, 100), (130, 64, 352), (2, 1000, 4096)])
def test_gemm_generic(a_t, w_t, o_t, m, n, k):
    from llama_cu_amd.kernels import ops
    a = rnd(m, k, seed=m).to(DT[a_t])
    w = rnd(n, k, seed=n + 1).to(DT[w_t])
    out = ops.gemm_nt(a.cuda(), w.cuda(), out_dtype=DT[o_t])
    close(out, plain.linear(a, w), o_t)


def test_gemm_generic_accumulates_in_32_bit_and_rows_are_independent():
    from llama_cu_amd.kernels import ops
    a, w = rnd(70, 300, seed=1), rnd(50, 300, seed=2)
    c = rnd(70, 50, seed=3)
    cg = c.cuda()
    ops.gemm_nt(a.cuda(), w.cuda(), out=cg, accumulate=True)
    close(cg, c.double() + plain.linear(a, w), "float32")
    # a row's result does not depend on the other rows (bitwise)
    whole = ops.gemm_nt(a.cuda(), w.cuda())
    one = ops.gemm_nt(a[17:18].cuda(), w.cuda())
    assert torch.equal(whole[17:18], one)


def test_float32_product_is_a_true_32_bit_product():
    """Operands 1 + 2^-12: exact in 32-bit, rounded to 1 by any matrix mode with 10 or fewer
    mantissa bits.  Each of the 256 products is 1 + 2^-11 + 2^-24, so the true sum is
    256.125; a reduced-precision mode gives 256."""
    from llama_cu_amd.kernels import ops
    a = torch.full((4, 256), 1.0 + 2.0 ** -12)
    w = torch.full((8, 256), 1.0 + 2.0 ** -12)
    out = ops.gemm_nt(a.cuda(), w.cuda())
    assert float((out.double().cpu() - 256.125).abs().max()) < 1e-3


# ------------------------------------------------------------------ rotation and cache write
def key_offset(kvh, tok, dim, dh, page):
    return ((kvh * (dh // 8) + dim // 8) * page + tok) * 8 + dim % 8


def value_offset(nkv, kvh, tok, dim, dh, page):
    return nkv * dh * page + (kvh * dh + dim) * page + tok


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,dh,page,pairing", [(4, 4, 16, 16, "half"), (6, 2, 48, 8, "adjacent"), (32, 8, 128, 32, "half"),
                                                     (3, 1, 80, 24, "adjacent")])
def test_rope_and_cache_write(dtype, nh, nkv, dh, page, pairing):
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.position import Rotary
    n, max_pos, pages = 11, 300, 9
    theta = 500000.0
    rot = Rotary(dh, theta, max_pos, interleaved=(pairing == "adjacent"))
    cos, sin = rot.host_tables()
    sin_p, cos_p = plain.rope_tables(max_pos, dh, theta)
    # a frequency may differ in its last bit between two correct implementations of powf
    bound = max_pos * 2.0 ** -23
    assert np.abs(cos - cos_p.numpy()).max() < bound and np.abs(sin - sin_p.numpy()).max() < bound
    qkv = rnd(n, (nh + 2 * nkv) * dh, seed=dh).to(DT[dtype])
    pos = torch.tensor(random.Random(1).sample(range(max_pos), n), dtype=torch.int32)
    slots = torch.tensor(random.Random(2).sample(range(pages * page), n), dtype=torch.int32)
    slots[4] = -1                                              # nothing is stored for this token
    cache = torch.full((pages, 2, nkv * dh * page), 7.0, dtype=DT[dtype])
    cg, qg = cache.cuda(), qkv.cuda()
    ops.rope_kv_store(qg, pos.cuda(), nh, nkv, dh, torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda(), dh,
                      1 if pairing == "adjacent" else 0, cg, slots.cuda(), page)
    q = qkv[:, :nh * dh].view(n, nh, dh)
    k = qkv[:, nh * dh:(nh + nkv) * dh].view(n, nkv, dh)
    v = qkv[:, (nh + nkv) * dh:].view(n, nkv, dh)
    q_want = plain.rope(q, pos.tolist(), sin_p, cos_p, pairing)
    k_want = plain.rope(k, pos.tolist(), sin_p, cos_p, pairing)
    close(qg[:, :nh * dh].reshape(n, nh, dh), q_want, dtype, "q")
    assert torch.equal(qg[:, nh * dh:].cpu(), qkv[:, nh * dh:])           # k and v in the step's buffer stay
    flat = cg.cpu().view(pages, -1)
    expect = torch.full_like(flat, 7.0).double()
    for t in range(n):
        if slots[t] < 0:
            continue
        pg, tok = int(slots[t]) // page, int(slots[t]) % page
        for h in range(nkv):
            for c in range(dh):
                expect[pg, key_offset(h, tok, c, dh, page)] = k_want[t, h, c]
                expect[pg, value_offset(nkv, h, tok, c, dh, page)] = v[t, h, c].double()
    close(flat, expect, dtype, "cache")
    assert torch.equal(flat == 7.0, expect == 7.0)                        # nothing else was touched


@pytest.mark.parametrize("dtype,nh,nkv,dh,page", [("bfloat16", 4, 2, 128, 16), ("float32", 3, 1, 32, 32),
                                                   ("bfloat16", 2, 2, 16, 8)])
def test_rope_and_cache_write_many_tokens(dtype, nh, nkv, dh, page):
    """The kernel for many tokens takes eight tokens a block: runs of places in a page that
    start at a multiple of eight, runs that do not, places in no order, tokens that store
    nothing, and a last block that is not full."""
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.position import Rotary
    max_pos, pages, theta = 400, 40, 10000.0
    rot = Rotary(dh, theta, max_pos)
    cos, sin = rot.host_tables()
    sin_p, cos_p = plain.rope_tables(max_pos, dh, theta)
    rng = random.Random(5)
    free = list(range(pages))
    rng.shuffle(free)
    slots, pos = [], []

    def run(start_place, length, first_pos):
        """A request's portion: consecutive positions, places that go on through its pages."""
        place = start_place
        pg = free.pop()
        for i in range(length):
            if place == page:
                pg, place = free.pop(), 0
            slots.append(pg * page + place)
            pos.append(first_pos + i)
            place += 1

    run(0, 5 * page // 2 + 8, 0)            # starts a page: rows of eight all along (batch offset 0)
    run(3, 29, 100)                         # starts in the middle of a page: no row of eight fits
    n_run = len(slots)
    rest = [pg * page + k for pg in free[:3] for k in range(page)]
    rng.shuffle(rest)
    extra = 64 + 13
    slots += rest[:extra] if len(rest) >= extra else (rest + [-1] * (extra - len(rest)))
    pos += [rng.randrange(max_pos) for _ in range(len(slots) - n_run)]
    for i in (2, n_run + 5):
        slots[i] = -1
    n = len(slots)
    assert n >= 64 and n % 8 != 0
    qkv = rnd(n, (nh + 2 * nkv) * dh, seed=dh + 1).to(DT[dtype])
    cache = torch.full((pages, 2, nkv * dh * page), 7.0, dtype=DT[dtype])
    cg, qg = cache.cuda(), qkv.cuda()
    ops.rope_kv_store(qg, torch.tensor(pos, dtype=torch.int32).cuda(), nh, nkv, dh, torch.from_numpy(cos).cuda(),
                      torch.from_numpy(sin).cuda(), dh, 0, cg, torch.tensor(slots, dtype=torch.int32).cuda(), page)
    q = qkv[:, :nh * dh].view(n, nh, dh)
    k = qkv[:, nh * dh:(nh + nkv) * dh].view(n, nkv, dh)
    v = qkv[:, (nh + nkv) * dh:].view(n, nkv, dh)
    close(qg[:, :nh * dh].reshape(n, nh, dh), plain.rope(q, pos, sin_p, cos_p, "half"), dtype, "q")
    assert torch.equal(qg[:, nh * dh:].cpu(), qkv[:, nh * dh:])
    k_want = plain.rope(k, pos, sin_p, cos_p, "half")
    flat = cg.cpu().view(pages, -1)
    expect = torch.full_like(flat, 7.0).double()
    for t in range(n):
        if slots[t] < 0:
            continue
        pg, tok = slots[t] // page, slots[t] % page
        for h in range(nkv):
            for c in range(dh):
                expect[pg, key_offset(h, tok, c, dh, page)] = k_want[t, h, c]
                expect[pg, value_offset(nkv, h, tok, c, dh, page)] = v[t, h, c].double()
    close(flat, expect, dtype, "cache")
    assert torch.equal(flat == 7.0, expect == 7.0)


def test_rope_partial_rotation_and_no_rotation():
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.position import Rotary
    n, nh, dh, rot_dim = 4, 2, 32, 16
    rot = Rotary(dh, 10000.0, 64, rot_dim=rot_dim)
    cos, sin = rot.host_tables()
    q = rnd(n, nh * dh, seed=3)
    pos = torch.tensor([0, 5, 17, 63], dtype=torch.int32)
    qg = q.clone().cuda()
    ops.rope_kv_store(qg, pos.cuda(), nh, 0, dh, torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda(), rot_dim, 0,
                      None, None, 16)
    sin_p, cos_p = plain.rope_tables(64, rot_dim, 10000.0)
    qv = q.view(n, nh, dh)
    want = qv.clone().double()
    want[..., :rot_dim] = plain.rope(qv[..., :rot_dim], pos.tolist(), sin_p, cos_p, "half")
    close(qg.view(n, nh, dh), want, "float32")
    qg2 = q.clone().cuda()
    ops.rope_kv_store(qg2, pos.cuda(), nh, 0, dh, None, None, 0, 0, None, None, 16)
    assert torch.equal(qg2.cpu(), q)


# ------------------------------------------------------------------ attention
class Batch:
    """The facts of a step that the attention kernels need, made by hand."""

    def __init__(self, q_lens, ctx_lens, tables, max_pages):
        from llama_cu_amd.engine.batch import StepContext
        n = sum(q_lens)
        qs = [0]
        for x in q_lens:
            qs.append(qs[-1] + x)
        rot = [r for r, x in enumerate(q_lens) for _ in range(x)]
        bt = torch.zeros(len(q_lens), max_pages, dtype=torch.int32)
        for r, t in enumerate(tables):
            bt[r, :len(t)] = torch.tensor(t, dtype=torch.int32)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32).cuda()
        self.step = StepContext(n=n, n_req=len(q_lens), tokens=i32([0] * n), positions=i32([0] * n), req_of_token=i32(rot),
                                q_start=i32(qs), ctx_len=i32(ctx_lens), state_slot=i32([0] * len(q_lens)),
                                logit_rows=i32([]), n_logits=0, block_tables=[bt.cuda()], slot_maps=[i32([0] * n)],
                                q_lens=list(q_lens), ctx_lens=list(ctx_lens))


def paged_case(dtype, nh, nkv, dh, page, q_lens, ctx_lens, window, seed, standout=True, poison=True):
    """Random keys, values and queries for requests with the given lengths, laid into pages
    in a random order; returns what the kernels need and the plain answer."""
    rng = random.Random(seed)
    tdt = DT[dtype]
    need = [(c + page - 1) // page for c in ctx_lens]
    n_pages = sum(need) + 3
    order = list(range(n_pages))
    rng.shuffle(order)
    fill = float("nan") if poison else 0.0
    cache = torch.full((n_pages, 2 * nkv * dh * page), fill, dtype=torch.float32)
    tables, outs, qs = [], [], []
    for r, (ql, cl) in enumerate(zip(q_lens, ctx_lens)):
        k = rnd(cl, nkv, dh, seed=seed * 100 + r).to(tdt).float()
        v = rnd(cl, nkv, dh, seed=seed * 100 + r + 50).to(tdt).float()
        q = rnd(ql, nh, dh, seed=seed * 100 + r + 70).to(tdt).float()
        if standout and cl > 3:
            # one key far back that every head's last query points at: it must dominate
            j = 1 if window == 0 else max(cl - window, 0) + 0
            j = min(j, cl - 1)
            for h in range(nh):
                k[j, h // (nh // nkv)] = (q[-1, h] * 1.5).to(tdt).float() if h % (nh // nkv) == 0 else k[j, h // (nh // nkv)]
        table = [order.pop() for _ in range(need[r])]
        if window > 0:
            # pages that the window of the first query has passed are gone (they hold poison)
            first_needed = max(cl - ql - window + 1, 0) // page
        else:
            first_needed = 0
        for j in range(cl):
            pg, tok = table[j // page], j % page
            if j // page < first_needed:
                continue
            for h in range(nkv):
                for c8 in range(dh // 8):
                    base = key_offset(h, tok, c8 * 8, dh, page)
                    cache[pg, base:base + 8] = k[j, h, c8 * 8:c8 * 8 + 8]
                cache[pg, value_offset(nkv, h, tok, 0, dh, page):value_offset(nkv, h, tok, 0, dh, page) + dh * page:page] = v[j, h]
        for p in range(first_needed):
            table[p] = 0 if poison else table[p]
        tables.append(table)
        qs.append(q)
        outs.append(plain.attention(q, k, v, dh ** -0.5, first_pos=cl - ql, window=window or None))
    q_all = torch.cat(qs).reshape(sum(q_lens), nh * dh).to(tdt)
    want = torch.cat(outs).reshape(sum(q_lens), nh * dh)
    cache = cache.to(tdt).view(n_pages, 2, nkv * dh * page)
    max_pages = max(need) + 2
    return q_all, cache, Batch(q_lens, ctx_lens, tables, max_pages).step, want


SHAPES = [  # nh, nkv, dh, page
    (4, 4, 16, 16), (4, 1, 32, 32), (6, 2, 48, 8), (8, 2, 64, 16), (32, 8, 128, 16), (6, 2, 128, 48), (32, 2, 64, 32),
    (5, 5, 256, 16), (6, 3, 96, 16)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,dh,page", SHAPES)
@pytest.mark.parametrize("window", [0, 37])
def test_attention_mixed_batch(dtype, nh, nkv, dh, page, window):
    """Portions beside single tokens, from the cache: the kernel the dispatcher picks and
    the generic kernel both give the plain answer."""
    from llama_cu_amd.kernels import ops
    q_lens, ctx_lens = [1, 7, 33, 2, 1], [1, 40, 33, 131, 300]
    q, cache, step, want = paged_case(dtype, nh, nkv, dh, page, q_lens, ctx_lens, window, seed=nh + dh)
    for force in (False, True):
        out = torch.empty(q.shape[0], nh * dh, dtype=DT[dtype], device="cuda")
        ops.paged_attention(q.cuda(), out, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, window, force_generic=force)
        close(out, want, dtype, f"force_generic={force}")


@pytest.mark.parametrize("nh,nkv,dh,page", [(8, 2, 64, 16), (32, 8, 128, 16), (16, 16, 128, 32), (32, 1, 64, 16), (6, 2, 128, 48),
                                            (4, 1, 32, 32), (6, 3, 96, 16)])
@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("splits", [None, 1, 3, 16])
def test_attention_decode_kernel(nh, nkv, dh, page, window, splits):
    """Every request feeds one token: the matrix-core decode kernel, with its keys cut
    into parts or not, against the plain answer; a far key dominates."""
    from llama_cu_amd.kernels import ops
    ctx_lens = [1, 31, 32, 33, 500, 2049]
    q, cache, step, want = paged_case("bfloat16", nh, nkv, dh, page, [1] * len(ctx_lens), ctx_lens, window, seed=dh + page)
    step.attn_splits = splits
    assert ops.mfma_attention_supported(q, nh, nkv, dh, page)
    out = torch.empty(q.shape[0], nh * dh, dtype=torch.bfloat16, device="cuda")
    ops.paged_attention(q.cuda(), out, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, window)
    close(out, want, "bfloat16")
    # the order in which the workgroups take the requests (the batch builder names the longest first) changes no bit
    step.decode_order = torch.tensor([5, 4, 3, 2, 1, 0], dtype=torch.int32, device="cuda")
    ordered = torch.full_like(out, float("nan"))
    ops.paged_attention(q.cuda(), ordered, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, window)
    assert torch.equal(ordered, out)


@pytest.mark.parametrize("nh,nkv,dh,page", [(8, 2, 128, 16), (4, 1, 64, 32)])
def test_attention_decode_kernel_long_context_in_many_parts(nh, nkv, dh, page):
    """One request with thousands of keys: its keys are cut into 32 parts (the most), each
    walked by another workgroup, and merged; a key far back dominates."""
    from llama_cu_amd.kernels import ops
    ctx_lens = [9001, 700]
    q, cache, step, want = paged_case("bfloat16", nh, nkv, dh, page, [1, 1], ctx_lens, 0, seed=dh)
    assert ops.decode_splits(1, nh, nkv, 9001) == 32
    for splits in (None, 32):
        step.attn_splits = splits
        out = torch.empty(q.shape[0], nh * dh, dtype=torch.bfloat16, device="cuda")
        ops.paged_attention(q.cuda(), out, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, 0)
        close(out, want, "bfloat16")


@pytest.mark.parametrize("nh,nkv,dh,page", [(8, 2, 64, 16), (32, 8, 128, 16), (3, 1, 128, 32), (7, 7, 64, 16), (4, 1, 32, 32), (6, 3, 96, 16)])
def test_attention_prefill_kernel_long(nh, nkv, dh, page):
    """Whole prompts and portions with history on the matrix cores, long enough that a
    wave walks many steps and tasks end inside a request."""
    from llama_cu_amd.kernels import ops
    q_lens, ctx_lens = [300, 77, 5], [300, 500, 1030]
    q, cache, step, want = paged_case("bfloat16", nh, nkv, dh, page, q_lens, ctx_lens, 0, seed=page + nh)
    out = torch.empty(q.shape[0], nh * dh, dtype=torch.bfloat16, device="cuda")
    ops.paged_attention(q.cuda(), out, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, 0)
    close(out, want, "bfloat16")


@pytest.mark.parametrize("per_wg", [2, 3])
def test_attention_prefill_kernel_with_several_tasks_a_workgroup(per_wg):
    """A workgroup that takes several tasks one after the other (the ring in LDS and the registers are
    used again): portions and single tokens, with a window."""
    from llama_cu_amd.kernels import build, ops
    nh, nkv, dh, page, window = 8, 2, 64, 16, 70
    q_lens, ctx_lens = [100, 1, 37, 64], [100, 90, 300, 64]
    q, cache, step, want = paged_case("bfloat16", nh, nkv, dh, page, q_lens, ctx_lens, window, seed=per_wg)
    tpt = build.load("attention_mfma").lcu_attention_prefill_tokens_per_task(nh, nkv)
    task_req, task_tok0, n_tasks, got_per_wg = ops.prefill_tasks(q_lens, ctx_lens, tpt, "cuda", per_wg=per_wg)
    assert got_per_wg == per_wg and n_tasks == sum((n + tpt - 1) // tpt for n in q_lens)
    out = torch.empty(q.shape[0], nh * dh, dtype=torch.bfloat16, device="cuda")
    ops.attention_prefill(q.cuda(), out, cache.cuda(), step.block_tables[0], step.q_start, step.ctx_len, task_req, task_tok0,
                          n_tasks, per_wg, nh, nkv, dh, page, dh ** -0.5, window)
    close(out, want, "bfloat16")


@pytest.mark.parametrize("page", [16, 32])
def test_attention_in_a_cache_of_more_than_4_gib(page):
    """A layer's cache beyond 4 GiB: a page's place no longer fits a 32-bit offset from the cache's start,
    and the kernels must address it by its own 64-bit address.  The requests' pages lie spread over the
    whole cache, its last page among them."""
    from llama_cu_amd.kernels import ops
    nh, nkv, dh = 8, 4, 128
    q_lens, ctx_lens = [150, 1, 40], [150, 333, 600]
    q, cache, step, want = paged_case("bfloat16", nh, nkv, dh, page, q_lens, ctx_lens, 0, seed=page)
    page_bytes = 2 * nkv * dh * page * 2
    n_big = (4 << 30) // page_bytes + 1000
    big = torch.empty(n_big, 2, nkv * dh * page, dtype=torch.bfloat16, device="cuda")
    n_small = cache.shape[0]
    place = torch.linspace(0, n_big - 1, n_small).round().long()       # small page i lies in big page place[i]
    assert place[-1] == n_big - 1 and len(set(place.tolist())) == n_small
    big[place.cuda()] = cache.cuda()
    step.block_tables[0] = place.cuda()[step.block_tables[0].long()].int()
    assert int(step.block_tables[0].max()) * page_bytes >= 1 << 32
    out = torch.empty(q.shape[0], nh * dh, dtype=torch.bfloat16, device="cuda")
    ops.paged_attention(q.cuda(), out, big, step, 0, nh, nkv, dh, page, dh ** -0.5, 0)
    close(out, want, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [0, 20])
def test_attention_with_a_bias_that_grows_with_the_distance(dtype, window):
    """``head_slopes``: slope[h] * (key position - query position) inside the scores, for portions and
    single tokens from the cache.  The expectation is written out here (the plain implementation has no
    such bias); slopes so steep that leaving the bias out, or its sign, would be far off."""
    from llama_cu_amd.kernels import ops
    nh, nkv, dh, page = 6, 2, 32, 16
    q_lens, ctx_lens = [30, 1, 7], [30, 65, 50]
    q, cache, step, _ = paged_case(dtype, nh, nkv, dh, page, q_lens, ctx_lens, window, seed=9, standout=False, poison=False)
    slopes = torch.tensor([0.5, 0.25, 0.125, 0.3, 0.0, 1.0])
    # the keys and values back from the pages, then the formula
    want, row = [], 0
    cf = cache.float().view(cache.shape[0], -1)
    for r, (ql, cl) in enumerate(zip(q_lens, ctx_lens)):
        table = step.block_tables[0][r].tolist()
        k = torch.zeros(cl, nkv, dh, dtype=torch.float64); v = torch.zeros(cl, nkv, dh, dtype=torch.float64)
        lo_all = max(cl - ql - window + 1, 0) if window else 0
        for j in range(lo_all, cl):
            pg, tok = table[j // page], j % page
            for h in range(nkv):
                for c8 in range(dh // 8):
                    base = key_offset(h, tok, c8 * 8, dh, page)
                    k[j, h, c8 * 8:c8 * 8 + 8] = cf[pg, base:base + 8]
                vo = value_offset(nkv, h, tok, 0, dh, page)
                v[j, h] = cf[pg, vo:vo + dh * page:page]
        qq = q[row:row + ql].double().view(ql, nh, dh)
        for i in range(ql):
            p = cl - ql + i
            lo = max(p - window + 1, 0) if window else 0
            js = torch.arange(lo, p + 1)
            for h in range(nh):
                sc = (k[lo:p + 1, h // (nh // nkv)] @ qq[i, h]) * dh ** -0.5 + float(slopes[h]) * (js - p).double()
                want.append(torch.softmax(sc, dim=0) @ v[lo:p + 1, h // (nh // nkv)])
        row += ql
    want = torch.stack(want).view(sum(q_lens), nh * dh)
    out = torch.empty(q.shape[0], nh * dh, dtype=DT[dtype], device="cuda")
    ops.paged_attention(q.cuda(), out, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, window, head_slopes=slopes.cuda())
    close(out, want, dtype)
    flat = torch.empty_like(out)
    ops.paged_attention(q.cuda(), flat, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, window)
    assert float((flat.double().cpu() - want).abs().max()) > 20 * TOL[dtype] * float(want.abs().max()), "the bias must matter here"
    with pytest.raises(ops.KernelError):
        ops.paged_attention(q.cuda(), out, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5, window, head_slopes=slopes[:3].cuda())


def _pages_of(k, v, page):
    """Keys and values ``[tokens, kv_heads, dim]`` as whole pages in the cache's layout (kv_layout.h): keys
    [kv_head][dim / 8][token][8], values [kv_head][dim][token]; the last page is filled up with NaN."""
    n, nkv, dh = k.shape
    n_pages = (n + page - 1) // page
    pad = n_pages * page - n
    if pad:
        k = torch.cat([k, torch.full((pad, nkv, dh), float("nan"))])
        v = torch.cat([v, torch.full((pad, nkv, dh), float("nan"))])
    kp = k.view(n_pages, page, nkv, dh // 8, 8).permute(0, 2, 3, 1, 4).reshape(n_pages, -1)
    vp = v.view(n_pages, page, nkv, dh).permute(0, 2, 3, 1).reshape(n_pages, -1)
    return torch.stack([kp, vp], dim=1)                  # [pages, 2, kv_heads * dim * page]


@pytest.mark.parametrize("top_of_a_cache_just_below_4_gib", [False, True])
def test_attention_over_more_than_32k_keys(top_of_a_cache_just_below_4_gib):
    """A portion and a single token over 33,000 and 40,000 keys (the counters of tiles and turns, the
    offsets of pages); with the pages at the top of a cache of just under 4 GiB, where a page's offset
    from the cache's start still fits 32 bits and nearly fills them."""
    from llama_cu_amd.kernels import ops
    nh, nkv, dh, page = 16, 8, 128, 16
    q_lens, ctx_lens = [48, 1], [33000, 40000]
    page_bytes = 2 * nkv * dh * page * 2
    need = [(c + page - 1) // page for c in ctx_lens]
    n_pages = ((1 << 32) - 1) // page_bytes if top_of_a_cache_just_below_4_gib else sum(need) + 5
    assert n_pages * page_bytes < 1 << 32
    cache = torch.empty(n_pages, 2, nkv * dh * page, dtype=torch.bfloat16, device="cuda")
    rng = random.Random(5)
    ids = list(range(n_pages - sum(need), n_pages))       # the last pages of the cache, in a random order
    rng.shuffle(ids)
    tables, qs, wants = [], [], []
    for r, (ql, cl) in enumerate(zip(q_lens, ctx_lens)):
        k = rnd(cl, nkv, dh, seed=70 + r).to(torch.bfloat16).float()
        v = rnd(cl, nkv, dh, seed=80 + r).to(torch.bfloat16).float()
        q = rnd(ql, nh, dh, seed=90 + r).to(torch.bfloat16).float()
        k[7, :] = (q[-1, ::nh // nkv] * 1.5).to(torch.bfloat16).float()       # a key far back that the last query points at
        table = [ids.pop() for _ in range(need[r])]
        cache[torch.tensor(table, device="cuda")] = _pages_of(k, v, page).to(torch.bfloat16).cuda()
        tables.append(table)
        qs.append(q)
        wants.append(plain.attention(q, k, v, dh ** -0.5, first_pos=cl - ql, window=None))
    step = Batch(q_lens, ctx_lens, tables, max(need) + 1).step
    q_all = torch.cat(qs).reshape(sum(q_lens), nh * dh).to(torch.bfloat16)
    out = torch.empty(sum(q_lens), nh * dh, dtype=torch.bfloat16, device="cuda")
    ops.paged_attention(q_all.cuda(), out, cache, step, 0, nh, nkv, dh, page, dh ** -0.5, 0)
    close(out, torch.cat(wants).reshape(sum(q_lens), nh * dh), "bfloat16")


def test_attention_float32_result_does_not_depend_on_the_batch():
    from llama_cu_amd.kernels import ops
    nh, nkv, dh, page = 4, 2, 32, 16
    q, cache, step, want = paged_case("float32", nh, nkv, dh, page, [9, 1], [100, 64], 0, seed=3)
    out = torch.empty(q.shape[0], nh * dh, device="cuda")
    ops.paged_attention(q.cuda(), out, cache.cuda(), step, 0, nh, nkv, dh, page, dh ** -0.5)
    # the same last token of request 0, alone in a batch of one token
    q1, cache1, step1, _ = paged_case("float32", nh, nkv, dh, page, [9, 1], [100, 64], 0, seed=3)
    step1 = Batch([1], [100], [step.block_tables[0][0].tolist()], step.block_tables[0].shape[1]).step
    out1 = torch.empty(1, nh * dh, device="cuda")
    ops.paged_attention(q[8:9].cuda(), out1, cache.cuda(), step1, 0, nh, nkv, dh, page, dh ** -0.5)
    assert torch.equal(out[8:9], out1)


# ------------------------------------------------------------------ weight-streaming product for few rows
@pytest.mark.parametrize("m", [1, 8, 16, 17, 25, 32])
@pytest.mark.parametrize("n,k", [(16, 8), (100, 64), (301, 136), (1000, 4096), (4096, 1000)])
@pytest.mark.parametrize("tiles", [1, 2, 4])
def test_gemm_skinny(m, n, k, tiles):
    from llama_cu_amd.kernels import ops
    x = rnd(m, k, seed=m + k).to(torch.bfloat16)
    w = rnd(n, k, seed=n).to(torch.bfloat16)
    want = plain.linear(x, w)
    close(ops.gemm_skinny(x.cuda(), w.cuda(), tiles=tiles), want, "bfloat16", "bf16 out")
    close(ops.gemm_skinny(x.cuda(), w.cuda(), out_dtype=torch.float32, tiles=tiles), want, "float32", "f32 out")
    c = rnd(m, n, seed=5)
    cg = c.cuda()
    ops.gemm_skinny(x.cuda(), w.cuda(), out=cg, accumulate=True, tiles=tiles)
    close(cg, c.double() + want, "float32", "accumulate")


@pytest.mark.parametrize("m,di,k", [(1, 8, 16), (8, 172, 64), (23, 1000, 128), (32, 14336, 256)])
def test_gemm_skinny_swiglu(m, di, k):
    from llama_cu_amd.kernels import ops
    x = rnd(m, k, seed=m).to(torch.bfloat16)
    w = rnd(2 * di, k, seed=di, scale=0.3).to(torch.bfloat16)
    gu = plain.linear(x, w)
    close(ops.gemm_skinny(x.cuda(), w.cuda(), swiglu=True), plain.swiglu(gu[:, :di], gu[:, di:]), "bfloat16")


def test_gemm_skinny_result_does_not_depend_on_the_batch():
    from llama_cu_amd.kernels import ops
    x = rnd(30, 512, seed=1).to(torch.bfloat16).cuda()
    w = rnd(300, 512, seed=2).to(torch.bfloat16).cuda()
    whole = ops.gemm_skinny(x, w, out_dtype=torch.float32)
    one = ops.gemm_skinny(x[23:24], w, out_dtype=torch.float32)
    assert torch.equal(whole[23:24], one)


def test_gemm_skinny_refuses_what_it_cannot_take():
    from llama_cu_amd.kernels import ops
    x = rnd(4, 172).to(torch.bfloat16).cuda()        # K no multiple of 8
    w = rnd(16, 172).to(torch.bfloat16).cuda()
    assert not ops.skinny_supported(x, w, torch.bfloat16)
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(x, w)
    assert not ops.skinny_supported(rnd(33, 64).to(torch.bfloat16).cuda(), rnd(16, 64).to(torch.bfloat16).cuda(), torch.bfloat16)


# ------------------------------------------------------------------ product that shares the rows through LDS (to 256 rows)
@pytest.mark.parametrize("m", [5, 33, 47, 48, 64, 65, 96, 97, 128, 129, 177, 192, 193, 256])
@pytest.mark.parametrize("n,k", [(16, 128), (208, 384), (1008, 1024), (64, 2176)])
@pytest.mark.parametrize("packed", [False, True])
def test_gemm_mid(m, n, k, packed):
    from llama_cu_amd.kernels import ops
    x = rnd(m, k, seed=m + k).to(torch.bfloat16)
    w = rnd(n, k, seed=n).to(torch.bfloat16)
    want = plain.linear(x, w)
    wg = ops.pack_weight(w.cuda()) if packed else w.cuda()
    # the rows of x lie in a larger buffer whose other rows are poison: nothing beyond row m may count
    buf = torch.full((m + 3, k + 8), float("nan"), dtype=torch.bfloat16, device="cuda")
    buf[:m, :k] = x.cuda()
    xg = buf[:m, :k]
    close(ops.gemm_mid(xg, wg, packed=packed), want, "bfloat16", "bf16 out")
    for slices in (1, 2, 3, 5, 64):
        planes = ops.gemm_mid(xg, wg, slices=slices, packed=packed)
        assert planes.shape == (ops.mid_planes(k, slices), m, n) and planes.dtype == torch.float32
        assert planes.shape[0] <= min(slices, k // 128)
        close(planes.double().sum(0), want, "float32", f"{slices} slices")
    # a slice's plane is that slice's sum alone
    if k >= 256:
        planes = ops.gemm_mid(xg, wg, slices=2, packed=packed)
        half = 128 * (-(-(k // 128) // 2))
        close(planes[0], plain.linear(x[:, :half], w[:, :half]), "float32", "first slice")


@pytest.mark.parametrize("m,di,k", [(15, 48, 128), (17, 176, 256), (32, 1008, 384), (33, 16, 128), (40, 176, 256), (64, 1008, 640), (90, 176, 384), (128, 1008, 256),
                                    (130, 176, 640), (192, 1008, 384), (255, 48, 1152), (256, 176, 128)])
@pytest.mark.parametrize("packed", [False, True])
def test_gemm_mid_swiglu(m, di, k, packed):
    from llama_cu_amd.kernels import ops
    x = rnd(m, k, seed=m).to(torch.bfloat16)
    w = rnd(2 * di, k, seed=di, scale=0.3).to(torch.bfloat16)
    gu = plain.linear(x, w)
    wg = ops.pack_weight(w.cuda()) if packed else w.cuda()
    close(ops.gemm_mid(x.cuda(), wg, swiglu=True, packed=packed), plain.swiglu(gu[:, :di], gu[:, di:]), "bfloat16")


@pytest.mark.parametrize("m,di,k,parts", [(17, 16, 128, 1), (32, 176, 256, 256), (40, 1008, 640, 48), (64, 64, 128, 100)])
def test_gemm_mid_rows_that_wait_for_their_normalisation(m, di, k, parts):
    """The rows' factor, rsqrt(sum of the row's shares / width + eps), goes into the epilogue: of
    SwiGLU, of the plain product and of every plane of partial sums."""
    from llama_cu_amd.kernels import ops
    x = rnd(m, k, seed=m).to(torch.bfloat16)
    w = rnd(2 * di, k, seed=di, scale=0.3).to(torch.bfloat16)
    # shares in a buffer with poison behind them: only a row's own shares may count
    shares = torch.full((m + 1, parts), float("nan"))
    shares[:m] = rnd(m, parts, seed=3).abs() * k / parts
    sg = shares.cuda()[:m]
    eps, width = 1e-3, k
    factor = torch.rsqrt(shares[:m].double().sum(1, keepdim=True) / width + eps)
    gu = plain.linear(x, w) * factor
    for packed in (False, True):
        wg = ops.pack_weight(w.cuda()) if packed else w.cuda()
        kw = dict(packed=packed, row_sumsq=sg, norm_width=width, eps=eps)
        close(ops.gemm_mid(x.cuda(), wg, swiglu=True, **kw), plain.swiglu(gu[:, :di], gu[:, di:]), "bfloat16", "SwiGLU")
        close(ops.gemm_mid(x.cuda(), wg, **kw), gu, "bfloat16", "plain product")
        close(ops.gemm_mid(x.cuda(), wg, slices=2, **kw).double().sum(0), gu, "float32", "planes")


def test_gemm_mid_result_does_not_depend_on_the_batch_and_equals_the_sum_of_the_products():
    from llama_cu_amd.kernels import ops
    x = rnd(250, 512, seed=1).to(torch.bfloat16).cuda()
    w = rnd(304, 512, seed=2).to(torch.bfloat16).cuda()
    for rows in (110, 250):
        whole = ops.gemm_mid(x[:rows], w, slices=2)
        one = ops.gemm_mid(x[23:24], w, slices=2)
        assert torch.equal(whole[:, 23:24], one)
        assert torch.equal(whole[:, 70:110], ops.gemm_mid(x[70:110], w, slices=2))
        again = ops.gemm_mid(x[:rows], w, slices=2)
        assert torch.equal(whole, again)


def test_gemm_mid_refuses_what_it_cannot_take():
    from llama_cu_amd.kernels import ops
    w = rnd(16, 128).to(torch.bfloat16).cuda()
    assert not ops.mid_supported(rnd(257, 128).to(torch.bfloat16).cuda(), w)                # too many rows
    assert not ops.mid_supported(rnd(40, 136).to(torch.bfloat16).cuda(), rnd(16, 136).to(torch.bfloat16).cuda())   # K no multiple of 128
    assert not ops.mid_supported(rnd(40, 128).to(torch.bfloat16).cuda(), rnd(24, 128).to(torch.bfloat16).cuda())   # features no multiple of 16
    assert not ops.mid_supported(rnd(40, 128).cuda(), w)                                      # float32 rows
    with pytest.raises(ops.KernelError):
        ops.gemm_mid(rnd(257, 128).to(torch.bfloat16).cuda(), w)
    with pytest.raises(ops.KernelError):                                                      # rows that wait for their factor: at most 64
        ops.gemm_mid(rnd(65, 128).to(torch.bfloat16).cuda(), w, row_sumsq=torch.ones(65, 4, device="cuda"), norm_width=128, eps=1e-5)
    with pytest.raises(ops.KernelError):
        ops.gemm_mid(rnd(40, 128).to(torch.bfloat16).cuda(), w, swiglu=True)                  # 16 rows are no gate and up tiles
    with pytest.raises(ops.KernelError):
        ops.gemm_mid(rnd(40, 128).to(torch.bfloat16).cuda(), w, slices=65)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [172, 4096, 8192])
def test_rmsnorm_of_a_row_does_not_depend_on_the_number_of_rows(dtype, d):
    """Many rows go to smaller blocks than few rows; the sum is added in the same order."""
    from llama_cu_amd.kernels import ops
    x = rnd(300, d, seed=4)
    delta = rnd(300, d, seed=5).to(DT[dtype])
    w = (1 + rnd(d, seed=6, scale=0.1)).to(DT[dtype]).cuda()
    xa, xb = x.cuda(), x[7:9].cuda()
    many = ops.rmsnorm(xa, w, 1e-5, torch.empty(300, d, dtype=DT[dtype], device="cuda"), delta=delta.cuda())
    few = ops.rmsnorm(xb, w, 1e-5, torch.empty(2, d, dtype=DT[dtype], device="cuda"), delta=delta[7:9].cuda())
    assert torch.equal(many[7:9], few) and torch.equal(xa[7:9], xb)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,d,planes", [(1, 16, 1), (5, 172, 3), (40, 4096, 4), (2, 8200, 2)])
def test_rmsnorm_adds_planes_of_partial_sums(dtype, n, d, planes):
    from llama_cu_amd.kernels import ops
    x = rnd(n, d, seed=1, scale=0.05)
    parts = rnd(planes, n, d, seed=2, scale=0.05)
    w = (1 + rnd(d, seed=3, scale=0.1)).to(DT[dtype])
    xg = x.cuda()
    out = torch.empty(n, d, dtype=DT[dtype], device="cuda")
    ops.rmsnorm(xg, w.cuda(), 1e-5, out, delta=parts.cuda())
    xs = x.double() + parts.double().sum(0)
    close(xg, xs, "float32", "residual sum")
    close(out, plain.rms_norm(xs, w, 1e-5), dtype, "norm")
    # the planes are added one after the other: the same bits as adding them one by one
    xg2 = x.cuda()
    for p in range(planes):
        ops.residual_add(xg2, parts[p].cuda())
    assert torch.equal(xg, xg2)


@pytest.mark.parametrize("m,n,k,tiles,wdtype", [(1, 16, 8, 1, "bfloat16"), (8, 304, 136, 1, "float32"), (16, 4096, 1000, 1, "bfloat16"),
                                                (5, 104, 64, 2, "bfloat16"), (13, 1000, 4096, 2, "float32"),
                                                (17, 304, 256, 1, "bfloat16"), (32, 1000, 512, 2, "float32"), (27, 96, 136, 2, "bfloat16")])
def test_gemm_skinny_residual_sum_and_norm_weight_in_the_epilogue(m, n, k, tiles, wdtype):
    """``residual += x w^T``; the new rows times the norm's weight as bfloat16, not yet normalised;
    the workgroups' shares of the rows' sums of squares.  Then a second product applies the
    norm's factor per row in its epilogue, plain and with SwiGLU: together they equal residual
    sum, RMS norm and product done one after the other."""
    from llama_cu_amd.kernels import ops
    eps = 1e-5
    x = rnd(m, k, seed=m + k).to(torch.bfloat16)
    w = rnd(n, k, seed=n, scale=0.3).to(torch.bfloat16)
    res = rnd(m, n, seed=3) * 3.0
    nw = (1.0 + 0.2 * rnd(n, seed=4)).to(DT[wdtype])
    res_g = res.clone().cuda()
    h, sumsq = ops.gemm_skinny_add_norm(x.cuda(), w.cuda(), res_g, nw.cuda(), tiles=tiles)
    new = res.double() + plain.linear(x, w)
    close(res_g, new, "float32", "residual")
    assert sumsq.shape == (m, (n + 16 * tiles - 1) // (16 * tiles))
    close(sumsq.sum(dim=1), (new ** 2).sum(dim=1), "float32", "sums of squares")
    close(h, new * nw.double()[None, :], "bfloat16", "rows with the norm's weight")
    # the product that follows: n features in, n2 out
    n2 = 72
    w2 = rnd(2 * n2, n, seed=5, scale=0.2).to(torch.bfloat16)
    normed = plain.rms_norm(new, nw, eps)
    got = ops.gemm_skinny(h, w2.cuda(), row_sumsq=sumsq, norm_width=n, eps=eps)
    close(got, plain.linear(normed, w2), "bfloat16", "scaled product")
    got = ops.gemm_skinny(h, w2.cuda(), swiglu=True, row_sumsq=sumsq, norm_width=n, eps=eps)
    gu = plain.linear(normed, w2)
    close(got, plain.swiglu(gu[:, :n2], gu[:, n2:]), "bfloat16", "scaled product with SwiGLU")
    # the same shares on every call: no atomics
    res_g2 = res.clone().cuda()
    h2, sumsq2 = ops.gemm_skinny_add_norm(x.cuda(), w.cuda(), res_g2, nw.cuda(), tiles=tiles)
    assert torch.equal(sumsq, sumsq2) and torch.equal(h, h2) and torch.equal(res_g, res_g2)


@pytest.mark.parametrize("m,n,k,packed,wdtype", [(1, 16, 128, False, "bfloat16"), (16, 304, 256, True, "float32"),
                                                 (17, 4096, 1024, True, "bfloat16"), (33, 96, 384, False, "float32"),
                                                 (48, 1008, 2176, True, "bfloat16"), (49, 64, 128, True, "float32"),
                                                 (64, 608, 640, True, "bfloat16")])
def test_gemm_mid_residual_sum_and_norm_weight_in_the_epilogue(m, n, k, packed, wdtype):
    """The same for up to 64 rows, by the kernel that shares the rows through LDS (a workgroup takes 16 output features
    over all of K, its waves share each 128 k): ``residual += x w^T``, the new rows times the norm's weight, the
    workgroups' shares of the sums of squares; the product that follows applies the factor.  The residual's and h's other
    rows and the rows of x beyond the last are poison."""
    from llama_cu_amd.kernels import ops
    eps = 1e-5
    x = rnd(m, k, seed=m + k).to(torch.bfloat16)
    w = rnd(n, k, seed=n, scale=0.3).to(torch.bfloat16)
    res = rnd(m, n, seed=3) * 3.0
    nw = (1.0 + 0.2 * rnd(n, seed=4)).to(DT[wdtype])
    buf = torch.full((m + 3, k + 8), float("nan"), dtype=torch.bfloat16, device="cuda")
    buf[:m, :k] = x.cuda()
    res_buf = torch.full((m + 2, n + 4), float("nan"), device="cuda")
    res_buf[:m, :n] = res.cuda()
    res_g = res_buf[:m, :n]
    wg = ops.pack_weight(w.cuda()) if packed else w.cuda()
    h, sumsq = ops.gemm_mid_add_norm(buf[:m, :k], wg, res_g, nw.cuda(), packed=packed)
    new = res.double() + plain.linear(x, w)
    close(res_g, new, "float32", "residual")
    assert bool(torch.isnan(res_buf[m:]).all()) and bool(torch.isnan(res_buf[:, n:]).all())
    assert sumsq.shape == (m, n // 16)
    close(sumsq.sum(dim=1), (new ** 2).sum(dim=1), "float32", "sums of squares")
    close(h, new * nw.double()[None, :], "bfloat16", "rows with the norm's weight")
    n2 = 80
    w2 = rnd(2 * n2, n, seed=5, scale=0.2).to(torch.bfloat16)
    normed = plain.rms_norm(new, nw, eps)
    gu = plain.linear(normed, w2)
    if n % 128 == 0:                                  # the product that follows, in the same kernel family
        got = ops.gemm_mid(h, w2.cuda(), swiglu=True, row_sumsq=sumsq, norm_width=n, eps=eps)
        close(got, plain.swiglu(gu[:, :n2], gu[:, n2:]), "bfloat16", "scaled product with SwiGLU")
    if m <= 32 and n % 8 == 0:
        close(ops.gemm_skinny(h, w2.cuda(), row_sumsq=sumsq, norm_width=n, eps=eps), gu, "bfloat16", "scaled product")
    res_buf2 = torch.full((m + 2, n + 4), float("nan"), device="cuda")
    res_buf2[:m, :n] = res.cuda()
    h2, sumsq2 = ops.gemm_mid_add_norm(buf[:m, :k], wg, res_buf2[:m, :n], nw.cuda(), packed=packed)
    assert torch.equal(sumsq, sumsq2) and torch.equal(h, h2) and torch.equal(res_g, res_buf2[:m, :n])   # no atomics
    with pytest.raises(ops.KernelError):
        ops.gemm_mid_add_norm(rnd(65, k).to(torch.bfloat16).cuda(), wg, torch.zeros(65, n).cuda(), nw.cuda(), packed=packed)


@pytest.mark.parametrize("m,n,k", [(1, 16, 128), (8, 304, 256), (16, 4096, 1024), (13, 96, 384), (30, 608, 256)])
def test_gemm_skinny_with_a_packed_weight_equals_the_plain_one_bit_for_bit(m, n, k):
    """``pack_weight`` only changes where the kernel finds its operands, not what it adds in
    which order: every epilogue gives the same bits as with the plain weight.  The packed
    copy is checked against its definition too."""
    from llama_cu_amd.kernels import ops
    x = rnd(m, k, seed=m).to(torch.bfloat16).cuda()
    w = rnd(n, k, seed=n, scale=0.3).to(torch.bfloat16)
    p = ops.pack_weight(w.cuda())
    assert p.shape == w.shape
    # [tile of 16 rows][block of 128 k][load j][lane = 16 * group + row][8 k], k = 32 * group + 8 * j + e
    flat = p.cpu().view(n // 16, k // 128, 4, 4, 16, 8)
    for (t, b, j, g, r, e) in [(0, 0, 0, 0, 0, 0), (n // 16 - 1, k // 128 - 1, 3, 2, 15, 7), (0, k // 128 - 1, 1, 3, 4, 2)]:
        assert flat[t, b, j, g, r, e] == w[16 * t + r, 128 * b + 32 * g + 8 * j + e]
    wg = w.cuda()
    for tiles in (1, 2, 4):
        assert torch.equal(ops.gemm_skinny(x, wg, tiles=tiles), ops.gemm_skinny(x, p, tiles=tiles, packed=True))
    assert torch.equal(ops.gemm_skinny(x, wg, out_dtype=torch.float32), ops.gemm_skinny(x, p, out_dtype=torch.float32, packed=True))
    if n % 32 == 0:
        assert torch.equal(ops.gemm_skinny(x, wg, swiglu=True), ops.gemm_skinny(x, p, swiglu=True, packed=True))
    res = rnd(m, n, seed=3).cuda()
    nw = (1.0 + 0.2 * rnd(n, seed=4)).to(torch.bfloat16).cuda()
    r1, r2 = res.clone(), res.clone()
    h1, s1 = ops.gemm_skinny_add_norm(x, wg, r1, nw)
    h2, s2 = ops.gemm_skinny_add_norm(x, p, r2, nw, packed=True)
    assert torch.equal(r1, r2) and torch.equal(h1, h2) and torch.equal(s1, s2)
    close(ops.gemm_skinny(x, p, packed=True), plain.linear(x.cpu(), w), "bfloat16")
    with pytest.raises(ops.KernelError):
        ops.pack_weight(rnd(24, 128).to(torch.bfloat16).cuda())            # no whole tiles of 16 rows
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(x, wg[:, :k - 8], packed=True)


@pytest.mark.parametrize("m,k,nh,nkv,dh,page,packed,scaled", [(1, 64, 4, 2, 32, 8, False, False), (8, 256, 6, 2, 64, 16, True, True),
                                                              (16, 136, 3, 1, 96, 24, False, True), (5, 512, 8, 8, 128, 32, True, False),
                                                              (13, 128, 5, 5, 160, 16, True, False), (17, 256, 4, 2, 64, 16, True, True),
                                                              (32, 136, 3, 3, 32, 8, False, False), (29, 128, 8, 2, 128, 16, True, True)])
def test_gemm_skinny_q_k_v_with_rotation_and_cache_write(m, k, nh, nkv, dh, page, packed, scaled):
    """The product of few rows with the q, k and v weights whose epilogue rotates q and k and
    writes k and v into the pages: against product, rotation and cache layout done one after
    the other; a token that stores nothing; nothing else in the cache is touched."""
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.position import Rotary
    max_pos, pages, theta, eps = 300, 7, 10000.0, 1e-5
    n = (nh + 2 * nkv) * dh
    cos, sin = Rotary(dh, theta, max_pos).host_tables()
    sin_p, cos_p = plain.rope_tables(max_pos, dh, theta)
    x = rnd(m, k, seed=m + k).to(torch.bfloat16)
    w = rnd(n, k, seed=n, scale=0.3).to(torch.bfloat16)
    pos = random.Random(1).sample(range(max_pos), m)
    slots = random.Random(2).sample(range(pages * page), m)
    if m > 2:
        slots[2] = -1
    cache = torch.full((pages, 2, nkv * dh * page), 7.0, dtype=torch.bfloat16).cuda()
    kw, rows = {}, x.double()
    if scaled:
        sumsq = rnd(m, 5, seed=9).abs() * 40.0
        kw = dict(row_sumsq=sumsq.cuda(), norm_width=k, eps=eps)
        rows = rows * torch.rsqrt(sumsq.double().sum(dim=1) / k + eps)[:, None]
    wg = ops.pack_weight(w.cuda()) if packed else w.cuda()
    q_got = ops.gemm_skinny_qkv_rope(x.cuda(), wg, torch.tensor(pos, dtype=torch.int32).cuda(),
                                     torch.tensor(slots, dtype=torch.int32).cuda(), torch.from_numpy(cos).cuda(),
                                     torch.from_numpy(sin).cuda(), cache, nh, nkv, dh, page, packed=packed, **kw)
    qkv = plain.linear(rows, w)
    q = qkv[:, :nh * dh].view(m, nh, dh)
    kk = qkv[:, nh * dh:(nh + nkv) * dh].view(m, nkv, dh)
    v = qkv[:, (nh + nkv) * dh:].view(m, nkv, dh)
    close(q_got.reshape(m, nh, dh), plain.rope(q, pos, sin_p, cos_p, "half"), "bfloat16", "q")
    k_want = plain.rope(kk, pos, sin_p, cos_p, "half")
    flat = cache.cpu().view(pages, -1)
    expect = torch.full_like(flat, 7.0).double()
    written = torch.zeros_like(flat, dtype=torch.bool)
    for t in range(m):
        if slots[t] < 0:
            continue
        pg, tok = slots[t] // page, slots[t] % page
        for h in range(nkv):
            for c in range(dh):
                expect[pg, key_offset(h, tok, c, dh, page)] = k_want[t, h, c]
                expect[pg, value_offset(nkv, h, tok, c, dh, page)] = v[t, h, c]
                written[pg, key_offset(h, tok, c, dh, page)] = written[pg, value_offset(nkv, h, tok, c, dh, page)] = True
    close(flat, expect, "bfloat16", "cache")
    assert bool((flat[~written] == 7.0).all())                              # nothing else was touched
    with pytest.raises(ops.KernelError):                                    # halves of a head that are no multiple of 16
        ops.gemm_skinny_qkv_rope(x.cuda(), rnd(4 * 48, k).to(torch.bfloat16).cuda(), torch.zeros(m, dtype=torch.int32).cuda(),
                                 torch.zeros(m, dtype=torch.int32).cuda(), torch.zeros(max_pos, 24).cuda(),
                                 torch.zeros(max_pos, 24).cuda(), torch.zeros(2, 2, 48 * page, dtype=torch.bfloat16).cuda(),
                                 2, 1, 48, page)


@pytest.mark.parametrize("m,k,nh,nkv,dh,page,packed", [(5, 128, 4, 2, 32, 8, False), (33, 256, 6, 2, 64, 16, True),
                                                       (48, 384, 3, 1, 96, 24, False), (64, 512, 8, 8, 128, 32, True),
                                                       (65, 128, 5, 5, 160, 16, True), (100, 1152, 4, 2, 64, 16, True),
                                                       (128, 256, 3, 3, 32, 8, False), (129, 640, 8, 2, 128, 16, True),
                                                       (192, 128, 2, 1, 64, 48, True), (193, 256, 2, 2, 32, 16, False),
                                                       (256, 2176, 4, 1, 128, 64, True)])
def test_gemm_mid_q_k_v_with_rotation_and_cache_write(m, k, nh, nkv, dh, page, packed):
    """The same for up to 256 rows, by the kernel that shares the rows through LDS (its consumer waves share each
    128 k and add their sums at the end): against product, rotation and cache layout done one after the other; a
    token that stores nothing; nothing else in the cache is touched; rows beyond the last are poison."""
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.position import Rotary
    max_pos, theta = 700, 10000.0
    pages = m // page + 4
    n = (nh + 2 * nkv) * dh
    cos, sin = Rotary(dh, theta, max_pos).host_tables()
    sin_p, cos_p = plain.rope_tables(max_pos, dh, theta)
    x = rnd(m, k, seed=m + k).to(torch.bfloat16)
    w = rnd(n, k, seed=n, scale=0.3).to(torch.bfloat16)
    pos = random.Random(1).sample(range(max_pos), m)
    slots = random.Random(2).sample(range(pages * page), m)
    if m > 2:
        slots[2] = -1
    cache = torch.full((pages, 2, nkv * dh * page), 7.0, dtype=torch.bfloat16).cuda()
    buf = torch.full((m + 3, k + 8), float("nan"), dtype=torch.bfloat16, device="cuda")
    buf[:m, :k] = x.cuda()
    wg = ops.pack_weight(w.cuda()) if packed else w.cuda()
    q_got = ops.gemm_mid_qkv_rope(buf[:m, :k], wg, torch.tensor(pos, dtype=torch.int32).cuda(),
                                  torch.tensor(slots, dtype=torch.int32).cuda(), torch.from_numpy(cos).cuda(),
                                  torch.from_numpy(sin).cuda(), cache, nh, nkv, dh, page, packed=packed)
    qkv = plain.linear(x.double(), w)
    q = qkv[:, :nh * dh].view(m, nh, dh)
    kk = qkv[:, nh * dh:(nh + nkv) * dh].view(m, nkv, dh)
    v = qkv[:, (nh + nkv) * dh:].view(m, nkv, dh)
    close(q_got.reshape(m, nh, dh), plain.rope(q, pos, sin_p, cos_p, "half"), "bfloat16", "q")
    k_want = plain.rope(kk, pos, sin_p, cos_p, "half")
    flat = cache.cpu().view(pages, -1)
    expect = torch.full_like(flat, 7.0).double()
    written = torch.zeros_like(flat, dtype=torch.bool)
    dims = torch.arange(dh)
    for t in range(m):
        if slots[t] < 0:
            continue
        pg, tok = slots[t] // page, slots[t] % page
        for h in range(nkv):
            ko = torch.tensor([key_offset(h, tok, int(c), dh, page) for c in dims])
            vo = torch.tensor([value_offset(nkv, h, tok, int(c), dh, page) for c in dims])
            expect[pg, ko] = k_want[t, h]
            expect[pg, vo] = v[t, h]
            written[pg, ko] = True
            written[pg, vo] = True
    close(flat, expect, "bfloat16", "cache")
    assert bool((flat[~written] == 7.0).all())                              # nothing else was touched
    # the same bits as the product in bfloat16 followed by the rotation kernel, when the sums agree: the product that
    # shares the rows adds a row's k in another order than this kernel's four waves, so only nearly
    cache_b = torch.full_like(cache, 7.0)
    rows = ops.gemm_mid(buf[:m, :k], wg, packed=packed)
    ops.rope_kv_store(rows, torch.tensor(pos, dtype=torch.int32).cuda(), nh, nkv, dh, torch.from_numpy(cos).cuda(),
                      torch.from_numpy(sin).cuda(), dh, 0, cache_b, torch.tensor(slots, dtype=torch.int32).cuda(), page)
    assert float((q_got.float() - rows[:, :nh * dh].float()).abs().max()) <= 0.02 * float(rows.float().abs().max())
    assert float((cache.float() - cache_b.float()).abs().max()) <= 0.02 * float(cache_b.float().abs().max())


def test_gemm_mid_q_k_v_refuses_what_it_cannot_take():
    from llama_cu_amd.kernels import ops
    page, max_pos = 16, 64
    z = lambda *s: torch.zeros(*s, dtype=torch.int32).cuda()
    tables = lambda dh: (torch.zeros(max_pos, dh // 2).cuda(), torch.zeros(max_pos, dh // 2).cuda())
    cache = lambda nkv, dh: torch.zeros(2, 2, nkv * dh * page, dtype=torch.bfloat16).cuda()
    x = rnd(40, 128).to(torch.bfloat16).cuda()
    with pytest.raises(ops.KernelError):                                    # halves of a head that are no multiple of 16
        ops.gemm_mid_qkv_rope(x, rnd(4 * 48, 128).to(torch.bfloat16).cuda(), z(40), z(40), *tables(48), cache(1, 48), 2, 1, 48, page)
    with pytest.raises(ops.KernelError):                                    # more than 256 rows
        ops.gemm_mid_qkv_rope(rnd(257, 128).to(torch.bfloat16).cuda(), rnd(4 * 64, 128).to(torch.bfloat16).cuda(), z(257), z(257),
                              *tables(64), cache(1, 64), 2, 1, 64, page)
    with pytest.raises(ops.KernelError):                                    # K no multiple of 128
        ops.gemm_mid_qkv_rope(rnd(40, 136).to(torch.bfloat16).cuda(), rnd(4 * 64, 136).to(torch.bfloat16).cuda(), z(40), z(40),
                              *tables(64), cache(1, 64), 2, 1, 64, page)
    with pytest.raises(ops.KernelError):                                    # a weight that is not q, k and v heads
        ops.gemm_mid_qkv_rope(x, rnd(3 * 64, 128).to(torch.bfloat16).cuda(), z(40), z(40), *tables(64), cache(1, 64), 2, 1, 64, page)


@pytest.mark.parametrize("m", [1, 17, 32])
@pytest.mark.parametrize("packed,scaled", [(False, False), (True, True)])
def test_q_k_v_epilogue_leaves_the_same_bits_as_product_then_rotation_kernel(m, packed, scaled):
    """A token's query and its key and value in the cache are the same bits whether the product's
    epilogue rotates and stores them or the product stores bfloat16 rows and the rotation kernel
    follows: both round the product to bfloat16 first and rotate with one formula."""
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.position import Rotary
    k, nh, nkv, dh, page, max_pos, pages = 384, 6, 2, 64, 16, 500, 9
    cos, sin = (torch.from_numpy(t).cuda() for t in Rotary(dh, 500000.0, max_pos).host_tables())
    x = rnd(m, k, seed=m).to(torch.bfloat16).cuda()
    w = rnd((nh + 2 * nkv) * dh, k, seed=5, scale=0.3).to(torch.bfloat16).cuda()
    wg = ops.pack_weight(w) if packed else w
    pos = torch.tensor(random.Random(3).sample(range(max_pos), m), dtype=torch.int32).cuda()
    slots = torch.tensor(random.Random(4).sample(range(pages * page), m), dtype=torch.int32).cuda()
    kw = {}
    if scaled:
        kw = dict(row_sumsq=(rnd(m, 3, seed=9).abs() * 40.0).cuda(), norm_width=k, eps=1e-5)
    cache_a = torch.zeros((pages, 2, nkv * dh * page), dtype=torch.bfloat16).cuda()
    cache_b = torch.zeros_like(cache_a)
    q_a = ops.gemm_skinny_qkv_rope(x, wg, pos, slots, cos, sin, cache_a, nh, nkv, dh, page, packed=packed, **kw)
    qkv = ops.gemm_skinny(x, wg, tiles=2, waves=8, packed=packed, **kw)
    ops.rope_kv_store(qkv, pos, nh, nkv, dh, cos, sin, dh, 0, cache_b, slots, page)
    assert torch.equal(q_a, qkv[:, :nh * dh])
    assert torch.equal(cache_a, cache_b)
    assert float(cache_a.float().abs().max()) > 0


def test_gemm_skinny_add_norm_refuses_what_it_cannot_take():
    from llama_cu_amd.kernels import ops
    x = rnd(33, 64).to(torch.bfloat16).cuda()
    w = rnd(32, 64).to(torch.bfloat16).cuda()
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny_add_norm(x, w, torch.zeros(33, 32).cuda(), torch.ones(32).cuda())        # more than 32 rows
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny_add_norm(x[:4], w, torch.zeros(4, 32, dtype=torch.bfloat16).cuda(), torch.ones(32).cuda())
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(x[:4], w, row_sumsq=torch.zeros(3, 2).cuda(), norm_width=64, eps=1e-5)    # rows do not match


@pytest.mark.parametrize("m,n,k", [(1, 16, 4), (8, 301, 172), (17, 100, 64), (70, 4096, 352), (300, 1000, 4096)])
def test_gemm_skinny_f32(m, n, k):
    from llama_cu_amd.kernels import ops
    x, w = rnd(m, k, seed=m), rnd(n, k, seed=n + 3)
    want = plain.linear(x, w)
    close(ops.gemm_skinny_f32(x.cuda(), w.cuda()), want, "float32")
    c = rnd(m, n, seed=9)
    cg = c.cuda()
    ops.gemm_skinny_f32(x.cuda(), w.cuda(), out=cg, accumulate=True)
    close(cg, c.double() + want, "float32", "accumulate")


def test_gemm_skinny_f32_is_true_32_bit_and_rows_are_independent():
    from llama_cu_amd.kernels import ops
    a = torch.full((4, 256), 1.0 + 2.0 ** -12)
    w = torch.full((20, 256), 1.0 + 2.0 ** -12)
    out = ops.gemm_skinny_f32(a.cuda(), w.cuda())
    assert float((out.double().cpu() - 256.125).abs().max()) < 1e-3          # a reduced-precision mode gives 256
    x, w = rnd(150, 512, seed=1).cuda(), rnd(77, 512, seed=2).cuda()
    whole = ops.gemm_skinny_f32(x, w)
    for r in (0, 15, 16, 63, 64, 149):                                        # alone, in a batch of few, in any tile of 64
        assert torch.equal(whole[r:r + 1], ops.gemm_skinny_f32(x[r:r + 1], w))
    assert torch.equal(whole[60:70], ops.gemm_skinny_f32(x[60:70], w))


def test_feed_tokens():
    """tokens[dst[i]] = sampled[src[i]]; pairs outside either array are left out."""
    from llama_cu_amd.kernels import ops
    g = torch.Generator().manual_seed(0)
    tokens = torch.randint(0, 1000, (37,), generator=g, dtype=torch.int32)
    sampled = torch.randint(0, 1000, (9,), generator=g, dtype=torch.int32)
    src = torch.tensor([8, 0, 3, 5], dtype=torch.int32)
    dst = torch.tensor([36, 1, 20, 7], dtype=torch.int32)
    want = tokens.clone()
    want[dst.long()] = sampled[src.long()]
    got = tokens.cuda()
    ops.feed_tokens(got, sampled.cuda(), src.cuda(), dst.cuda())
    assert torch.equal(got.cpu(), want)
    got2 = tokens.cuda()
    ops.feed_tokens(got2, sampled.cuda(), torch.tensor([9, -1, 2], dtype=torch.int32).cuda(),
                    torch.tensor([0, 1, 37], dtype=torch.int32).cuda())
    assert torch.equal(got2.cpu(), tokens)


# ------------------------------------------------------------------ random weights
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_weights_are_the_same_bits_on_the_host_and_on_the_gpu(dtype):
    """One generator for both: every tensor of Tiny B and one matrix of the Llama-3-8B shape
    (4096 x 14336) made on the GPU equal, bit for bit, the ones made on the host from the same
    seed; other names and other seeds give other streams."""
    import common
    from llama_cu_amd.config import LlamaConfig
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import DecoderModel, TensorSpec
    from llama_cu_amd.weights import fill_normal, random_tensors, stream_key
    expected = DecoderModel(llama_spec(LlamaConfig.from_dict(common.TINY_B))).tensors()
    host = random_tensors(expected, 11, dtype=DT[dtype], device="cpu")
    dev = random_tensors(expected, 11, dtype=DT[dtype], device="cuda")
    assert set(host) == set(dev) and len(host) > 20
    for name in host:
        assert torch.equal(host[name], dev[name].cpu()), name
    other = random_tensors(expected, 12, dtype=DT[dtype], device="cuda")
    assert not torch.equal(other["model.norm.weight"], dev["model.norm.weight"])
    assert not torch.equal(dev["model.layers.0.mlp.up_proj.weight"], dev["model.layers.0.mlp.gate_proj.weight"])
    big = {"model.layers.31.mlp.down_proj.weight": TensorSpec((4096, 14336))}
    h = random_tensors(big, 3, dtype=DT[dtype], device="cpu")["model.layers.31.mlp.down_proj.weight"]
    g = random_tensors(big, 3, dtype=DT[dtype], device="cuda")["model.layers.31.mlp.down_proj.weight"]
    assert torch.equal(h, g.cpu())
    assert abs(float(h.float().std()) - 0.02) < 1e-4 and abs(float(h.float().mean())) < 1e-4
    # a part of a stream made alone
    from llama_cu_amd.kernels import ops
    key = stream_key(3, "x")
    whole = fill_normal(torch.empty(5000, dtype=DT[dtype]), key, 1.0)
    part = ops.random_fill(torch.empty(777, dtype=DT[dtype], device="cuda"), key, 1.0, first=1234)
    assert torch.equal(part.cpu(), whole[1234:1234 + 777])
