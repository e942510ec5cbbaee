"""Every kernel against its plain C++ reference (csrc/ref/ref.cpp) at ragged shapes: widths 64,
128 and 4096, head sizes 16, 32 and 128, feed-forward widths 172, 352 and 14336, and 1, 2, 3, 17,
48 and 2,048 rows; in 32-bit and in bfloat16."""
import random

import pytest
import torch

from test_gpu_kernels import DT, close, rnd

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 3, 17, 48, 2048]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [64, 128, 4096])
def test_embedding_and_rmsnorm_against_the_c_reference(dtype, d):
    from llama_cu_amd.kernels import ops, ref
    table = rnd(300, d, seed=d).to(DT[dtype])
    w = (1 + rnd(d, seed=3, scale=0.1)).to(DT[dtype])
    for n in ROWS:
        ids = torch.randint(0, 300, (n,), dtype=torch.int32, generator=torch.Generator().manual_seed(n))
        x = torch.empty(n, d, dtype=torch.float32, device="cuda")
        ops.embedding_gather(table.cuda(), ids.cuda(), x)
        assert torch.equal(x.cpu(), ref.embedding(table.float(), ids))
        out = torch.empty(n, d, dtype=DT[dtype], device="cuda")
        ops.rmsnorm(x, w.cuda(), 1e-5, out)
        close(out, ref.rms_norm(x.cpu(), w.float(), 1e-5), dtype, f"rmsnorm {n} x {d}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("di", [172, 352, 14336])
def test_swiglu_against_the_c_reference(dtype, di):
    from llama_cu_amd.kernels import ops, ref
    for n in ROWS:
        gu = rnd(n, 2 * di, seed=n, scale=2.0).to(DT[dtype])
        close(ops.swiglu(gu.cuda()), ref.swiglu(gu.float()), dtype, f"swiglu {n} x {di}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (2, 172, 128), (3, 4096, 4096), (17, 352, 128), (48, 4096, 352 * 4), (17, 128, 14336),
                                   (48, 14336, 128), (2048, 64, 128), (2048, 172, 64)])
def test_products_against_the_c_reference(dtype, m, n, k):
    """Through ``parts.linear.linear``, which picks the kernel for the shape: the weight-streaming
    kernels, the kernel that shares the rows through LDS, the library for many bfloat16 rows, the
    32-bit kernel."""
    from llama_cu_amd.kernels import ref
    from llama_cu_amd.parts.linear import Weight, linear
    a = rnd(m, k, seed=m).to(DT[dtype])
    w = rnd(n, k, seed=n, scale=0.05).to(DT[dtype])
    got = linear(a.cuda(), Weight(w.cuda()), out_dtype=DT[dtype])
    close(got, ref.gemm_nt(a.float(), w.float()), dtype, f"{m} x {n} x {k}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,dh,page", [(4, 4, 16, 16), (4, 1, 32, 32), (8, 2, 128, 16)])
def test_rotation_cache_write_and_attention_against_the_c_reference(dtype, nh, nkv, dh, page):
    """A batch of requests that feed 1, 2, 3, 17 and 48 tokens after histories of several lengths:
    the rotation kernel writes the step's keys and values into shuffled pages as the reference
    does, and the attention kernels read what the reference reads."""
    from llama_cu_amd.kernels import ops, ref
    from llama_cu_amd.parts.position import Rotary
    from test_gpu_kernels import Batch
    theta = 10000.0
    q_lens, ctx_lens = [1, 2, 3, 17, 48], [300, 2, 35, 17, 200]
    rng = random.Random(dh)
    need = [(c + page - 1) // page for c in ctx_lens]
    free = list(range(sum(need) + 2))
    rng.shuffle(free)
    tables = [[free.pop() for _ in range(k)] for k in need]
    tdt = DT[dtype]
    cache_ref = torch.zeros(sum(need) + 2, 2, nkv * dh * page)
    width = (nh + 2 * nkv) * dh
    # the histories first (by the reference alone), then the step by both
    hist, step_rows, positions, slots = [], [], [], []
    for r, (ql, cl) in enumerate(zip(q_lens, ctx_lens)):
        rows = rnd(cl, width, seed=100 + r).to(tdt).float()
        sl = [tables[r][j // page] * page + j % page for j in range(cl)]
        if cl > ql:
            ref.rope_kv_write(rows[:cl - ql].clone(), list(range(cl - ql)), sl[:cl - ql], theta, nh, nkv, dh, dh, 0, page, cache_ref)
        step_rows.append(rows[cl - ql:])
        positions += list(range(cl - ql, cl))
        slots += sl[cl - ql:]
    cache_ref = cache_ref.to(tdt).float()                              # what the engine's cache holds of the history
    cache_gpu = cache_ref.to(tdt).cuda()
    qkv = torch.cat(step_rows).contiguous()
    cos, sin = (torch.from_numpy(t).cuda() for t in Rotary(dh, theta, 512).host_tables())
    qkv_gpu = qkv.to(tdt).cuda()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    ops.rope_kv_store(qkv_gpu, i32(positions), nh, nkv, dh, cos, sin, dh, 0, cache_gpu, i32(slots), page)
    qkv_ref = ref.rope_kv_write(qkv.clone(), positions, slots, theta, nh, nkv, dh, dh, 0, page, cache_ref)
    close(qkv_gpu[:, :nh * dh], qkv_ref[:, :nh * dh], dtype, "rotated queries")
    close(cache_gpu, cache_ref, dtype, "cache after the step")
    step = Batch(q_lens, ctx_lens, tables, max(need) + 1).step
    out = torch.empty(qkv.shape[0], nh * dh, dtype=tdt, device="cuda")
    ops.paged_attention(qkv_gpu, out, cache_gpu, step, 0, nh, nkv, dh, page, dh ** -0.5, 0)
    bt = step.block_table(0).cpu()
    want = ref.paged_attention(qkv_gpu.float().cpu(), cache_gpu.float().cpu(), bt, step.q_start.cpu(), ctx_lens, nh, nkv, dh,
                               page, dh ** -0.5, 0)
    close(out, want, dtype, "attention")


def test_attention_of_2048_tokens_against_the_c_reference():
    from llama_cu_amd.kernels import ops, ref
    from test_gpu_kernels import Batch
    nh, nkv, dh, page, n = 2, 1, 128, 16, 2048
    qkv = rnd(n, (nh + 2 * nkv) * dh, seed=5).to(torch.bfloat16)
    table = list(range(n // page))
    random.Random(3).shuffle(table)
    slots = [table[j // page] * page + j % page for j in range(n)]
    cache = torch.zeros(n // page, 2, nkv * dh * page)
    rot = ref.rope_kv_write(qkv.float(), list(range(n)), slots, 5e5, nh, nkv, dh, dh, 0, page, cache)
    cache_gpu = cache.to(torch.bfloat16).cuda()
    q_gpu = rot.to(torch.bfloat16).cuda()
    step = Batch([n], [n], [table], n // page + 1).step
    out = torch.empty(n, nh * dh, dtype=torch.bfloat16, device="cuda")
    ops.paged_attention(q_gpu, out, cache_gpu, step, 0, nh, nkv, dh, page, dh ** -0.5, 0)
    want = ref.paged_attention(q_gpu.float().cpu(), cache_gpu.float().cpu(), step.block_table(0).cpu(), [0, n], [n], nh, nkv, dh,
                               page, dh ** -0.5, 0)
    close(out, want, "bfloat16", "prefill of 2,048 tokens")


@pytest.mark.parametrize("vocab", [301, 4096, 128256])
def test_sampling_against_the_c_reference(vocab):
    from llama_cu_amd.kernels import ref
    from llama_cu_amd.sampling import sampler
    rng = random.Random(vocab)
    rows = 24
    logits = rnd(rows, vocab, seed=vocab, scale=2.5)
    temperature = [rng.choice([0.5, 0.8, 1.0, 1.7]) for _ in range(rows)]
    top_p = [rng.choice([1.0, 0.9, 0.5]) for _ in range(rows)]
    top_k = [rng.choice([vocab, 40, 3]) for _ in range(rows)]
    u = [float(torch.tensor(rng.random(), dtype=torch.float32)) for _ in range(rows)]
    got = sampler.sample_rows(logits.cuda(), temperature, top_p, top_k, u).cpu().tolist()
    assert sampler.argmax(logits.cuda()).cpu().tolist() == [ref.sample(logits[r], 0.0, 1.0, vocab, 0.5) for r in range(rows)]
    differ = 0
    for r in range(rows):
        want = ref.sample(logits[r], temperature[r], top_p[r], top_k[r], u[r])
        if got[r] != want:
            # the kernel adds fixed-point weights, the reference 64-bit ones: a draw that falls within rounding of
            # the boundary between two tokens may go to the neighbour in the sorted order
            order = torch.sort(logits[r], descending=True, stable=True).indices.tolist()
            assert abs(order.index(got[r]) - order.index(want)) == 1, (r, got[r], want)
            differ += 1
    assert differ <= 1
