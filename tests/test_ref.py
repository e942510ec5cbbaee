"""The plain C++ references of the kernels (csrc/ref/ref.cpp) against the plain Python
implementation: two independent texts of the same formulas must agree."""
import random

import pytest
import torch

import llama_cu_amd
from llama_cu_amd.kernels import ref

import plain


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, tol=2e-6):
    want = want.double()
    scale = float(want.abs().max()) + 1e-30
    assert float((got.double() - want).abs().max()) <= tol * scale


def test_rows():
    table = rnd(301, 100, seed=1)
    ids = [5, 300, 0, 5]
    assert torch.equal(ref.embedding(table, ids), plain.embedding(table, ids).float())
    for n, d, eps in ((1, 64, 1e-5), (3, 172, 1e-6), (2, 4096, 1e-2)):
        x, w = rnd(n, d, seed=2, scale=0.03), 1 + rnd(d, seed=3, scale=0.1)
        close(ref.rms_norm(x, w, eps), plain.rms_norm(x, w, eps))
    a, w = rnd(5, 136, seed=4), rnd(301, 136, seed=5)
    close(ref.gemm_nt(a, w), plain.linear(a, w))
    gu = rnd(7, 2 * 172, seed=6, scale=3.0)
    close(ref.swiglu(gu), plain.swiglu(gu[:, :172], gu[:, 172:]))


@pytest.mark.parametrize("nh,nkv,dh,page,pairing,rot", [(4, 4, 16, 16, "half", 16), (6, 2, 48, 8, "adjacent", 48),
                                                        (8, 2, 128, 32, "half", 128), (3, 1, 32, 16, "adjacent", 32)])
def test_rotation_and_cache_layout_and_attention_over_pages(nh, nkv, dh, page, pairing, rot):
    """Tokens of two requests are rotated and written into shuffled pages by the C++ reference,
    which then attends over those pages: equal to the plain rotation and the plain attention over
    contiguous keys and values."""
    theta, lens = 10000.0, [37, 5]
    rng = random.Random(dh)
    n_pages = sum((l + page - 1) // page for l in lens) + 2
    free = list(range(n_pages))
    rng.shuffle(free)
    cache = torch.full((n_pages, 2, nkv * dh * page), float("nan"))
    sin, cos = plain.rope_tables(64, rot, theta)
    tables, qs, wants = [], [], []
    for r, l in enumerate(lens):
        qkv = rnd(l, (nh + 2 * nkv) * dh, seed=10 + r)
        q = qkv[:, :nh * dh].view(l, nh, dh)
        k = qkv[:, nh * dh:(nh + nkv) * dh].view(l, nkv, dh)
        v = qkv[:, (nh + nkv) * dh:].view(l, nkv, dh)
        table = [free.pop() for _ in range((l + page - 1) // page)]
        slots = [table[j // page] * page + j % page for j in range(l)]
        pos = list(range(l))
        out = ref.rope_kv_write(qkv.clone(), pos, slots, theta, nh, nkv, dh, rot, 1 if pairing == "adjacent" else 0, page, cache)
        q_rot = plain.rope(q, pos, sin, cos, pairing)
        close(out[:, :nh * dh].view(l, nh, dh), q_rot)
        k_rot = plain.rope(k, pos, sin, cos, pairing)
        tables.append(table + [0] * (8 - len(table)))
        # the last 3 tokens of the request are the step's queries
        qs.append(q_rot[-3:].reshape(3, nh * dh).float())
        wants.append(plain.attention(q_rot[-3:], k_rot, v, dh ** -0.5, first_pos=l - 3, window=None).reshape(3, nh * dh))
    got = ref.paged_attention(torch.cat(qs).contiguous(), cache, torch.tensor(tables), [0, 3, 6], lens, nh, nkv, dh, page, dh ** -0.5)
    close(got, torch.cat(wants), 1e-5)


def test_attention_with_a_window_over_pages():
    nh, nkv, dh, page, l = 4, 2, 16, 8, 29
    qkv = rnd(l, (nh + 2 * nkv) * dh, seed=3)
    cache = torch.zeros(5, 2, nkv * dh * page)
    table = [3, 0, 4, 1]
    slots = [table[j // page] * page + j % page for j in range(l)]
    ref.rope_kv_write(qkv, list(range(l)), slots, 1e4, nh, nkv, dh, 0, 0, page, cache)          # rot_dim 0: no rotation
    q = qkv[:, :nh * dh].view(l, nh, dh)
    k = qkv[:, nh * dh:(nh + nkv) * dh].view(l, nkv, dh)
    v = qkv[:, (nh + nkv) * dh:].view(l, nkv, dh)
    for window in (0, 5):
        got = ref.paged_attention(qkv[:, :nh * dh], cache, torch.tensor([table]), [0, l], [l], nh, nkv, dh, page, 0.3, window)
        # (q is a strided view: its rows are the whole qkv rows apart)
        want = plain.attention(q, k, v, 0.3, first_pos=0, window=window or None).reshape(l, nh * dh)
        close(got, want, 1e-5)


def test_sampling():
    """The sorted inverse-CDF draw: equal to the plain implementation for many numbers u, with
    top-k, top-p and ties."""
    logits = rnd(301, seed=7, scale=2.0)
    logits[17] = logits[200] = logits.max() + 0.5                    # two equal largest logits
    assert ref.sample(logits, 0.0, 1.0, 10 ** 9, 0.3) == 17 == plain.sample(logits, 0.0, 1.0, 10 ** 9, 0.3)
    assert ref.sample(logits, 0.7, 1.0, 1, 0.9) == 17
    rng = random.Random(1)
    for temperature, top_p, top_k in ((0.8, 1.0, 10 ** 9), (1.3, 0.6, 10 ** 9), (0.5, 1.0, 5), (1.0, 0.9, 40)):
        for _ in range(60):
            u = rng.random()
            assert ref.sample(logits, temperature, top_p, top_k, u) == plain.sample(logits, temperature, top_p, top_k, float(torch.tensor(u, dtype=torch.float32)))
