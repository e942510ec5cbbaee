"""The decode attention entry point that allocates nothing (csrc/kernels/attention_static.h),
called through ctypes as a caller that cannot allocate would call it: its output against the
existing entry point's, which takes the parts' memory from its caller, on two calls in a row, the
second with a smaller input (so that what the first call left in the library's buffer is there
when the second runs); a call that needs more than the buffer holds is refused."""
import ctypes

import pytest
import torch

from test_gpu_kernels import paged_case

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _decode(lib, entry, q, out, cache, step, nh, nkv, dh, page, splits, parts=None):
    bt = step.block_table(0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(cache), _ptr(bt), bt.shape[1], _ptr(step.q_start),
            _ptr(step.ctx_len), _ptr(None), step.n_req, nh, nkv, dh, page, ctypes.c_float(dh ** -0.5), 0, splits]
    if parts is not None:
        args += [_ptr(parts[0]), _ptr(parts[1])]
    return getattr(lib, entry)(*args, stream)


def test_decode_attention_that_allocates_nothing_equals_the_one_that_is_given_its_memory():
    from llama_cu_amd.kernels import build
    lib = build.load("attention_mfma")
    lib.lcu_attention_static_scratch_bytes.restype = ctypes.c_longlong
    lib.lcu_attention_static_scratch_needed.restype = ctypes.c_longlong
    limit = lib.lcu_attention_static_scratch_bytes()
    assert limit == 16 << 20
    assert lib.lcu_attention_static_init() == 0
    # the first call is the larger one: five requests in six parts; the second, three requests in four parts, runs
    # over what the first left in the buffer; then other head sizes, head counts and page sizes over what those left
    calls = [((8, 2, 128, 16), [700, 33, 2049, 1, 512], 6), ((8, 2, 128, 16), [300, 64, 1500], 4), ((8, 2, 128, 16), [90, 17], 1),
             ((6, 3, 64, 32), [400, 77, 1030, 2], 5), ((6, 3, 64, 32), [129, 9], 2), ((4, 4, 96, 48), [1000, 333], 3),
             ((16, 1, 32, 16), [65], 2)]
    for (nh, nkv, dh, page), ctx_lens, splits in calls:
        n = len(ctx_lens)
        q, cache, step, _ = paged_case("bfloat16", nh, nkv, dh, page, [1] * n, ctx_lens, 0, seed=n + dh)
        q, cache = q.cuda(), cache.cuda()
        need = lib.lcu_attention_static_scratch_needed(n, nh, dh, splits)
        assert need == (n * nh * splits * (dh + 2) * 4 if splits > 1 else 0) and need <= limit
        want = torch.full((n, nh * dh), float("nan"), dtype=torch.bfloat16, device="cuda")
        parts = (torch.empty(n * nh * splits * dh, dtype=torch.float32, device="cuda"),
                 torch.empty(n * nh * splits * 2, dtype=torch.float32, device="cuda"))
        assert _decode(lib, "lcu_attention_decode_bf16", q, want, cache, step, nh, nkv, dh, page, splits, parts) == 0
        got = torch.full_like(want, float("nan"))
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        assert _decode(lib, "lcu_attention_decode_bf16_static", q, got, cache, step, nh, nkv, dh, page, splits) == 0
        torch.cuda.synchronize()
        # the call took no memory from the driver (the kernels are loaded: the other entry point has just run them)
        assert torch.cuda.mem_get_info()[0] == free_before, (free_before, torch.cuda.mem_get_info()[0])
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got, want), f"{n} requests in {splits} parts, head size {dh}"
    nh, nkv, dh, page = 8, 2, 128, 16
    # more than the buffer holds: refused, nothing launched, the output untouched
    n, splits = 64, 512
    assert lib.lcu_attention_static_scratch_needed(n, nh, dh, splits) > limit
    q = torch.zeros(n, nh * dh, dtype=torch.bfloat16, device="cuda")
    out = torch.full_like(q, 3.0)
    bt = torch.zeros(n, 4, dtype=torch.int32, device="cuda")
    ones = torch.ones(n + 1, dtype=torch.int32, device="cuda")
    cache = torch.zeros(4, 2, nkv * dh * page, dtype=torch.bfloat16, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.lcu_attention_decode_bf16_static(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(cache), _ptr(bt), 4,
                                              _ptr(ones), _ptr(ones), _ptr(None), n, nh, nkv, dh, page,
                                              ctypes.c_float(1.0), 0, splits, stream)
    torch.cuda.synchronize()
    assert rc == -3 and bool((out == 3.0).all())
    # sizes that no kernel takes are told so, also where the parts would not fit the buffer: the arguments are
    # checked first, as the other entry point checks them
    for bad in (dict(nkv=3), dict(page=24), dict(dh=40)):
        a = {"nkv": nkv, "page": page, "dh": dh, **bad}
        rc = lib.lcu_attention_decode_bf16_static(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(cache), _ptr(bt), 4,
                                                  _ptr(ones), _ptr(ones), _ptr(None), n, nh, a["nkv"], a["dh"], a["page"],
                                                  ctypes.c_float(1.0), 0, splits, stream)
        assert rc in (-1, -2), (bad, rc)
    assert lib.lcu_attention_static_scratch_needed(2 ** 31 - 1, 2 ** 31 - 1, 2 ** 31 - 3, 2 ** 31 - 1) == 2 ** 63 - 1
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())
