"""The entry point that allocates nothing (csrc/no_alloc.h): nva_linear_skinny_static_bf16, called
through ctypes, against nva_linear_skinny_bf16 with a workspace that the caller brings - on two
calls in a row, the second with a smaller input, so that what the first left in the library's
static array would show if it were read."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
c_i32, c_i64, c_ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p
STATIC_FLOATS = 4 << 20


def _lib():
    from nano_vllm_amd.kernels import library
    lib = library.load("gemm_skinny", "bf16")
    for name in ("nva_linear_skinny_bf16", "nva_linear_skinny_static_bf16"):
        getattr(lib, name).restype = ctypes.c_int
    lib.nva_linear_skinny_static_need_bf16.restype = ctypes.c_int64
    lib.nva_gemm_skinny_last_error.restype = ctypes.c_char_p
    return lib


def _p(t):
    return None if t is None else c_ptr(t.data_ptr())


def _rand(shape, seed, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(torch.bfloat16).to(DEV)


def _both(lib, m, n, k, splits, kw, bias, swiglu, out_f32, seed):
    """The product through the entry point with a workspace and through the one without."""
    x, w = _rand((m, k), seed), _rand((n, k), seed + 1, 0.05)
    b = _rand((n,), seed + 2) if bias else None
    width = n // 2 if swiglu else n
    dtype = torch.float32 if out_f32 else torch.bfloat16
    stream = c_ptr(torch.cuda.current_stream().cuda_stream)
    used_a, used_b = ctypes.c_int(0), ctypes.c_int(0)
    workspace = torch.full((splits * m * n,), float("nan"), dtype=torch.float32, device=DEV)
    want = torch.empty((m, width), dtype=dtype, device=DEV)
    rc = lib.nva_linear_skinny_bf16(_p(x), c_i64(k), _p(w), c_i64(k), _p(b), _p(want), c_i64(width), c_i32(out_f32),
                                    c_i32(swiglu), _p(workspace), c_i32(splits), c_i32(kw), c_i32(0), c_i64(m), c_i64(n),
                                    c_i64(k), ctypes.byref(used_a), stream)
    assert rc == 0, lib.nva_gemm_skinny_last_error()
    got = torch.full((m, width), float("nan"), dtype=dtype, device=DEV)
    before = torch.cuda.memory_allocated()
    rc = lib.nva_linear_skinny_static_bf16(_p(x), c_i64(k), _p(w), c_i64(k), _p(b), _p(got), c_i64(width), c_i32(out_f32),
                                           c_i32(swiglu), c_i32(splits), c_i32(kw), c_i64(m), c_i64(n), c_i64(k),
                                           ctypes.byref(used_b), stream)
    assert rc == 0, lib.nva_gemm_skinny_last_error()
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert used_a.value == used_b.value
    need = lib.nva_linear_skinny_static_need_bf16(_p(b), c_i32(swiglu), c_i32(splits), c_i64(m), c_i64(n), c_i64(k))
    assert need == (0 if splits == 1 and not bias else used_b.value * m * n) and need <= STATIC_FLOATS
    # against plain arithmetic as well
    y = x.double() @ w.double().T
    if bias:
        y = y + b.double()
    if swiglu:
        y = y.float().to(torch.bfloat16).float()
        y = torch.nn.functional.silu(y[:, : n // 2]) * y[:, n // 2:]
    plain = y.float() if out_f32 else y.float().to(torch.bfloat16).float()
    assert float((got.float() - plain).abs().max()) <= 2.0 ** -7 * float(plain.abs().max())
    return got, want


def test_static_scratch_entry_point_equals_the_one_with_a_workspace():
    lib = _lib()
    # the first call fills a good part of the static array ...
    got, want = _both(lib, m=8, n=4096, k=4096, splits=8, kw=1, bias=True, swiglu=False, out_f32=False, seed=1)
    assert torch.equal(got, want)
    # ... the second is smaller in every size, with another split and another form of the result
    got, want = _both(lib, m=3, n=1000, k=1288, splits=4, kw=4, bias=False, swiglu=False, out_f32=True, seed=5)
    assert torch.equal(got, want)
    # more forms, each after the other on the same array: gated through partial sums, more rows
    # of x, one range of k (no partial sums at all)
    for case in (dict(m=5, n=2048, k=520, splits=2, kw=2, bias=False, swiglu=True, out_f32=False, seed=9),
                 dict(m=40, n=320, k=12288, splits=16, kw=1, bias=True, swiglu=False, out_f32=False, seed=13),
                 dict(m=2, n=130, k=72, splits=1, kw=1, bias=False, swiglu=False, out_f32=False, seed=17),
                 dict(m=1, n=4096, k=4096, splits=4, kw=4, bias=False, swiglu=False, out_f32=False, seed=21)):
        got, want = _both(lib, **case)
        assert torch.equal(got, want), case


def test_static_scratch_entry_point_refuses_what_its_array_cannot_hold():
    lib = _lib()
    m, n, k, splits = 64, 151936, 512, 2                     # 2 x 64 x 151936 floats = 74 MiB of partial sums
    x, w = _rand((m, k), 1), torch.zeros((n, k), dtype=torch.bfloat16, device=DEV)
    y = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=DEV)
    used = ctypes.c_int(0)
    rc = lib.nva_linear_skinny_static_bf16(_p(x), c_i64(k), _p(w), c_i64(k), None, _p(y), c_i64(n), c_i32(0), c_i32(0),
                                           c_i32(splits), c_i32(1), c_i64(m), c_i64(n), c_i64(k), ctypes.byref(used),
                                           c_ptr(torch.cuda.current_stream().cuda_stream))
    assert rc != 0
    msg = lib.nva_gemm_skinny_last_error().decode()
    assert "static array holds 4194304" in msg and "16 MiB" in msg, msg
    torch.cuda.synchronize()
    assert float(y.min()) == 7.0                             # nothing ran
    # what the other entry point refuses is refused here too
    rc = lib.nva_linear_skinny_static_bf16(_p(x), c_i64(k), _p(w), c_i64(k), None, _p(y), c_i64(n), c_i32(0), c_i32(0),
                                           c_i32(1), c_i32(3), c_i64(m), c_i64(n), c_i64(k), ctypes.byref(used),
                                           c_ptr(torch.cuda.current_stream().cuda_stream))
    assert rc != 0 and "waves share rows" in lib.nva_gemm_skinny_last_error().decode()
