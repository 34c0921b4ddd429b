"""The product that allocates nothing (``atom_linear_skinny_static``), called through ctypes, against
the entry points it shares its kernels with (``atom_gemm_skinny`` + ``atom_splitk_reduce`` with a
workspace that the caller allocates): the same bits, on two calls in a row of which the second is
smaller, with the library's own buffer still holding the first call's slices."""

import ctypes

import pytest
import torch

from helpers import gpu_ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _rnd(shape, seed, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


def _existing(lib, x, w, bias, out_f32):
    """The existing entry points, with the slices in a tensor allocated here."""
    m, k = x.shape
    n = w.shape[0]
    y = torch.empty((m, n), dtype=torch.float32 if out_f32 else torch.bfloat16, device=DEV)
    splits = lib.atom_gemm_skinny_splits(m, n, k, 0)
    if splits == 1:
        assert lib.atom_gemm_skinny(_ptr(x), _ptr(w), _ptr(bias), _ptr(y), None, m, n, k, int(out_f32), 0,
                                    _stream()) == 0
        return y, splits
    partial = torch.empty((splits, m, n), dtype=torch.float32, device=DEV)
    assert lib.atom_gemm_skinny(_ptr(x), _ptr(w), None, None, _ptr(partial), m, n, k, 0, 0, _stream()) == 0
    assert lib.atom_splitk_reduce(_ptr(partial), _ptr(bias), _ptr(y), m, n, splits, int(out_f32), _stream()) == 0
    return y, splits


def _static(lib, x, w, bias, out_f32, y=None):
    m, k = x.shape
    n = w.shape[0]
    if y is None:
        y = torch.full((m, n), float("nan"), dtype=torch.float32 if out_f32 else torch.bfloat16, device=DEV)
    status = lib.atom_linear_skinny_static(_ptr(x), _ptr(w), _ptr(bias), _ptr(y), m, n, k, int(out_f32), _stream())
    return status, y


def test_static_product_matches_the_allocating_one_on_two_calls_in_a_row():
    lib = gpu_ops().lib
    for fn in ("atom_linear_skinny_static", "atom_linear_skinny_static_init"):
        getattr(lib, fn).restype = ctypes.c_int
    lib.atom_linear_skinny_static_limit.restype = ctypes.c_long
    assert lib.atom_linear_skinny_static_init() == 0
    limit = lib.atom_linear_skinny_static_limit()
    assert limit == 4 * 1024 * 1024

    # first call: 8 rows, a width that is no multiple of 64, K cut into slices, bias, bfloat16 out;
    # second call, at once: fewer rows, narrower, float32 out, no bias (the buffer still holds the first's slices)
    calls = [((8, 2056, 1000), True, False), ((3, 1032, 264), False, True)]
    inputs = []
    for (m, k, n), with_bias, out_f32 in calls:
        x = _rnd((m, k), 1 + m)
        w = _rnd((n, k), 2 + n, scale=0.05)
        bias = _rnd((n,), 3 + n, torch.float32) if with_bias else None
        inputs.append((x, w, bias, out_f32))
    results = []
    outs = [torch.full((x.shape[0], w.shape[0]), float("nan"), dtype=torch.float32 if f else torch.bfloat16,
                       device=DEV) for x, w, _, f in inputs]
    before = torch.cuda.memory_allocated()
    for (x, w, bias, out_f32), y in zip(inputs, outs):
        status, got = _static(lib, x, w, bias, out_f32, y)
        assert status == 0
        results.append(got)
    assert torch.cuda.memory_allocated() == before, "the entry point must not allocate through torch either"
    torch.cuda.synchronize()
    for (x, w, bias, out_f32), got in zip(inputs, results):
        want, splits = _existing(lib, x, w, bias, out_f32)
        assert splits > 1, "the case must go through the slices"
        torch.cuda.synchronize()
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, want), f"max diff {(got.float() - want.float()).abs().max().item():.3e}"
        # and against the product itself
        ref = x.float() @ w.float().T + (bias if bias is not None else 0)
        assert (got.float() - ref).abs().max().item() <= 2e-2 * ref.abs().max().item()


def test_static_product_without_slices_and_refusals():
    lib = gpu_ops().lib
    lib.atom_linear_skinny_static.restype = ctypes.c_int
    # a product whose K the kernel does not cut goes straight to y
    x, w = _rnd((20, 512), 5), _rnd((40000, 512), 6, scale=0.05)
    status, got = _static(lib, x, w, None, False)
    assert status == 0
    want, splits = _existing(lib, x, w, None, False)
    torch.cuda.synchronize()
    assert splits == 1 and torch.equal(got, want)
    # more slice elements than the library's buffer holds: refused, nothing launched, y untouched
    x, w = _rnd((8, 4096), 7), torch.zeros((151936, 4096), dtype=torch.bfloat16, device=DEV)
    splits = lib.atom_gemm_skinny_splits(8, 151936, 4096, 0)
    assert splits * 8 * 151936 > lib.atom_linear_skinny_static_limit()
    status, y = _static(lib, x, w, None, False)
    torch.cuda.synchronize()
    assert status == 5 and torch.isnan(y.float()).all()
    # more rows than the skinny kernels take, K not a multiple of 8, a null operand
    assert _static(lib, _rnd((200, 512), 9), _rnd((256, 512), 10), None, False)[0] == 3
    assert _static(lib, _rnd((4, 100), 11), _rnd((256, 100), 12), None, False)[0] == 3
    assert lib.atom_linear_skinny_static(None, _ptr(w), None, _ptr(y), 4, 151936, 4096, 0, _stream()) == 2
