"""dsdpa_fwd_noalloc: the forward whose workspace is a buffer built into the library (for callers that cannot
allocate), against dsdpa_fwd_f32 / dsdpa_fwd_bf16 with a caller-owned workspace. Same kernels, so the results
must be identical bit for bit; two calls in a row, the second on a smaller input (the buffer keeps the first
call's contents)."""
import sys

import pytest
import torch

from ops import _native

pytestmark = pytest.mark.gpu

CODE = {torch.float32: _native.DSDPA_F32, torch.bfloat16: _native.DSDPA_BF16}
SFX = {torch.float32: "f32", torch.bfloat16: "bf16"}


def _inputs(seed, B, V, H, Himg, Wimg, D, P, dtype):
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v = (torch.randn(B, V, H, L, D, generator=g).to(dtype).cuda() for _ in range(3))
    c = (torch.rand(B, V, L, V, P, 2, generator=g) * 1.2 - 0.1).cuda()
    return q, k, v, c


def _both(lib, shape, dtype, seed):
    B, V, H, Himg, Wimg, D, P = shape
    q, k, v, c = _inputs(seed, *shape, dtype)
    st = torch.cuda.current_stream().cuda_stream
    need = lib.dsdpa_fwd_workspace_bytes(CODE[dtype], B, V, H, Himg, Wimg, D, P)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    out_a, out_b = torch.full_like(q, float("nan")), torch.full_like(q, float("nan"))
    lse_a = torch.full((B, V, H, Himg * Wimg), float("nan"), device="cuda")
    lse_b = lse_a.clone()
    _native.check(getattr(lib, "dsdpa_fwd_" + SFX[dtype])(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), out_a.data_ptr(), lse_a.data_ptr(), ws.data_ptr(),
        B, V, H, Himg, Wimg, D, P, 0.25, None, st))
    torch.cuda.synchronize()

    def call():
        _native.check(lib.dsdpa_fwd_noalloc(
            CODE[dtype], q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), out_b.data_ptr(), lse_b.data_ptr(),
            B, V, H, Himg, Wimg, D, P, 0.25, None, st))
        torch.cuda.synchronize()

    # The first call on a device may load the code object and looks the built-in buffer's address up; from the
    # second on, a call must leave the DRIVER's free memory as it found it (torch's own counters would not see a
    # hipMalloc made inside the library) -- and torch's allocator must not have been asked for anything either.
    call()
    out_b.fill_(float("nan")), lse_b.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before, reserved_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    call()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    return need, (out_a, lse_a), (out_b, lse_b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_noalloc_forward_matches_workspace_forward_twice(dtype):
    lib = _native.load()
    # first a larger shape, then a smaller one: both on the staged kernels (they are the ones with a workspace)
    for seed, shape in ((51, (2, 4, 3, 9, 11, 32, 37)), (52, (1, 3, 2, 5, 6, 32, 13))):
        print(f"[case] no-alloc forward {shape} {dtype}", flush=True)
        sys.stdout.flush()
        need, (out_a, lse_a), (out_b, lse_b) = _both(lib, shape, dtype, seed)
        assert 0 < need <= _native.NOALLOC_SCRATCH_BYTES
        assert torch.isfinite(out_b.float()).all() and torch.isfinite(lse_b).all()
        assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)


def test_noalloc_forward_tile_flags_and_slabs():
    lib = _native.load()
    # 16-bit storage, 64 samples per view, planes too large for LDS: the kernel on tiles of 16 queries keeps its
    # tile flags in the built-in buffer (uniform coordinates: most tiles are left to the per-query kernel behind it)
    for seed, shape in ((55, (1, 2, 2, 40, 36, 64, 64)), (56, (1, 2, 1, 33, 30, 128, 64))):
        print(f"[case] no-alloc forward, tile flags {shape}", flush=True)
        need, (out_a, lse_a), (out_b, lse_b) = _both(lib, shape, torch.bfloat16, seed)
        assert 0 < need <= _native.NOALLOC_SCRATCH_BYTES
        assert torch.isfinite(out_b.float()).all()
        assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    # fp32, 16 samples per view: the slab kernel (no workspace, 150 KB of LDS)
    print("[case] no-alloc forward, slab kernel", flush=True)
    need, (out_a, lse_a), (out_b, lse_b) = _both(lib, (1, 2, 2, 28, 30, 64, 16), torch.float32, 57)
    assert need == 0
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)


def test_noalloc_forward_without_workspace_and_refusal():
    lib = _native.load()
    # planes too large for LDS: the gather kernels, no workspace at all
    print("[case] no-alloc forward, shape without a workspace", flush=True)
    need, (out_a, lse_a), (out_b, lse_b) = _both(lib, (1, 2, 2, 40, 40, 64, 6), torch.float32, 53)
    assert need == 0
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    # a shape whose table does not fit in the built-in buffer is refused before anything is launched
    print("[case] no-alloc forward, refusal", flush=True)
    shape = (4, 8, 1, 14, 14, 32, 64)
    B, V, H, Himg, Wimg, D, P = shape
    assert lib.dsdpa_fwd_workspace_bytes(_native.DSDPA_F32, *shape) > _native.NOALLOC_SCRATCH_BYTES
    q, k, v, c = _inputs(54, *shape, torch.float32)
    out = torch.full_like(q, 7.0)
    lse = torch.zeros(B, V, H, Himg * Wimg, device="cuda")
    rc = lib.dsdpa_fwd_noalloc(_native.DSDPA_F32, q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(),
                               out.data_ptr(), lse.data_ptr(), *shape, 0.25, None, None)
    torch.cuda.synchronize()
    assert rc == _native.ERR_SCRATCH
    assert (out == 7.0).all()
    assert b"scratch" in lib.dsdpa_error_string(rc)
