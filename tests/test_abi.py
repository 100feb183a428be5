"""CPU-side checks of the C ABI: the library loads without a GPU and exports
every symbol include/dsdpa.h declares; argument validation happens before any
launch, so the error paths run here too."""
import ctypes
import os
import re

import pytest

from ops import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dsdpa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dsdpa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_all_exported():
    lib = _native.load()
    declared = _declared_symbols()
    assert len(declared) >= 11
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/dsdpa.h but not exported"
    assert sorted(_native.SYMBOLS) == declared


def test_version_and_error_strings():
    lib = _native.load()
    assert lib.dsdpa_version() >= 200
    assert lib.dsdpa_error_string(0) == b"ok"
    for code in range(1, 10):
        assert len(lib.dsdpa_error_string(code)) > 3
    assert b"unknown" in lib.dsdpa_error_string(99)


def test_workspace_bytes():
    lib = _native.load()
    r256 = lambda b: (b + 255) // 256 * 256

    def table(B, V, Himg, Wimg, D, P, storage16):
        """per-coordinate table of the staged kernels: only when one K and one V plane fit in LDS"""
        L, e = Himg * Wimg, 2 if storage16 else 4
        if (L + 2) * 2 * D * e + 16 * 96 * 24 > 160 * 1024:
            return 0
        m = B * V * L * V * P
        return r256(m * 16) + r256(m * 4)

    def groups(V, H, L, D, e, P, NC, handed):
        # lists per (group of query views, cell) where the pairs are handed over and the q and dout rows of one
        # (batch, head) outgrow L2
        rows_bytes, M, cap = 2 * V * L * D * e, V * L * P, 4 << 20
        if not handed or rows_bytes <= cap:
            return 1
        g = min(V, (rows_bytes + cap - 1) // cap)
        while g > 1 and M // (g * NC) < 48:
            g -= 1
        vpg = (V + g - 1) // g
        return (V + vpg - 1) // vpg

    def handed_group(B, V, H, Himg, Wimg, D, P, storage16):
        """(batch, head) pairs whose (p, ds) pairs the backward workspace holds at a time: on shapes whose planes
        do not fit in LDS, as many as 128 MiB hold, in groups of equal size; 0 when one pair's do not fit"""
        per_bh, cap = V * Himg * Wimg * V * P * 8, 128 << 20
        if table(B, V, Himg, Wimg, D, P, storage16) != 0 or per_bh > cap:
            return 0
        g = min(B * H, cap // per_bh)
        ngroups = (B * H + g - 1) // g
        return (B * H + ngroups - 1) // ngroups

    def expect(B, V, H, Himg, Wimg, D, P, storage16):
        rows, NC = B * V * H * Himg * Wimg, (Himg + 1) * (Wimg + 1)
        handed = handed_group(B, V, H, Himg, Wimg, D, P, storage16) > 0
        NC = NC * groups(V, H, Himg * Wimg, D, 2 if storage16 else 4, P, NC, handed)
        total = r256(rows * 8) + r256(B * V * NC * 4) + r256(B * V * (NC + 1) * 4) + r256(B * V * V * Himg * Wimg * P * 4)
        total += r256(B * V * V * Himg * Wimg * P * 8)          # positions beside the ids
        # work list of the dk/dv kernel: items of at most `piece` list entries, (cell, first entry, end) in 16 bytes each
        M = V * Himg * Wimg * P
        piece = (max(768, 4 * M // NC) + 63) // 64 * 64
        total += r256(B * V * (NC + M // piece + 1) * 16)
        # (p, ds) per query*sample of one group of (batch, head) pairs, dq kernel -> dk/dv kernel
        total += r256(handed_group(B, V, H, Himg, Wimg, D, P, storage16) * V * Himg * Wimg * V * P * 8)
        total += r256(2 * rows * D * 4) if storage16 else 0
        return total + table(B, V, Himg, Wimg, D, P, storage16)

    assert lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, 2, 6, 8, 18, 18, 32, 32, 0) == expect(2, 6, 8, 18, 18, 32, 32, False)
    assert lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_BF16, 2, 6, 8, 48, 48, 64, 32, 0) == expect(2, 6, 8, 48, 48, 64, 32, True)
    assert lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F16, 1, 2, 1, 3, 5, 16, 7, 0) == expect(1, 2, 1, 3, 5, 16, 7, True)
    # the pairs handed from dq to dk/dv never take more than 128 MiB, whatever the shape: 64x64, 64 samples per
    # view, 4 views, D = 128 (16 (batch, head) pairs of 32 MiB each) goes in groups of 4 ...
    assert handed_group(2, 4, 8, 64, 64, 128, 64, True) == 4
    c5 = lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_BF16, 2, 4, 8, 64, 64, 128, 64, 0)
    assert c5 == expect(2, 4, 8, 64, 64, 128, 64, True) and c5 < 2 * 2 * 4 * 8 * 4096 * 128 * 4 + (256 << 20)
    # ... and a shape where one pair's alone would take more (96x96, 6 views) hands nothing over
    assert handed_group(1, 6, 2, 96, 96, 64, 64, True) == 0
    assert lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_BF16, 1, 6, 2, 96, 96, 64, 64, 0) == expect(1, 6, 2, 96, 96, 64, 64, True)
    assert lib.dsdpa_fwd_workspace_bytes(_native.DSDPA_F32, 2, 6, 8, 18, 18, 32, 32) == table(2, 6, 18, 18, 32, 32, False) > 0
    assert lib.dsdpa_fwd_workspace_bytes(_native.DSDPA_F16, 1, 2, 1, 3, 5, 16, 7) == table(1, 2, 3, 5, 16, 7, True) > 0
    assert lib.dsdpa_fwd_workspace_bytes(_native.DSDPA_BF16, 2, 6, 8, 48, 48, 64, 32) == 0      # planes too large for LDS
    assert lib.dsdpa_fwd_workspace_bytes(7, 2, 6, 8, 18, 18, 32, 32) == 0
    assert lib.dsdpa_bwd_workspace_bytes(7, 2, 6, 8, 48, 48, 64, 32, 0) == 0
    assert lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, 0, 6, 8, 48, 48, 64, 32, 0) == 0
    # deterministic backward: a second id array and the list bounds on top (plus the sort's scratch, whose
    # size the sort routine reports on a machine with a GPU)
    plain = lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, 2, 6, 8, 18, 18, 32, 32, 0)
    det = lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, 2, 6, 8, 18, 18, 32, 32, _native.FLAG_DETERMINISTIC)
    assert det >= plain + r256(2 * 6 * 6 * 324 * 32 * 4) + r256(2 * 2 * 6 * 361 * 4)
    # coordinate gradient: 16 more bytes per coordinate pair where the planes and the larger descriptor block fit
    cg = lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, 2, 6, 8, 18, 18, 32, 32, _native.FLAG_COORDS_GRAD)
    assert cg == plain + r256(2 * 6 * 324 * 6 * 32 * 16)
    # 21x22 fp32 D32: 118784 plane bytes + 36864 fit, + 12288 more do not: no table at all with the flag
    fits = lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, 1, 2, 1, 21, 22, 32, 4, 0)
    nofit = lib.dsdpa_bwd_workspace_bytes(_native.DSDPA_F32, 1, 2, 1, 21, 22, 32, 4, _native.FLAG_COORDS_GRAD)
    assert fits == expect(1, 2, 1, 21, 22, 32, 4, False) and nofit == fits - table(1, 2, 21, 22, 32, 4, False)


def test_argument_validation_before_launch():
    """Bad arguments are rejected with an error code before anything touches the GPU."""
    lib = _native.load()
    fake = ctypes.c_void_p(0x1000)   # never dereferenced: validation fails first
    ok_dims = (1, 2, 2, 3, 4, 32, 2, 0.5, None, None)              # ... sm_scale, strides, stream
    bwd_dims = (1, 2, 2, 3, 4, 32, 2, 0.5, None, 0, None)    # ... sm_scale, strides, flags, stream
    assert lib.dsdpa_fwd_f32(None, fake, fake, fake, fake, fake, fake, *ok_dims) == 1
    assert lib.dsdpa_fwd_f32(fake, fake, fake, fake, fake, fake, None, *ok_dims) == 1    # this shape needs the workspace
    assert lib.dsdpa_fwd_f32(fake, fake, fake, fake, fake, fake, fake, 0, 2, 2, 3, 4, 32, 2, 0.5, None, None) == 2
    assert lib.dsdpa_fwd_bf16(fake, fake, fake, fake, fake, fake, fake, 1, 2, 2, 3, 4, 48, 2, 0.5, None, None) == 3
    assert lib.dsdpa_fwd_f16(fake, fake, fake, fake, fake, fake, fake, 1, 2, 2, 3, 4, 8, 2, 0.5, None, None) == 3
    assert lib.dsdpa_fwd_f32(fake, fake, fake, fake, fake, fake, fake, 1, 64, 64, 1024, 1024, 256, 2, 0.5, None, None) == 4
    # strides (host array: q's then k/v's element strides over batch, view, head, pixel)
    ll8 = ctypes.c_longlong * 8
    L, D = 12, 32
    contiguous = ll8(2 * 2 * L * D, 2 * L * D, L * D, D, 2 * 2 * L * D, 2 * L * D, L * D, D)
    odd_row = ll8(2 * 2 * L * D, 2 * L * D, L * D, D + 2, 2 * 2 * L * D, 2 * L * D, L * D, D)     # rows not 16-byte aligned
    short_row = ll8(2 * 2 * L * D, 2 * L * D, L * D, D - 4, 2 * 2 * L * D, 2 * L * D, L * D, D)   # rows overlap
    assert lib.dsdpa_fwd_f32(None, fake, fake, fake, fake, fake, fake, 1, 2, 2, 3, 4, 32, 2, 0.5, contiguous, None) == 1
    assert lib.dsdpa_fwd_f32(fake, fake, fake, fake, fake, fake, fake, 1, 2, 2, 3, 4, 32, 2, 0.5, odd_row, None) == 9
    assert lib.dsdpa_fwd_f32(fake, fake, fake, fake, fake, fake, fake, 1, 2, 2, 3, 4, 32, 2, 0.5, short_row, None) == 9
    # backward: the workspace is required
    args = [fake] * 10
    assert lib.dsdpa_bwd_bf16(*args, None, None, *bwd_dims) == 1
    assert lib.dsdpa_bwd_f32(*args, fake, None, *bwd_dims) == 1
    assert lib.dsdpa_bwd_f32(*args[:9], None, None, fake, *bwd_dims) == 1
    assert lib.dsdpa_bwd_f32(*args, None, fake, 1, 2, 2, 3, 4, 33, 2, 0.5, None, 0, None) == 3     # dcoords is optional
    assert lib.dsdpa_bwd_f32(*args, None, fake, 1, 2, 2, 3, 4, 32, 2, 0.5, None, 8, None) == 7     # unknown flag
    assert lib.dsdpa_bwd_f32(*args, fake, fake, 1, 2, 2, 3, 4, 32, 2, 0.5, None, _native.FLAG_DETERMINISTIC, None) == 7


def test_path_selector():
    assert _native.set_path(_native.PATH_AUTO) in (0, 1, 2)
    prev = _native.set_path(_native.PATH_GATHER)
    assert prev == _native.PATH_AUTO
    assert _native.set_path(_native.PATH_AUTO) == _native.PATH_GATHER
    with pytest.raises(ValueError):
        _native.set_path(77)


def test_operator_contract_errors_on_cpu():
    """The Python front-end raises the reference's exception classes (ops/triton.py:375,385-388)."""
    import torch
    from ops.triton import deform_sdpa_triton
    q = torch.randn(1, 2, 2, 12, 32)
    c = torch.rand(1, 2, 12, 2, 3, 2)
    with pytest.raises(NotImplementedError):
        deform_sdpa_triton(q.double(), q.double(), q.double(), c, 4, 3, 0.5)
    with pytest.raises(AssertionError):
        deform_sdpa_triton(q, q, q, c, 4, 4, 0.5)                      # L != W*H
    with pytest.raises(AssertionError):
        deform_sdpa_triton(q[..., :24], q[..., :24], q[..., :24], c, 4, 3, 0.5)   # head dim 24
    with pytest.raises(AssertionError):
        deform_sdpa_triton(q, q, q, c.transpose(3, 4).contiguous().transpose(3, 4), 4, 3, 0.5)
    with pytest.raises(RuntimeError):
        deform_sdpa_triton(q, q, q, c, 4, 3, 0.5)                      # CPU tensors: no fallback
