"""Fused deformable multi-view SDPA: the autograd front-end over libdsdpa.so.

Drop-in for the reference operator ``deform_sdpa_triton`` (``ops/triton.py:466``;
the module and function names are kept so ``from ops.triton import
deform_sdpa_triton`` keeps working -- there is no Triton here, the kernels are
hand-written HIP for gfx950 reached through a C ABI).

Contract mirrored from ``_fused_deform_sdpa`` (``ops/triton.py:377-466``):

* ``deform_sdpa_triton(q, k, v, coords, WIDTH, HEIGHT, sm_scale) -> out``,
  positional; q/k/v ``(B, N_VIEWS, N_HEADS, H*W, D)``, coords
  ``(B, N_VIEWS, H*W, N_VIEWS, N_SAMPLES, 2)`` normalised ``(x, y)``;
* gradients for q, k, v only; coords/WIDTH/HEIGHT/sm_scale get ``None``;
* ``AssertionError`` for unequal head dims, ``D`` outside {16,32,64,128,256},
  ``q.shape[3] != WIDTH*HEIGHT``, non-contiguous coords;
  ``NotImplementedError`` for an unsupported dtype;
* fp32 storage, or bf16/fp16 storage with fp32 accumulation.

Differences, all on purpose: coords are not cloned or pre-scaled (the kernels
un-normalise), ``out``/``dq`` are not zero-filled first, no scaled copy of K is
made, out-of-image taps follow the eager operator's per-tap zero padding
(``ops/torch.py:14-15``) rather than ``ops/triton.py:129,135-136``, strided
q/k/v are read in place where the head dimension is contiguous (and copied
otherwise) instead of asserted, dout is made contiguous, and only the
log-sum-exp is saved on top of the inputs and output.
"""
import torch

from . import _native

_SUFFIX = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}
_DTYPE_CODE = {torch.float32: _native.DSDPA_F32, torch.bfloat16: _native.DSDPA_BF16,
               torch.float16: _native.DSDPA_F16}


def _suffix_from(t):
    """Storage mode of a tensor (the reference's ``_dtype_mode_from``, ops/triton.py:367-375)."""
    try:
        return _SUFFIX[t.dtype]
    except KeyError:
        raise NotImplementedError(f"unsupported dtype {t.dtype}") from None


def _stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


def _check_inputs(q, k, v, coords, WIDTH, HEIGHT):
    sfx = _suffix_from(q)
    assert q.dim() == 5 and k.shape == q.shape and v.shape == q.shape, "q, k, v must share (B, V, H, L, D)"
    assert q.shape[-1] == k.shape[-1] == v.shape[-1]
    assert q.shape[-1] in {16, 32, 64, 128, 256}
    assert q.shape[3] == WIDTH * HEIGHT
    assert coords.is_contiguous()
    B, V, H, L, D = q.shape
    if coords.dim() != 6 or coords.shape[:4] != (B, V, L, V) or coords.shape[-1] != 2:
        raise RuntimeError(f"coords must be (B, V, L, V, P, 2) = ({B}, {V}, {L}, {V}, P, 2), got {tuple(coords.shape)}")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("q, k, v must share one dtype")
    if not q.is_cuda:
        raise RuntimeError("deform_sdpa_triton runs on the GPU only (HIP kernels); "
                           "use ops.torch.deform_sdpa_torch for an eager operator")
    if not (k.device == q.device and v.device == q.device and coords.device == q.device):
        raise RuntimeError("q, k, v, coords must be on one device")
    return sfx


# The backward runs its dk/dv side beside the dq side on a second stream of the library's (forked from and joined
# to the caller's stream inside the call). True keeps every launch on the caller's stream (same results).
SINGLE_STREAM = False


class _fused_deform_sdpa(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, coords, WIDTH, HEIGHT, sm_scale, *extra):
        # extra = (coords_grad,): an eighth, optional argument the reference does not have. Left out (or False) the
        # operator behaves like the reference's: no gradient for coords (ops/triton.py:464). True asks for
        # the gradient of coords as well, the one the eager operator gets through grid_sample
        # (ops/torch.py:14-15).
        if len(extra) > 1:
            raise TypeError("deform_sdpa_triton takes 7 arguments and an optional coords_grad flag")
        ctx.n_inputs = 7 + len(extra)
        ctx.coords_grad = bool(extra[0]) if extra else False
        sfx = _check_inputs(q, k, v, coords, WIDTH, HEIGHT)
        lib = _native.load()
        B, V, H, L, D = q.shape
        P = coords.shape[-2]
        # strided q, k, v are read in place where the kernels can (the reference's forward takes their strides,
        # ops/triton.py:396-405): head dimension contiguous, rows 16-byte aligned, k and v laid out alike
        strides = _native.strides_arg(q, k, v)
        if strides is False:
            q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
            strides = None
        if coords.dtype != torch.float32:
            coords = coords.float()
        out = torch.empty(q.shape, device=q.device, dtype=q.dtype)          # contiguous whatever q's layout
        lse = torch.empty((B, V, H, L), device=q.device, dtype=torch.float32)
        ws_bytes = lib.dsdpa_fwd_workspace_bytes(_DTYPE_CODE[q.dtype], B, V, H, HEIGHT, WIDTH, D, P)
        ws = torch.empty(ws_bytes, device=q.device, dtype=torch.uint8)     # scratch, not saved for backward
        with torch.cuda.device(q.device):
            rc = getattr(lib, "dsdpa_fwd_" + sfx)(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), coords.data_ptr(), out.data_ptr(), lse.data_ptr(),
                ws.data_ptr() if ws_bytes else None,
                B, V, H, HEIGHT, WIDTH, D, P, float(sm_scale), strides, _stream_ptr(q.device))
        _native.check(rc)
        ctx.save_for_backward(q, k, v, coords, out, lse)
        ctx.sm_scale = float(sm_scale)
        ctx.WIDTH, ctx.HEIGHT = WIDTH, HEIGHT
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, coords, out, lse = ctx.saved_tensors
        lib = _native.load()
        sfx = _SUFFIX[q.dtype]
        B, V, H, L, D = q.shape
        P = coords.shape[-2]
        do = do.contiguous()
        if do.dtype != q.dtype:
            do = do.to(q.dtype)
        dq, dk, dv = (torch.empty(q.shape, device=q.device, dtype=q.dtype) for _ in range(3))
        strides = _native.strides_arg(q, k, v)          # (what forward saved: contiguous, or readable in place)
        dcoords = torch.empty_like(coords) if ctx.coords_grad and ctx.needs_input_grad[3] else None
        # torch.use_deterministic_algorithms(True) selects the bitwise reproducible backward
        flags = _native.FLAG_DETERMINISTIC if torch.are_deterministic_algorithms_enabled() else 0
        if flags and dcoords is not None:
            raise RuntimeError("deform_sdpa_triton: the coordinate gradient has no deterministic implementation "
                               "(it sums over heads with float atomics); turn one of the two off")
        if dcoords is not None:
            flags |= _native.FLAG_COORDS_GRAD
        if SINGLE_STREAM:
            flags |= _native.FLAG_SINGLE_STREAM
        ws_bytes = lib.dsdpa_bwd_workspace_bytes(_DTYPE_CODE[q.dtype], B, V, H, ctx.HEIGHT, ctx.WIDTH, D, P, flags)
        ws = torch.empty(ws_bytes, device=q.device, dtype=torch.uint8)
        with torch.cuda.device(q.device):
            rc = getattr(lib, "dsdpa_bwd_" + sfx)(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), coords.data_ptr(), out.data_ptr(), lse.data_ptr(),
                do.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                dcoords.data_ptr() if dcoords is not None else None, ws.data_ptr(),
                B, V, H, ctx.HEIGHT, ctx.WIDTH, D, P, ctx.sm_scale, strides, flags, _stream_ptr(q.device))
        _native.check(rc)
        grads = (dq, dk, dv, dcoords, None, None, None)
        return grads if ctx.n_inputs == 7 else grads + (None,)


deform_sdpa_triton = _fused_deform_sdpa.apply
