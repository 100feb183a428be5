"""ctypes binding of the C oracle (``dsdpa_oracle.c``). Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdsdpa_oracle.so")
_lib = None


def build_oracle(force=False):
    """Compile ``dsdpa_oracle.c`` with gcc (CPU only, about a second)."""
    src = os.path.join(_HERE, "dsdpa_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(
            ["gcc", "-O2", "-fPIC", "-fopenmp", "-std=c11", "-shared", "-o", _LIB_PATH, src, "-lm"]
        )
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build_oracle()
        lib = ctypes.CDLL(_LIB_PATH)
        fp = ctypes.POINTER(ctypes.c_float)
        ip = ctypes.POINTER(ctypes.c_int)
        i, f = ctypes.c_int, ctypes.c_float
        lib.dsdpa_oracle_fwd.argtypes = [fp, fp, fp, fp, fp, fp, i, i, i, i, i, i, i, f]
        lib.dsdpa_oracle_fwd.restype = i
        lib.dsdpa_oracle_bwd.argtypes = [fp, fp, fp, fp, fp, fp, fp, fp, fp, i, i, i, i, i, i, i, f]
        lib.dsdpa_oracle_bwd.restype = i
        lib.dsdpa_oracle_taps.argtypes = [f, f, i, i, ip, fp]
        lib.dsdpa_oracle_taps.restype = None
        _lib = lib
    return _lib


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _ptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _dims(q, coords, W, Himg):
    B, V, H, L, D = q.shape
    assert L == W * Himg, "q.shape[3] must equal WIDTH*HEIGHT"
    P = coords.shape[-2]
    assert coords.shape == (B, V, L, V, P, 2), coords.shape
    return B, V, H, L, D, P


def oracle_fwd(q, k, v, coords, WIDTH, HEIGHT, sm_scale):
    """Forward. Arrays are numpy float32 (B,V,H,L,D) / coords (B,V,L,V,P,2).

    Argument order mirrors the operator: WIDTH before HEIGHT. Returns
    ``(out, lse2)`` with ``lse2`` the base-2 log-sum-exp per query row.
    """
    q, k, v, coords = _f32(q), _f32(k), _f32(v), _f32(coords)
    B, V, H, L, D, P = _dims(q, coords, WIDTH, HEIGHT)
    out = np.empty_like(q)
    lse = np.empty((B, V, H, L), dtype=np.float32)
    rc = _load().dsdpa_oracle_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(coords), _ptr(out), _ptr(lse),
                                  B, V, H, HEIGHT, WIDTH, D, P, float(sm_scale))
    assert rc == 0
    return out, lse


def oracle_bwd(q, k, v, coords, dout, WIDTH, HEIGHT, sm_scale, with_coords=False):
    """Backward. Returns ``(dq, dk, dv)`` as float32 arrays shaped like q; with ``with_coords`` also the
    gradient of the normalised coordinates (shaped like coords, summed over heads)."""
    q, k, v, coords, dout = _f32(q), _f32(k), _f32(v), _f32(coords), _f32(dout)
    B, V, H, L, D, P = _dims(q, coords, WIDTH, HEIGHT)
    dq, dk, dv = np.empty_like(q), np.empty_like(q), np.empty_like(q)
    dc = np.empty_like(coords) if with_coords else None
    rc = _load().dsdpa_oracle_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(coords), _ptr(dout),
                                  _ptr(dq), _ptr(dk), _ptr(dv), _ptr(dc) if with_coords else None,
                                  B, V, H, HEIGHT, WIDTH, D, P, float(sm_scale))
    assert rc == 0
    return (dq, dk, dv, dc) if with_coords else (dq, dk, dv)


def oracle_taps(cx, cy, WIDTH, HEIGHT):
    """The four (pixel, weight) taps of one normalised coordinate; pixel -1 = outside."""
    pix = (ctypes.c_int * 4)()
    w = (ctypes.c_float * 4)()
    _load().dsdpa_oracle_taps(float(cx), float(cy), WIDTH, HEIGHT, pix, w)
    return list(pix), list(w)
