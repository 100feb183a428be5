"""ctypes binding of libdsdpa.so (the C ABI declared in ``include/dsdpa.h``).

The library is loaded from ``lib/libdsdpa.so`` next to this package. There is
no fallback: if the library is missing, or a call returns an error code, an
exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libdsdpa.so")

# every symbol include/dsdpa.h declares
SYMBOLS = (
    "dsdpa_fwd_f32", "dsdpa_fwd_bf16", "dsdpa_fwd_f16",
    "dsdpa_bwd_f32", "dsdpa_bwd_bf16", "dsdpa_bwd_f16", "dsdpa_fwd_noalloc",
    "dsdpa_fwd_workspace_bytes", "dsdpa_bwd_workspace_bytes", "dsdpa_error_string", "dsdpa_last_hip_error",
    "dsdpa_version", "dsdpa_set_path", "dsdpa_timer_enable", "dsdpa_timer_collect",
)

DSDPA_F32, DSDPA_BF16, DSDPA_F16 = 0, 1, 2
PATH_AUTO, PATH_GATHER, PATH_LDS = 0, 1, 2
FLAG_DETERMINISTIC = 1
FLAG_COORDS_GRAD = 2
FLAG_SINGLE_STREAM = 4
ERR_SCRATCH = 8
ERR_BAD_STRIDES = 9
NOALLOC_SCRATCH_BYTES = 32 << 20

_lib = None


class DsdpaError(RuntimeError):
    """A libdsdpa entry point returned a non-zero code."""


def load():
    """Load libdsdpa.so once and declare the signatures. Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python build.py` (hipcc, gfx950). "
            "There is no fallback path for the fused operator.")
    lib = ctypes.CDLL(LIB_PATH)
    vp, i, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    ll = ctypes.POINTER(ctypes.c_longlong)
    dims = [i, i, i, i, i, i, i, f, ll, vp]        # B V H Himg Wimg D P sm_scale strides stream
    u = ctypes.c_uint
    for sfx in ("f32", "bf16", "f16"):
        fwd = getattr(lib, "dsdpa_fwd_" + sfx)
        fwd.argtypes = [vp] * 7 + dims          # q k v coords out lse workspace
        fwd.restype = i
        bwd = getattr(lib, "dsdpa_bwd_" + sfx)
        bwd.argtypes = [vp] * 12 + dims[:-1] + [u, vp]   # q k v coords out lse dout dq dk dv dcoords workspace, dims (with strides), flags, stream
        bwd.restype = i
    lib.dsdpa_fwd_noalloc.argtypes = [i] + [vp] * 6 + dims      # dtype, q k v coords out lse, dims
    lib.dsdpa_fwd_noalloc.restype = i
    lib.dsdpa_fwd_workspace_bytes.argtypes = [i] * 8
    lib.dsdpa_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.dsdpa_bwd_workspace_bytes.argtypes = [i] * 8 + [u]
    lib.dsdpa_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.dsdpa_error_string.argtypes = [i]
    lib.dsdpa_error_string.restype = ctypes.c_char_p
    lib.dsdpa_last_hip_error.argtypes = []
    lib.dsdpa_last_hip_error.restype = i
    lib.dsdpa_version.argtypes = []
    lib.dsdpa_version.restype = i
    lib.dsdpa_set_path.argtypes = [i]
    lib.dsdpa_set_path.restype = i
    lib.dsdpa_timer_enable.argtypes = [i]
    lib.dsdpa_timer_enable.restype = i
    lib.dsdpa_timer_collect.argtypes = [i, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(i)]
    lib.dsdpa_timer_collect.restype = i
    _lib = lib
    return lib


def strides_arg(q, k, v):
    """The `strides` argument of the entry points for q, k, v given as (B, V, H, L, D) tensors: None when all three
    are contiguous, else a ctypes array of q's and k/v's element strides over (batch, view, head, pixel), or
    False when the kernels cannot read the tensors in place (the head dimension is not contiguous, k and v are
    laid out differently, a row start is not 16-byte aligned, or the views and pixels of one (batch, head) lie
    more than 2^30 elements apart): the caller then copies."""
    if q.is_contiguous() and k.is_contiguous() and v.is_contiguous():
        return None
    align = 16 // q.element_size()
    V, L, D = q.shape[1], q.shape[3], q.shape[4]
    for t in (q, k, v):
        st = t.stride()
        if st[4] != 1 or t.data_ptr() % 16 or any(x % align or x < 0 for x in st[:4]) or st[3] < t.shape[4]:
            return False
        # the kernels address a pixel of one (batch, head) as view*sv + pixel*sl in 32 bits: a layout that reaches
        # farther (the library would refuse it with DSDPA_ERR_TOO_LARGE) is copied as well
        if (V - 1) * st[1] + (L - 1) * st[3] + D > (1 << 30) or st[1] > (1 << 30):
            return False
    if k.stride() != v.stride():
        return False
    return (ctypes.c_longlong * 8)(*q.stride()[:4], *k.stride()[:4])


def check(code):
    if code != 0:
        lib = load()
        msg = lib.dsdpa_error_string(code).decode()
        raise DsdpaError(f"libdsdpa error {code}: {msg} (hip error {lib.dsdpa_last_hip_error()})")


def set_path(path):
    """Force a kernel path (PATH_AUTO / PATH_GATHER / PATH_LDS); returns the previous one."""
    prev = load().dsdpa_set_path(int(path))
    if prev < 0:
        raise ValueError(f"unknown kernel path {path}")
    return prev


def timer_enable(on):
    """Attach HIP events to every main fwd/bwd kernel launch (process-wide); returns the previous state."""
    return load().dsdpa_timer_enable(1 if on else 0)


def timer_collect(which):
    """(total kernel ms, launches) since the last collect; which: 0 forward, 1 backward dk/dv, 2 backward dq,
    3 cell binning (its launches together), 4 tap table fill."""
    ms, n = ctypes.c_double(0.0), ctypes.c_int(0)
    check(load().dsdpa_timer_collect(int(which), ctypes.byref(ms), ctypes.byref(n)))
    return ms.value, n.value
