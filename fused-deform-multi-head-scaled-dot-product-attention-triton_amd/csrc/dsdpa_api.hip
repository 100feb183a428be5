// C ABI of libdsdpa.so (declared in include/dsdpa.h): the extern "C" entry points and the shared
// host-side state. The kernels and their launchers are compiled per storage type (dsdpa_f32.hip,
// dsdpa_bf16.hip, dsdpa_f16.hip); the list sort of the deterministic backward lives in dsdpa_sort.hip.
#include "dsdpa_host.h"
#include "dsdpa_common.h"

using namespace dsdpa;

namespace dsdpa {
thread_local int g_last_hip_error = 0;
std::atomic<int> g_path{DSDPA_PATH_AUTO};
KernelTimer g_timer;
}  // namespace dsdpa

// Built-in scratch of dsdpa_fwd_noalloc: the forward's workspace (the per-coordinate tap table) for callers
// that cannot allocate. Every GPU the library runs on holds its own copy of the array, at its own address,
// until the process ends. In host code the array's name is only a handle for hipGetSymbolAddress: the
// device address is looked up once per device (with that device current) and kept in g_scratch_ptr; host
// code passes that pointer, never the array's name, to kernels.
static __device__ __align__(256) unsigned char scratch[DSDPA_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device; null (and the HIP error kept) if it cannot be had.
void *scratch_on_current_device()
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        g_last_hip_error = (int)(e != hipSuccess ? e : hipErrorInvalidDevice);
        return nullptr;
    }
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p) return p;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
        g_last_hip_error = (int)(e != hipSuccess ? e : hipErrorInvalidSymbol);
        return nullptr;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);      // (two threads racing here store the same address)
    return p;
}
}  // namespace

extern "C" {

int dsdpa_fwd_f32(const float *q, const float *k, const float *v, const float *coords, float *out, float *lse, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides, void *stream)
{
    return fwd_impl<F32>(q, k, v, coords, out, lse, workspace, B, V, H, Himg, Wimg, D, P, sm_scale, strides, stream, true);
}

int dsdpa_fwd_bf16(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides, void *stream)
{
    return fwd_impl<BF16>(q, k, v, coords, out, lse, workspace, B, V, H, Himg, Wimg, D, P, sm_scale, strides, stream, true);
}

int dsdpa_fwd_f16(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides, void *stream)
{
    return fwd_impl<F16>(q, k, v, coords, out, lse, workspace, B, V, H, Himg, Wimg, D, P, sm_scale, strides, stream, true);
}

int dsdpa_bwd_f32(const float *q, const float *k, const float *v, const float *coords, const float *out,
                  const float *lse, const float *dout, float *dq, float *dk, float *dv, float *dcoords, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides, unsigned flags, void *stream)
{
    return bwd_impl<F32>(q, k, v, coords, out, lse, dout, dq, dk, dv, dcoords, workspace, B, V, H, Himg, Wimg, D, P,
                         sm_scale, strides, flags, stream);
}

int dsdpa_bwd_bf16(const void *q, const void *k, const void *v, const float *coords, const void *out,
                   const float *lse, const void *dout, void *dq, void *dk, void *dv, float *dcoords, void *workspace,
                   int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides, unsigned flags, void *stream)
{
    return bwd_impl<BF16>(q, k, v, coords, out, lse, dout, dq, dk, dv, dcoords, workspace, B, V, H, Himg, Wimg, D, P,
                          sm_scale, strides, flags, stream);
}

int dsdpa_bwd_f16(const void *q, const void *k, const void *v, const float *coords, const void *out,
                  const float *lse, const void *dout, void *dq, void *dk, void *dv, float *dcoords, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides, unsigned flags, void *stream)
{
    return bwd_impl<F16>(q, k, v, coords, out, lse, dout, dq, dk, dv, dcoords, workspace, B, V, H, Himg, Wimg, D, P,
                         sm_scale, strides, flags, stream);
}

int dsdpa_fwd_noalloc(int dtype, const void *q, const void *k, const void *v, const float *coords, void *out,
                      float *lse, int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale,
                      const long long *strides, void *stream)
{
    if (dtype != DSDPA_F32 && dtype != DSDPA_BF16 && dtype != DSDPA_F16) return DSDPA_ERR_DTYPE;
    if (B < 1 || V < 1 || H < 1 || Himg < 1 || Wimg < 1 || P < 1) return DSDPA_ERR_BAD_SHAPE;
    if (!(D == 16 || D == 32 || D == 64 || D == 128 || D == 256)) return DSDPA_ERR_HEAD_DIM;
    const size_t esize = dtype != DSDPA_F32 ? 2 : 4;
    size_t need = desc_layout(B, V, Himg, Wimg, D, P, esize).bytes;
    if (need > (size_t)DSDPA_NOALLOC_SCRATCH_BYTES) return DSDPA_ERR_SCRATCH;
    // (the dense-box forward's transposed V is an optional speed-up: taken when it fits, never a reason to refuse)
    const size_t dense_need = dense_layout(B, V, H, Himg, Wimg, D, P, esize).bytes;
    const bool dense_ok = dense_need != 0 && dense_need <= (size_t)DSDPA_NOALLOC_SCRATCH_BYTES;
    if (dense_ok) need = dense_need;
    void *ws = nullptr;
    if (need) {
        ws = scratch_on_current_device();
        if (!ws) return DSDPA_ERR_HIP;
    }
    switch (dtype) {
    case DSDPA_F32: return fwd_impl<F32>(q, k, v, coords, out, lse, ws, B, V, H, Himg, Wimg, D, P, sm_scale, strides, stream, dense_ok);
    case DSDPA_BF16: return fwd_impl<BF16>(q, k, v, coords, out, lse, ws, B, V, H, Himg, Wimg, D, P, sm_scale, strides, stream, dense_ok);
    default: return fwd_impl<F16>(q, k, v, coords, out, lse, ws, B, V, H, Himg, Wimg, D, P, sm_scale, strides, stream, dense_ok);
    }
}

size_t dsdpa_fwd_workspace_bytes(int dtype, int B, int V, int H, int Himg, int Wimg, int D, int P)
{
    if (dtype != DSDPA_F32 && dtype != DSDPA_BF16 && dtype != DSDPA_F16) return 0;
    if (B < 1 || V < 1 || H < 1 || Himg < 1 || Wimg < 1 || D < 1 || P < 1) return 0;
    const size_t esize = dtype != DSDPA_F32 ? 2 : 4;
    return desc_layout(B, V, Himg, Wimg, D, P, esize).bytes + dense_layout(B, V, H, Himg, Wimg, D, P, esize).bytes;
}

size_t dsdpa_bwd_workspace_bytes(int dtype, int B, int V, int H, int Himg, int Wimg, int D, int P, unsigned flags)
{
    if (dtype != DSDPA_F32 && dtype != DSDPA_BF16 && dtype != DSDPA_F16) return 0;
    if (B < 1 || V < 1 || H < 1 || Himg < 1 || Wimg < 1 || D < 1 || P < 1) return 0;
    return workspace_layout(B, V, H, Himg, Wimg, D, P, dtype != DSDPA_F32,
                            (flags & DSDPA_FLAG_DETERMINISTIC) != 0, (flags & DSDPA_FLAG_COORDS_GRAD) != 0).total;
}

const char *dsdpa_error_string(int code)
{
    switch (code) {
    case DSDPA_OK: return "ok";
    case DSDPA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case DSDPA_ERR_BAD_SHAPE: return "a dimension is smaller than 1";
    case DSDPA_ERR_HEAD_DIM: return "head dim must be one of 16, 32, 64, 128, 256";
    case DSDPA_ERR_TOO_LARGE: return "shape exceeds the 32-bit indexing limits of the kernels";
    case DSDPA_ERR_HIP: return "a HIP launch failed (see dsdpa_last_hip_error)";
    case DSDPA_ERR_UNSUPPORTED: return "unknown flag, or a combination of options that is not supported";
    case DSDPA_ERR_DTYPE: return "unknown dtype code";
    case DSDPA_ERR_BAD_STRIDES: return "strides: the head dimension must be contiguous and every row 16-byte aligned";
    case DSDPA_ERR_SCRATCH: return "the shape needs more scratch memory than the library's built-in buffer holds";
    }
    return "unknown error code";
}

int dsdpa_last_hip_error(void) { return g_last_hip_error; }

int dsdpa_version(void) { return 200; }

int dsdpa_timer_enable(int on)
{
    return g_timer.on.exchange(on != 0) ? 1 : 0;
}

int dsdpa_timer_collect(int which, double *total_ms, int *launches)
{
    if (which < 0 || which > 4 || !total_ms || !launches) return DSDPA_ERR_NULL_POINTER;
    double sum = 0.0;
    int n = 0, rc = DSDPA_OK;
    std::vector<EventPair> taken;
    {
        std::lock_guard<std::mutex> lock(g_timer.mu);
        taken.swap(g_timer.pairs[which]);
    }
    for (EventPair &ev : taken) {
        float ms = 0.f;
        hipError_t e = hipEventSynchronize(ev.stop);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, ev.start, ev.stop);
        if (e == hipSuccess) { sum += ms; ++n; } else { g_last_hip_error = (int)e; rc = DSDPA_ERR_HIP; }
        (void)hipEventDestroy(ev.start);
        (void)hipEventDestroy(ev.stop);
    }
    *total_ms = sum;
    *launches = n;
    return rc;
}

int dsdpa_set_path(int path)
{
    if (path != DSDPA_PATH_AUTO && path != DSDPA_PATH_GATHER && path != DSDPA_PATH_LDS) return -1;
    return g_path.exchange(path);
}

}  // extern "C"
