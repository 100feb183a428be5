// C ABI of libdsdpa.so (declared in include/dsdpa.h): argument checks, kernel
// selection and launches. No allocation, no synchronisation, no torch types.
#include "../../include/dsdpa.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "dsdpa_common.h"
#include "dsdpa_gather.h"
#include "dsdpa_tile.h"
#include "dsdpa_cell.h"
#include "dsdpa_plane.h"

using namespace dsdpa;

namespace {

thread_local int g_last_hip_error = 0;
std::atomic<int> g_path{DSDPA_PATH_AUTO};

// Optional kernel timer: while enabled, every main forward/backward kernel
// launch is bracketed by a pair of HIP events on the launch stream. Process-wide
// (a framework may run the backward pass on another thread than the forward).
struct EventPair { hipEvent_t start, stop; };
struct KernelTimer {
    std::atomic<bool> on{false};
    std::mutex mu;
    std::vector<EventPair> pairs[4];   // [0] forward, [1] backward dk/dv, [2] backward dq, [3] cell binning
};
KernelTimer g_timer;

struct ScopedKernelTimer {
    hipStream_t st;
    EventPair ev{nullptr, nullptr};
    int which;
    bool armed = false;
    ScopedKernelTimer(int which_, hipStream_t st_) : st(st_), which(which_)
    {
        if (!g_timer.on.load(std::memory_order_relaxed)) return;
        if (hipEventCreate(&ev.start) != hipSuccess) return;
        if (hipEventCreate(&ev.stop) != hipSuccess) { (void)hipEventDestroy(ev.start); return; }
        armed = hipEventRecord(ev.start, st) == hipSuccess;
    }
    ~ScopedKernelTimer()
    {
        if (!armed) return;
        (void)hipEventRecord(ev.stop, st);
        std::lock_guard<std::mutex> lock(g_timer.mu);
        g_timer.pairs[which].push_back(ev);
    }
};

constexpr int kLdsBytes = 160 * 1024;                                   // LDS per workgroup on gfx950
// query rows per wave in the plane kernels: rows * elements-per-lane = 16 keeps them at 128 VGPRs
template <int DC> struct PlaneRows { static constexpr int value = 16 / DC >= 1 ? 16 / DC : 1; };

// ------------------------------------------------------------------ small kernels
// Zero up to three buffers in one launch (sizes in 16-byte units; unused slots have size 0).
struct ZeroJob { float4 *p[3]; size_t n4[3]; };
__global__ void fill_zero_kernel(ZeroJob job)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 3; ++k)
        for (size_t i = first; i < job.n4[k]; i += stride) job.p[k][i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// fp32 accumulators -> 16-bit storage, 8 elements per thread
template <typename S>
__global__ void cast_kernel(const float *__restrict__ src, void *__restrict__ dst, size_t n8)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n8; i += stride) {
        float v[8];
        const float4 *s4 = reinterpret_cast<const float4 *>(src) + 2 * i;
        float4 a = s4[0], b = s4[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        store_chunk<S, 8>((char *)dst + i * 16, v);
    }
}

int check_launch()
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return DSDPA_ERR_HIP;
    }
    return DSDPA_OK;
}

int make_dims(int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, Dims *dm)
{
    if (B < 1 || V < 1 || H < 1 || Himg < 1 || Wimg < 1 || P < 1) return DSDPA_ERR_BAD_SHAPE;
    if (!(D == 16 || D == 32 || D == 64 || D == 128 || D == 256)) return DSDPA_ERR_HEAD_DIM;
    const long long L = (long long)Himg * Wimg;
    const long long slab = (long long)V * H * L * D;           // one batch item of k/v
    const long long rows = (long long)B * V * H * L;
    const long long N = (long long)V * P;
    if (L > (1ll << 24) || slab > (1ll << 30) || rows > 0x7fffffffll - 1024 || N > (1ll << 24))
        return DSDPA_ERR_TOO_LARGE;
    dm->B = B; dm->V = V; dm->H = H; dm->Himg = Himg; dm->Wimg = Wimg;
    dm->L = (int)L; dm->P = P; dm->N = (int)N; dm->rows = (int)rows; dm->sm_scale = sm_scale;
    return DSDPA_OK;
}

// lanes per sample are D/DC; DC is chosen so that a lane moves 16 bytes per tap
// (32 or 64 for the widest heads) and a sample never spans more than 16 lanes.
template <typename S, int D> struct Chunk {
    static constexpr int kMin = 16 / S::kBytes;
    static constexpr int value = (D / kMin > 16) ? D / 16 : kMin;
};

template <typename S, int D>
int launch_fwd_gather(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
                      const Dims &dm, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const int blocks = (dm.rows + kGatherWaves - 1) / kGatherWaves;
    ScopedKernelTimer timer(0, st);
    hipLaunchKernelGGL((fwd_gather_kernel<S, D, DC>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                       q, k, v, coords, out, lse, dm);
    return check_launch();
}

template <typename S, int D>
int launch_bwd_gather(const void *q, const void *k, const void *v, const float *coords, const void *out,
                      const float *lse, const void *dout, void *dq, float *dk_acc, float *dv_acc,
                      const Dims &dm, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const int blocks = (dm.rows + kGatherWaves - 1) / kGatherWaves;
    ScopedKernelTimer timer(1, st);
    hipLaunchKernelGGL((bwd_gather_kernel<S, D, DC>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                       q, k, v, coords, out, lse, dout, dq, dk_acc, dv_acc, dm);
    return check_launch();
}

template <typename S, int D>
int launch_bwd_dq_gather(const void *q, const void *k, const void *v, const float *coords, const void *out,
                         const float *lse, const void *dout, void *dq, float *delta, const Dims &dm,
                         hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const int blocks = (dm.rows + kGatherWaves - 1) / kGatherWaves;
    ScopedKernelTimer timer(2, st);
    hipLaunchKernelGGL((bwd_dq_gather_kernel<S, D, DC>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                       q, k, v, coords, out, lse, dout, dq, delta, dm);
    return check_launch();
}

constexpr int kTileDescBytes = kTileWaves * kWave * (16 + 16 + 4);      // per-wave tap descriptors

// Tile geometry for the dk/dv kernel: as few tiles per plane as the LDS budget allows
// (every tile costs one more pass over the plane's coordinates and one halo ring).
TileGeom make_tile_geom(const Dims &dm, int D)
{
    const int maxpx = (kLdsBytes - kTileDescBytes) / (2 * (int)sizeof(double) * D);   // dK + dV, fp64
    const int Hh = dm.Himg, Ww = dm.Wimg;
    auto ceil_div = [](int a, int b) { return (a + b - 1) / b; };
    // option A: full-width row bands
    int a_nty = 1 << 30, a_th = 0;
    if (Ww * 2 <= maxpx || Hh * Ww <= maxpx) {
        const int rows = maxpx / Ww;                       // rows of pixels that fit
        const int th_max = rows >= Hh ? Hh : rows - 1;     // one halo row unless the whole image fits
        a_nty = ceil_div(Hh, th_max);
        a_th = ceil_div(Hh, a_nty);
    }
    // option B: square-ish 2-D tiles
    int side = 2;
    while ((side + 1) * (side + 1) <= maxpx) ++side;
    const int cells = side - 1 > 0 ? side - 1 : 1;
    const int b_nty = ceil_div(Hh, cells), b_ntx = ceil_div(Ww, cells);
    TileGeom tg;
    if (a_nty <= b_nty * b_ntx) {
        tg.th = a_th; tg.tw = Ww; tg.nty = a_nty; tg.ntx = 1;
    } else {
        tg.th = ceil_div(Hh, b_nty); tg.tw = ceil_div(Ww, b_ntx); tg.nty = b_nty; tg.ntx = b_ntx;
    }
    tg.lh = tg.nty == 1 ? Hh : tg.th + 1;
    tg.lw = tg.ntx == 1 ? Ww : tg.tw + 1;
    const long long groups = (long long)dm.B * dm.H * dm.V * tg.nty * tg.ntx;
    long long qsplit = (1024 + groups - 1) / groups;
    const long long max_split = ((long long)dm.V * dm.L + 63) / 64;    // keep >= 64 query rows per workgroup
    if (qsplit > max_split) qsplit = max_split;
    if (qsplit < 1) qsplit = 1;
    tg.qsplit = (int)qsplit;
    return tg;
}

template <typename S, int D>
int launch_bwd_dkdv_tile(const void *q, const void *k, const void *v, const float *coords, const float *lse,
                         const float *delta, const void *dout, float *dk_acc, float *dv_acc, const Dims &dm,
                         hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const TileGeom tg = make_tile_geom(dm, D);
    const size_t smem = (size_t)2 * sizeof(double) * tg.lh * tg.lw * D + kTileDescBytes;
    if (smem > (size_t)kLdsBytes) return DSDPA_ERR_TOO_LARGE;
    const long long blocks = (long long)dm.B * dm.H * dm.V * tg.nty * tg.ntx * tg.qsplit;
    if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
    auto kern = bwd_dkdv_tile_kernel<S, D, DC>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) { g_last_hip_error = (int)e; return DSDPA_ERR_HIP; }
    ScopedKernelTimer timer(1, st);
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kTileWaves * kWave), smem, st,
                       q, k, v, coords, lse, delta, dout, dk_acc, dv_acc, dm, tg);
    return check_launch();
}

// The plane kernels need one K and one V plane of a (b, s2, h) in LDS next to the descriptors.
template <typename S>
bool plane_fits(const Dims &dm, int D)
{
    return (size_t)(dm.L + 2) * 2 * D * S::kBytes + kPlaneDescBytes <= (size_t)kLdsBytes;
}

template <typename S, int D>
int launch_fwd_plane(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
                     const Dims &dm, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const size_t smem = (size_t)plane_lds_bytes<S, D>(dm.L) + kPlaneDescBytes;
    constexpr int QW = PlaneRows<DC>::value;
    const int rows_per_block = kPlaneWaves * QW;
    const long long blocks = (long long)dm.B * dm.H * ((dm.V * dm.L + rows_per_block - 1) / rows_per_block);
    constexpr bool kCanPair = QW % 2 == 0;
    // (a P == 32 compile-time instantiation was tried: the unrolled chunk spills 432 bytes per lane)
    auto kern = (kCanPair && dm.P <= 32) ? fwd_plane_kernel<S, D, DC, QW, kCanPair, 0>
                                         : fwd_plane_kernel<S, D, DC, QW, false, 0>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) { g_last_hip_error = (int)e; return DSDPA_ERR_HIP; }
    ScopedKernelTimer timer(0, st);
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kPlaneWaves * kWave), smem, st,
                       q, k, v, coords, out, lse, dm);
    return check_launch();
}

template <typename S, int D>
int launch_bwd_dq_plane(const void *q, const void *k, const void *v, const float *coords, const void *out,
                        const float *lse, const void *dout, void *dq, float *delta, const Dims &dm,
                        hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const size_t smem = (size_t)plane_lds_bytes<S, D>(dm.L) + kPlaneDescBytes;
    constexpr int QW = PlaneRows<DC>::value;
    const int rows_per_block = kPlaneWaves * QW;
    const long long blocks = (long long)dm.B * dm.H * ((dm.V * dm.L + rows_per_block - 1) / rows_per_block);
    constexpr bool kCanPair = QW % 2 == 0;
    auto kern = (kCanPair && dm.P <= 32) ? bwd_dq_plane_kernel<S, D, DC, QW, kCanPair, 0>
                                         : bwd_dq_plane_kernel<S, D, DC, QW, false, 0>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) { g_last_hip_error = (int)e; return DSDPA_ERR_HIP; }
    ScopedKernelTimer timer(2, st);
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kPlaneWaves * kWave), smem, st,
                       q, k, v, coords, out, lse, dout, dq, delta, dm);
    return check_launch();
}

template <typename S>
int fwd_impl(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
             int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    if (!q || !k || !v || !coords || !out || !lse) return DSDPA_ERR_NULL_POINTER;
    Dims dm;
    int rc = make_dims(B, V, H, Himg, Wimg, D, P, sm_scale, &dm);
    if (rc != DSDPA_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    const bool staged = g_path.load() != DSDPA_PATH_GATHER && plane_fits<S>(dm, D);
#define DSDPA_FWD_CASE(DD)                                                                        \
    case DD:                                                                                      \
        return staged ? launch_fwd_plane<S, DD>(q, k, v, coords, out, lse, dm, st)                \
                      : launch_fwd_gather<S, DD>(q, k, v, coords, out, lse, dm, st);
    switch (D) {
        DSDPA_FWD_CASE(16)
        DSDPA_FWD_CASE(32)
        DSDPA_FWD_CASE(64)
        DSDPA_FWD_CASE(128)
        DSDPA_FWD_CASE(256)
    }
#undef DSDPA_FWD_CASE
    return DSDPA_ERR_HEAD_DIM;
}

// element counts are multiples of 4 (D >= 16; workspace segments are 256-byte multiples)
int zero_fill(float *a, size_t na, float *b, size_t nb, float *c, size_t nc, hipStream_t st)
{
    ZeroJob job{{(float4 *)a, (float4 *)b, (float4 *)c}, {na / 4, nb / 4, nc / 4}};
    size_t big = job.n4[0] > job.n4[1] ? job.n4[0] : job.n4[1];
    if (job.n4[2] > big) big = job.n4[2];
    const int threads = 256;
    size_t blocks = (big + threads - 1) / threads;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(threads), 0, st, job);
    return check_launch();
}

// Backward workspace, every segment rounded up to 256 bytes:
//   delta    rows floats                     dout.out per query row
//   counters B*V*NC u32                      per (batch, key view) cell counts, then fill cursors
//   start    B*V*(NC+1) u32                  exclusive scan of the counts
//   sorted   B*V*(V*L*P) u32                 sample ids ordered by cell
//   acc      2*n floats                      fp32 dk/dv accumulators (16-bit storage only)
// with NC = (Himg+1)*(Wimg+1) cells.
size_t round256(size_t b) { return (b + 255) / 256 * 256; }
struct WorkspaceLayout {
    size_t delta, counters, start, sorted, acc, total;
    size_t counters_bytes;
    int NC;
};
WorkspaceLayout workspace_layout(size_t B, size_t V, size_t H, size_t Himg, size_t Wimg, size_t D, size_t P,
                                 bool storage16)
{
    WorkspaceLayout w;
    const size_t rows = B * V * H * Himg * Wimg;
    w.NC = (int)((Himg + 1) * (Wimg + 1));
    size_t off = 0;
    w.delta = off; off += round256(rows * 4);
    w.counters = off; w.counters_bytes = round256(B * V * (size_t)w.NC * 4); off += w.counters_bytes;
    w.start = off; off += round256(B * V * ((size_t)w.NC + 1) * 4);
    w.sorted = off; off += round256(B * V * (V * Himg * Wimg * P) * 4);
    w.acc = off; if (storage16) off += round256(2 * rows * D * 4);
    w.total = off;
    return w;
}

// elements per lane in the cell kernel: 4 up to D = 128 (32 lanes per sample at most), 8 beyond.
// With 4 the kernel holds 64 tap/accumulator registers and runs 4 waves per SIMD; 8 elements per
// lane at D = 32/64 were measured slower (211 VGPRs, 2 waves per SIMD, latency-bound).
template <typename S, int D> struct CellChunk {
    static constexpr int value = D <= 128 ? 4 : 8;
};

int launch_binning(const float *coords, const Dims &dm, const WorkspaceLayout &wl, char *ws, hipStream_t st)
{
    unsigned *counters = (unsigned *)(ws + wl.counters);
    unsigned *start = (unsigned *)(ws + wl.start);
    unsigned *sorted = (unsigned *)(ws + wl.sorted);
    const size_t hist_bytes = (size_t)dm.V * wl.NC * sizeof(unsigned);
    ScopedKernelTimer timer(3, st);
    if (2 * hist_bytes <= (size_t)kLdsBytes - 1024) {
        // LDS-aggregated passes: a workgroup per run of about 8k samples of one (b, s1)
        int lchunk = 8192 / dm.N;
        if (lchunk < 1) lchunk = 1;
        if (lchunk > dm.L) lchunk = dm.L;
        const int nlc = (dm.L + lchunk - 1) / lchunk;
        lchunk = (dm.L + nlc - 1) / nlc;
        const long long blocks = (long long)dm.B * dm.V * nlc;
        if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
        auto k0 = bin_samples_lds_kernel<0>;
        auto k1 = bin_samples_lds_kernel<1>;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k0),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)hist_bytes);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k1),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * hist_bytes));
        if (e != hipSuccess) { g_last_hip_error = (int)e; return DSDPA_ERR_HIP; }
        hipLaunchKernelGGL(k0, dim3((unsigned)blocks), dim3(kBinLdsThreads), hist_bytes, st,
                           coords, dm, wl.NC, lchunk, nlc, counters, sorted);
        hipLaunchKernelGGL(bin_scan_kernel, dim3((unsigned)(dm.B * dm.V)), dim3(1024), 0, st, counters, start, wl.NC);
        hipLaunchKernelGGL(k1, dim3((unsigned)blocks), dim3(kBinLdsThreads), 2 * hist_bytes, st,
                           coords, dm, wl.NC, lchunk, nlc, counters, sorted);
        return check_launch();
    }
    const long long total = (long long)dm.B * dm.V * dm.L * dm.N;
    const long long blocks = (total + kBinThreads - 1) / kBinThreads;
    if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(bin_samples_kernel<0>, dim3((unsigned)blocks), dim3(kBinThreads), 0, st,
                       coords, dm, wl.NC, counters, sorted);
    hipLaunchKernelGGL(bin_scan_kernel, dim3((unsigned)(dm.B * dm.V)), dim3(1024), 0, st, counters, start, wl.NC);
    hipLaunchKernelGGL(bin_samples_kernel<1>, dim3((unsigned)blocks), dim3(kBinThreads), 0, st,
                       coords, dm, wl.NC, counters, sorted);
    return check_launch();
}

template <typename S, int D>
int launch_bwd_dkdv_cell(const void *q, const void *k, const void *v, const float *coords, const float *lse,
                         const float *delta, const void *dout, const unsigned *start, const unsigned *sorted,
                         float *dk_acc, float *dv_acc, const Dims &dm, int NC, hipStream_t st)
{
    constexpr int DC = CellChunk<S, D>::value;
    const long long nwork = (long long)dm.B * dm.H * dm.V * NC;
    const long long blocks = (nwork + kCellWaves - 1) / kCellWaves;
    if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
    ScopedKernelTimer timer(1, st);
    hipLaunchKernelGGL((bwd_dkdv_cell_kernel<S, D, DC>), dim3((unsigned)blocks), dim3(kCellWaves * kWave), 0, st,
                       q, k, v, coords, lse, delta, dout, start, sorted, dk_acc, dv_acc, dm, NC);
    return check_launch();
}

template <typename S>
int bwd_impl(const void *q, const void *k, const void *v, const float *coords, const void *out,
             const float *lse, const void *dout, void *dq, void *dk, void *dv, void *workspace,
             int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    if (!q || !k || !v || !coords || !out || !lse || !dout || !dq || !dk || !dv || !workspace)
        return DSDPA_ERR_NULL_POINTER;
    Dims dm;
    int rc = make_dims(B, V, H, Himg, Wimg, D, P, sm_scale, &dm);
    if (rc != DSDPA_OK) return rc;
    if ((long long)dm.L * dm.N > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;   // sample ids are 32-bit
    hipStream_t st = (hipStream_t)stream;
    const size_t n = (size_t)dm.rows * D;
    const WorkspaceLayout wl = workspace_layout(B, V, H, Himg, Wimg, D, P, S::kBytes != 4);
    char *ws = (char *)workspace;
    float *delta = (float *)(ws + wl.delta);
    const int path = g_path.load();
    const bool fused_atomics = path == DSDPA_PATH_GATHER;
    const bool cell_binned = path == DSDPA_PATH_AUTO;
    const bool staged = plane_fits<S>(dm, D);
    const unsigned *start = (const unsigned *)(ws + wl.start);
    const unsigned *sorted = (const unsigned *)(ws + wl.sorted);
    // one launch zeroes the dk/dv accumulators and, for the cell-binned path, the cell counters
    float *dk_acc = S::kBytes == 4 ? (float *)dk : (float *)(ws + wl.acc);
    float *dv_acc = S::kBytes == 4 ? (float *)dv : dk_acc + n;
    rc = zero_fill(dk_acc, n, dv_acc, n, (float *)(ws + wl.counters), cell_binned ? wl.counters_bytes / 4 : 0, st);
    if (rc != DSDPA_OK) return rc;
    if (cell_binned && (rc = launch_binning(coords, dm, wl, ws, st)) != DSDPA_OK) return rc;
#define DSDPA_BWD_CASE(DD)                                                                                      \
    case DD:                                                                                                    \
        if (fused_atomics) {                                                                                    \
            rc = launch_bwd_gather<S, DD>(q, k, v, coords, out, lse, dout, dq, dk_acc, dv_acc, dm, st);         \
        } else {                                                                                                \
            rc = staged ? launch_bwd_dq_plane<S, DD>(q, k, v, coords, out, lse, dout, dq, delta, dm, st)        \
                        : launch_bwd_dq_gather<S, DD>(q, k, v, coords, out, lse, dout, dq, delta, dm, st);      \
            if (rc == DSDPA_OK && cell_binned)                                                                  \
                rc = launch_bwd_dkdv_cell<S, DD>(q, k, v, coords, lse, delta, dout, start, sorted, dk_acc,      \
                                                 dv_acc, dm, wl.NC, st);                                        \
            else if (rc == DSDPA_OK)                                                                            \
                rc = launch_bwd_dkdv_tile<S, DD>(q, k, v, coords, lse, delta, dout, dk_acc, dv_acc, dm, st);    \
        }                                                                                                       \
        break;
    switch (D) {
        DSDPA_BWD_CASE(16)
        DSDPA_BWD_CASE(32)
        DSDPA_BWD_CASE(64)
        DSDPA_BWD_CASE(128)
        DSDPA_BWD_CASE(256)
    default: return DSDPA_ERR_HEAD_DIM;
    }
#undef DSDPA_BWD_CASE
    if (rc != DSDPA_OK) return rc;
    if (S::kBytes != 4) {
        const size_t n8 = n / 8;
        const int threads = 256;
        size_t blocks = (n8 + threads - 1) / threads;
        if (blocks > 256 * 16) blocks = 256 * 16;
        hipLaunchKernelGGL((cast_kernel<S>), dim3((unsigned)blocks), dim3(threads), 0, st, dk_acc, dk, n8);
        hipLaunchKernelGGL((cast_kernel<S>), dim3((unsigned)blocks), dim3(threads), 0, st, dv_acc, dv, n8);
        rc = check_launch();
    }
    return rc;
}

}  // namespace

extern "C" {

int dsdpa_fwd_f32(const float *q, const float *k, const float *v, const float *coords, float *out, float *lse,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    return fwd_impl<F32>(q, k, v, coords, out, lse, B, V, H, Himg, Wimg, D, P, sm_scale, stream);
}

int dsdpa_fwd_bf16(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
                   int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    return fwd_impl<BF16>(q, k, v, coords, out, lse, B, V, H, Himg, Wimg, D, P, sm_scale, stream);
}

int dsdpa_fwd_f16(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    return fwd_impl<F16>(q, k, v, coords, out, lse, B, V, H, Himg, Wimg, D, P, sm_scale, stream);
}

int dsdpa_bwd_f32(const float *q, const float *k, const float *v, const float *coords, const float *out,
                  const float *lse, const float *dout, float *dq, float *dk, float *dv, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    return bwd_impl<F32>(q, k, v, coords, out, lse, dout, dq, dk, dv, workspace, B, V, H, Himg, Wimg, D, P,
                         sm_scale, stream);
}

int dsdpa_bwd_bf16(const void *q, const void *k, const void *v, const float *coords, const void *out,
                   const float *lse, const void *dout, void *dq, void *dk, void *dv, void *workspace,
                   int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    return bwd_impl<BF16>(q, k, v, coords, out, lse, dout, dq, dk, dv, workspace, B, V, H, Himg, Wimg, D, P,
                          sm_scale, stream);
}

int dsdpa_bwd_f16(const void *q, const void *k, const void *v, const float *coords, const void *out,
                  const float *lse, const void *dout, void *dq, void *dk, void *dv, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, void *stream)
{
    return bwd_impl<F16>(q, k, v, coords, out, lse, dout, dq, dk, dv, workspace, B, V, H, Himg, Wimg, D, P,
                         sm_scale, stream);
}

size_t dsdpa_bwd_workspace_bytes(int dtype, int B, int V, int H, int Himg, int Wimg, int D, int P)
{
    if (dtype != DSDPA_F32 && dtype != DSDPA_BF16 && dtype != DSDPA_F16) return 0;
    if (B < 1 || V < 1 || H < 1 || Himg < 1 || Wimg < 1 || D < 1 || P < 1) return 0;
    return workspace_layout(B, V, H, Himg, Wimg, D, P, dtype != DSDPA_F32).total;
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
    case DSDPA_ERR_DTYPE: return "unknown dtype code";
    }
    return "unknown error code";
}

int dsdpa_last_hip_error(void) { return g_last_hip_error; }

int dsdpa_version(void) { return 100; }

int dsdpa_timer_enable(int on)
{
    return g_timer.on.exchange(on != 0) ? 1 : 0;
}

int dsdpa_timer_collect(int which, double *total_ms, int *launches)
{
    if (which < 0 || which > 3 || !total_ms || !launches) return DSDPA_ERR_NULL_POINTER;
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
