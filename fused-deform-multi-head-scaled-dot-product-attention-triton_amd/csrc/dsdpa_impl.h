// Launchers and per-storage-type entry points (argument checks, kernel selection, launches).
// Included by one translation unit per storage type; no allocation, no synchronisation, no torch types.
#pragma once
#include "dsdpa_host.h"
#include "dsdpa_common.h"
#include "dsdpa_gather.h"
#include "dsdpa_tile.h"
#include "dsdpa_cell.h"
#include "dsdpa_plane.h"
#include "dsdpa_dense.h"
#include "dsdpa_slab.h"

namespace dsdpa {

static_assert(kPlaneDescLdsBytes == (size_t)kPlaneDescBytes && kPlaneGradLdsBytes == (size_t)kPlaneGradBytes,
              "host and device agree on the descriptor block");

// ------------------------------------------------------------------ small kernels
static __global__ void fill_zero_kernel(ZeroJob job) { zero_buffers(job); }

// A launch that may carry the kernel timer's events. Without them it is a plain launch: only those are
// known to be recorded by a stream capture.
#define DSDPA_LAUNCH(kern, grid, block, smem, st, ev0, ev1, ...)                                             \
    do {                                                                                                     \
        hipEvent_t ev0_ = (ev0), ev1_ = (ev1);                                                               \
        if (ev0_ || ev1_) hipExtLaunchKernelGGL(kern, grid, block, smem, st, ev0_, ev1_, 0, __VA_ARGS__);    \
        else hipLaunchKernelGGL(kern, grid, block, smem, st, __VA_ARGS__);                                   \
    } while (0)

// Lets a kernel instantiation use the whole 160 KB of LDS as dynamic shared memory. The attribute belongs to
// the kernel, not to the launch, so it is set once per instantiation and device (`done`: one bit per device),
// to the largest block any launch may ask for; a launch's own block size is an argument of that launch.
template <typename K>
int allow_full_lds(K kern, std::atomic<unsigned long long> &done)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        dev = 0;
    }
    const unsigned long long bit = 1ull << dev;
    if (done.load(std::memory_order_acquire) & bit) return DSDPA_OK;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
    if (e != hipSuccess) { g_last_hip_error = (int)e; return DSDPA_ERR_HIP; }
    done.fetch_or(bit, std::memory_order_release);
    return DSDPA_OK;
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

// stats[row] = (lse[row], delta[row]), delta = dout[row] . out[row] (the reference's _bwd_preprocess,
// ops/triton.py:197-215; the pair side by side so that the dk/dv kernels fetch both with one load), as a launch of
// its own, for when the dk/dv kernel does not run behind the dq kernel (which computes it on the way).
// Four lanes per row, four elements per lane and step.
template <typename S>
__global__ __launch_bounds__(256) void delta_kernel(const void *__restrict__ out_, const void *__restrict__ dout_,
                                                    const float *__restrict__ lse_, float2 *__restrict__ stats_,
                                                    size_t rows, int D)
{
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t row = t >> 2;
    const int j = (int)(t & 3);
    const size_t r = row < rows ? row : rows - 1;
    float acc = 0.f;
    for (int e = j * 4; e < D; e += 16) {
        float a[4], b[4];
        load_chunk<S, 4>((const char *)out_ + (r * D + e) * S::kBytes, a);
        load_chunk<S, 4>((const char *)dout_ + (r * D + e) * S::kBytes, b);
#pragma unroll
        for (int d = 0; d < 4; ++d) acc = fmaf(a[d], b[d], acc);
    }
    acc = group_sum<4>(acc);
    if (row < rows && j == 0) stats_[row] = make_float2(lse_[row], acc);
}

static inline int make_dims(int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, Dims *dm)
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
    dm->divP = FastDiv::make((unsigned)P);
    dm->divL = FastDiv::make((unsigned)L);
    dm->q_sl = dm->kv_sl = D;
    dm->q_sh = dm->kv_sh = L * D;
    dm->q_sv = dm->kv_sv = (int)((long long)H * L * D);
    dm->q_sb = dm->kv_sb = slab;
    return DSDPA_OK;
}

// Strides of q and of k/v as the caller gives them: element strides over (batch, view, head, pixel), q's four
// then k/v's four; the head dimension must be contiguous (a row is read with 16-byte loads). The kernels
// address a pixel of a (batch, head) as view*sv + pixel*sl in 32 bits, and every row start must be a
// multiple of 16 bytes.
static inline int apply_strides(const long long *st, int D, int esize, Dims *dm, bool *contiguous)
{
    *contiguous = true;
    if (!st) return DSDPA_OK;
    const long long align = 16 / esize;
    for (int t = 0; t < 2; ++t) {
        const long long sb = st[4 * t], sv = st[4 * t + 1], sh = st[4 * t + 2], sl = st[4 * t + 3];
        if (sb < 0 || sv < 0 || sh < 0 || sl < D) return DSDPA_ERR_BAD_STRIDES;
        if (sb % align || sv % align || sh % align || sl % align) return DSDPA_ERR_BAD_STRIDES;
        const long long reach = (long long)(dm->V - 1) * sv + (long long)(dm->L - 1) * sl + D;   // inside one (b, h)
        if (reach > (1ll << 30) || sv > (1ll << 30)) return DSDPA_ERR_TOO_LARGE;
        if (t == 0) { dm->q_sb = sb; dm->q_sv = (int)sv; dm->q_sh = sh; dm->q_sl = (int)sl; }
        else { dm->kv_sb = sb; dm->kv_sv = (int)sv; dm->kv_sh = sh; dm->kv_sl = (int)sl; }
    }
    const long long L = dm->L, H = dm->H;
    *contiguous = dm->q_sl == D && dm->q_sh == L * D && dm->q_sv == H * L * D && dm->q_sb == (long long)dm->V * H * L * D &&
                  dm->kv_sl == D && dm->kv_sh == L * D && dm->kv_sv == H * L * D && dm->kv_sb == (long long)dm->V * H * L * D;
    return DSDPA_OK;
}

// lanes per sample are D/DC; DC is chosen so that a lane moves 16 bytes per tap
// (32 or 64 for the widest heads) and a sample never spans more than 16 lanes.
template <typename S, int D> struct Chunk {
    static constexpr int kMin = 16 / S::kBytes;
    static constexpr int value = (D / kMin > 16) ? D / 16 : kMin;
};

// The gather kernels cut a row's samples into chunks per key view, each of which may be worked on per pixel of
// the window its samples fall into, when a view has at least a chunk's worth of samples; with fewer, chunks of
// 64 consecutive samples (several views each) keep the lanes busy and always gather.
static inline bool gather_window_mode(int P) { return P >= kWave; }

// todo (may be null): flags of the tiles of 16 queries that fwd_dense_kernel left undone; rows of the other tiles are skipped
template <typename S, int D>
int launch_fwd_gather(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
                      const unsigned char *todo, int ntl, const Dims &dm, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const int blocks = (dm.rows + kGatherWaves - 1) / kGatherWaves;
    ScopedKernelTimer timer(0, st);
    if (gather_window_mode(dm.P))
        DSDPA_LAUNCH((fwd_gather_kernel<S, D, DC, true>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                              timer.start(), timer.stop(),
                           q, k, v, coords, out, lse, todo, ntl, dm);
    else
        DSDPA_LAUNCH((fwd_gather_kernel<S, D, DC, false>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                              timer.start(), timer.stop(),
                           q, k, v, coords, out, lse, todo, ntl, dm);
    return check_launch();
}

// Waves per workgroup and samples per lane and view of the slab kernels: 12 x 4 (168 registers a lane, no spills at
// D = 64) measured 3-4 % ahead of 16 x 3 (128 registers) at 32x32, D = 64; both cover 192 query rows.
constexpr int kSlabWaves = 12, kSlabItems = 4;
// (D = 128 with 32 samples per view: two samples per lane and view -- one query row -- measured 15 % ahead of four,
//  which spill there; with 16 samples per view four stay ahead on the larger images)
template <int D, int KB> struct SlabItems { static constexpr int value = (D >= 128 && KB == 2) ? kSlabItems / 2 : kSlabItems; };
// The slab forward (fp32 storage, 16 samples per view): a workgroup per block of 192 query rows of a
// (batch, head); the whole image of a view in LDS, 16 columns at a time, in two buffers.
template <typename S, int D>
int launch_fwd_slab(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
                    const Dims &dm, hipStream_t st)
{
    if constexpr (S::kBytes != 4 || (D != 32 && D != 64 && D != 128)) {
        return DSDPA_ERR_UNSUPPORTED;
    } else {
        constexpr int IT1 = SlabItems<D, 1>::value, IT2 = SlabItems<D, 2>::value, NW = kSlabWaves;
        const int kb = dm.P / kSlabSamples;                  // 1 or 2 (slab_path_fits)
        const int IT = kb == 1 ? IT1 : IT2;
        const int RB = NW * 4 * IT / kb;
        const int nblk = (dm.V * dm.L + RB - 1) / RB;
        const long long blocks = (long long)dm.B * dm.H * nblk;
        if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
        auto kern = kb == 1 ? fwd_slab_kernel<D, IT1, NW, 1> : fwd_slab_kernel<D, IT2, NW, 2>;
        static std::atomic<unsigned long long> lds_set[2];
        if (int rc = allow_full_lds(kern, lds_set[kb >> 1])) return rc;
        ScopedKernelTimer timer(0, st);
        const unsigned buf_bytes = (unsigned)slab_buffer_bytes(dm.Himg, dm.Wimg);
        DSDPA_LAUNCH(kern, dim3((unsigned)blocks), dim3(NW * kWave), (size_t)2 * buf_bytes + NW * 4 * IT * kSlabBytes, st, timer.start(),
                     timer.stop(), (const float *)q, (const float *)k, (const float *)v, coords, (float *)out, lse, dm, nblk,
                     slab_pitch(dm.Wimg), buf_bytes);
        return check_launch();
    }
}

// dq of the same shapes, for the (batch, head) pairs [bh0, bh0 + nbh). With the coordinate gradient a lane takes
// half as many samples per view (the per-tap products it then keeps take the registers): 96 query rows a workgroup.
template <typename S, int D, bool CG>
int launch_bwd_dq_slab_cg(const void *q, const void *k, const void *v, const float *coords, const void *out,
                          const float *lse, const void *dout, void *dq, float2 *stats, float2 *handed, float *dcoords,
                          const Dims &dm, int bh0, int nbh, hipStream_t st)
{
    if constexpr (S::kBytes != 4 || (D != 32 && D != 64 && D != 128)) {
        return DSDPA_ERR_UNSUPPORTED;
    } else {
        constexpr int IT1 = CG ? kSlabItems / 2 : SlabItems<D, 1>::value, IT2 = CG ? kSlabItems / 2 : SlabItems<D, 2>::value;
        constexpr int NW = kSlabWaves;
        const int kb = dm.P / kSlabSamples;
        const int IT = kb == 1 ? IT1 : IT2;
        const int RB = NW * 4 * IT / kb;
        const int nblk = (dm.V * dm.L + RB - 1) / RB;
        const long long blocks = (long long)nbh * nblk;
        if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
        auto kern = kb == 1 ? bwd_dq_slab_kernel<D, IT1, NW, 1, CG> : bwd_dq_slab_kernel<D, IT2, NW, 2, CG>;
        static std::atomic<unsigned long long> lds_set[2];
        if (int rc = allow_full_lds(kern, lds_set[kb >> 1])) return rc;
        ScopedKernelTimer timer(2, st);
        const unsigned buf_bytes = (unsigned)slab_buffer_bytes(dm.Himg, dm.Wimg);
        DSDPA_LAUNCH(kern, dim3((unsigned)blocks), dim3(NW * kWave), (size_t)2 * buf_bytes + NW * 4 * IT * kSlabBytes, st,
                     timer.start(), timer.stop(), (const float *)q, (const float *)k, (const float *)v, coords,
                     (const float *)out, lse, (const float *)dout, (float *)dq, stats, handed, dcoords, dm, bh0, nblk,
                     slab_pitch(dm.Wimg), buf_bytes);
        return check_launch();
    }
}

template <typename S, int D>
int launch_bwd_dq_slab(const void *q, const void *k, const void *v, const float *coords, const void *out,
                       const float *lse, const void *dout, void *dq, float2 *stats, float2 *handed, float *dcoords,
                       const Dims &dm, int bh0, int nbh, hipStream_t st)
{
    return dcoords ? launch_bwd_dq_slab_cg<S, D, true>(q, k, v, coords, out, lse, dout, dq, stats, handed, dcoords, dm, bh0, nbh, st)
                   : launch_bwd_dq_slab_cg<S, D, false>(q, k, v, coords, out, lse, dout, dq, stats, handed, dcoords, dm, bh0, nbh, st);
}

// The dense-box forward (16-bit storage, D = 64 or 128): one workgroup per tile of 16 queries; the tiles it
// declines are flagged in the workspace (one flag per 16 queries) for the gather kernel that the caller launches
// behind it.
// (tiles of 32 queries -- every staged row then feeds two matrix instructions -- were measured slower: one workgroup
//  of eight waves per CU and boxes a fifth larger; 64x64, D = 128, clustered: 1.92 ms against 1.72)
template <int D> struct DenseTile { static constexpr int value = 16; };
template <typename S, int D>
int launch_fwd_dense(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
                     char *ws, const DenseLayout &dn, const Dims &dm, hipStream_t st)
{
    if constexpr (S::kBytes != 2 || (D != 64 && D != 128)) {
        return DSDPA_ERR_UNSUPPORTED;
    } else {
        constexpr int TQ = DenseTile<D>::value;
        using C = DenseCfg<D, TQ>;
        const int ntl = (dm.L + TQ - 1) / TQ;
        const long long tiles = (long long)dm.B * dm.H * dm.V * ntl;
        if (tiles > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
        auto kern = fwd_dense_kernel<S, D, TQ>;
        static std::atomic<unsigned long long> lds_set{0};
        if (int rc = allow_full_lds(kern, lds_set)) return rc;
        ScopedKernelTimer timer(0, st);
        DSDPA_LAUNCH(kern, dim3((unsigned)tiles), dim3(C::kThreads), (size_t)C::kLdsBytes, st, timer.start(), timer.stop(),
                     q, k, v, coords, out, lse, (unsigned char *)(ws + dn.todo), dm, ntl);
        return check_launch();
    }
}

template <typename S, int D>
int launch_bwd_gather(const void *q, const void *k, const void *v, const float *coords, const void *out,
                      const float *lse, const void *dout, void *dq, float *dk_acc, float *dv_acc,
                      const Dims &dm, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const int blocks = (dm.rows + kGatherWaves - 1) / kGatherWaves;
    ScopedKernelTimer timer(1, st);
    DSDPA_LAUNCH((bwd_gather_kernel<S, D, DC>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                          timer.start(), timer.stop(),
                       q, k, v, coords, out, lse, dout, dq, dk_acc, dv_acc, dm);
    return check_launch();
}

// The query rows of the (batch, head) pairs [bh0, bh0 + nbh) (all of them: 0, B*H).
template <typename S, int D>
int launch_bwd_dq_gather(const void *q, const void *k, const void *v, const float *coords, const void *out,
                         const float *lse, const void *dout, void *dq, float2 *stats, float *dcoords,
                         float2 *handed, const Dims &dm, int bh0, int nbh, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const int work0 = bh0 * dm.V * dm.L, work_end = (bh0 + nbh) * dm.V * dm.L;      // (at most dm.rows)
    const int blocks = (work_end - work0 + kGatherWaves - 1) / kGatherWaves;
    ScopedKernelTimer timer(2, st);
    if (dcoords && gather_window_mode(dm.P))
        DSDPA_LAUNCH((bwd_dq_gather_kernel<S, D, DC, true, true>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                              timer.start(), timer.stop(),
                           q, k, v, coords, out, lse, dout, dq, stats, dcoords, handed, dm, work0, work_end);
    else if (dcoords)
        DSDPA_LAUNCH((bwd_dq_gather_kernel<S, D, DC, true, false>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                              timer.start(), timer.stop(),
                           q, k, v, coords, out, lse, dout, dq, stats, dcoords, handed, dm, work0, work_end);
    else if (gather_window_mode(dm.P))
        DSDPA_LAUNCH((bwd_dq_gather_kernel<S, D, DC, false, true>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                              timer.start(), timer.stop(),
                           q, k, v, coords, out, lse, dout, dq, stats, dcoords, handed, dm, work0, work_end);
    else
        DSDPA_LAUNCH((bwd_dq_gather_kernel<S, D, DC, false, false>), dim3(blocks), dim3(kGatherWaves * kWave), 0, st,
                              timer.start(), timer.stop(),
                           q, k, v, coords, out, lse, dout, dq, stats, dcoords, handed, dm, work0, work_end);
    return check_launch();
}

constexpr int kTileDescBytes = kTileWaves * kWave * (16 + 16 + 4);      // per-wave tap descriptors

// Tile geometry for the dk/dv kernel: as few tiles per plane as the LDS budget allows
// (every tile costs one more pass over the plane's coordinates and one halo ring).
static inline TileGeom make_tile_geom(const Dims &dm, int D)
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
int launch_bwd_dkdv_tile(const void *q, const void *k, const void *v, const float *coords,
                         const float2 *stats, const void *dout, float *dk_acc, float *dv_acc, const Dims &dm,
                         hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const TileGeom tg = make_tile_geom(dm, D);
    const size_t smem = (size_t)2 * sizeof(double) * tg.lh * tg.lw * D + kTileDescBytes;
    if (smem > (size_t)kLdsBytes) return DSDPA_ERR_TOO_LARGE;
    const long long blocks = (long long)dm.B * dm.H * dm.V * tg.nty * tg.ntx * tg.qsplit;
    if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
    auto kern = bwd_dkdv_tile_kernel<S, D, DC>;
    static std::atomic<unsigned long long> lds_set{0};
    if (int rc = allow_full_lds(kern, lds_set)) return rc;
    ScopedKernelTimer timer(1, st);
    DSDPA_LAUNCH(kern, dim3((unsigned)blocks), dim3(kTileWaves * kWave), smem, st,
                          timer.start(), timer.stop(),
                       q, k, v, coords, stats, dout, dk_acc, dv_acc, dm, tg);
    return check_launch();
}

template <typename S>
bool plane_fits(const Dims &dm, int D)
{
    return plane_path_fits((size_t)dm.L, (size_t)D, S::kBytes);
}

// Fill the descriptor table of the plane kernels (one thread per coordinate pair, padded to whole waves).
// `zero`: buffers the same launch clears on the side (the backward's accumulators and counters).
static inline int launch_plane_descriptors(const float *coords, const Dims &dm, char *table, const DescLayout &dl,
                                           bool coords_grad, const ZeroJob &zero, int timer_slot, hipStream_t st)
{
    const long long nblk = (long long)dm.B * dm.V * dm.L * dm.V;
    const long long waves = dm.P <= 32 ? (nblk + 1) / 2 : nblk * ((dm.P + 63) / 64);
    const long long blocks = (waves * kWave + kDescThreads - 1) / kDescThreads;
    if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
    ScopedKernelTimer timer(timer_slot, st);
    DSDPA_LAUNCH(plane_descriptor_kernel, dim3((unsigned)blocks), dim3(kDescThreads), 0, st,
                          timer.start(), timer.stop(), coords, dm,
                       (float4 *)(table + dl.w), (uint32_t *)(table + dl.e),
                       coords_grad ? (float4 *)(table + dl.g) : (float4 *)nullptr, zero);
    return check_launch();
}

template <typename S, int D>
int launch_fwd_plane(const void *q, const void *k, const void *v, const float4 *desc_w, const uint32_t *desc_e,
                     void *out, float *lse, const Dims &dm, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const size_t smem = (size_t)plane_lds_bytes<S, D>(dm.L) + kPlaneDescBytes;
    int waves, row_blocks;
    plane_config((long long)dm.B * dm.H, dm.V * dm.L, kWave / (D / DC), dm.P, device_cus(), DC <= 8 ? 2 : 1, &waves,
                 &row_blocks);          // (16 elements per lane: two rows' state does not fit in the registers)
    const int rows_per_block = row_blocks * waves * (kWave / (D / DC));
    const long long blocks = (long long)dm.B * dm.H * ((dm.V * dm.L + rows_per_block - 1) / rows_per_block);
    auto kern = fwd_slot_kernel<S, D, DC, 1>;
    if constexpr (DC <= 8) {
        if (row_blocks == 2) kern = fwd_slot_kernel<S, D, DC, 2>;
    }
    static std::atomic<unsigned long long> lds_set[2];
    if (int rc = allow_full_lds(kern, lds_set[row_blocks - 1])) return rc;
    ScopedKernelTimer timer(0, st);
    DSDPA_LAUNCH(kern, dim3((unsigned)blocks), dim3(waves * kWave), smem, st,
                          timer.start(), timer.stop(), q, k, v, desc_w, desc_e, out, lse, dm);
    return check_launch();
}

template <typename S, int D>
int launch_bwd_dq_plane(const void *q, const void *k, const void *v, const float4 *desc_w,
                        const uint32_t *desc_e, const void *out,
                        const float *lse, const void *dout, void *dq, float2 *stats, const float4 *desc_g,
                        float *dcoords, const Dims &dm, hipStream_t st)
{
    constexpr int DC = Chunk<S, D>::value;
    const size_t smem = (size_t)plane_lds_bytes<S, D>(dm.L) + kPlaneDescBytes + (dcoords ? kPlaneGradBytes : 0);
    int waves, row_blocks;
    // (two row blocks only without the coordinate gradient and up to 8 elements per lane: registers)
    plane_config((long long)dm.B * dm.H, dm.V * dm.L, kWave / (D / DC), dm.P, device_cus(), (!dcoords && DC <= 8) ? 2 : 1,
                 &waves, &row_blocks);
    const int rows_per_block = row_blocks * waves * (kWave / (D / DC));
    const long long blocks = (long long)dm.B * dm.H * ((dm.V * dm.L + rows_per_block - 1) / rows_per_block);
    auto kern = dcoords ? bwd_dq_slot_kernel<S, D, DC, true, 1> : bwd_dq_slot_kernel<S, D, DC, false, 1>;
    if constexpr (DC <= 8) {
        if (row_blocks == 2) kern = bwd_dq_slot_kernel<S, D, DC, false, 2>;
    }
    static std::atomic<unsigned long long> lds_set[3];
    if (int rc = allow_full_lds(kern, lds_set[dcoords ? 2 : row_blocks - 1])) return rc;
    ScopedKernelTimer timer(2, st);
    DSDPA_LAUNCH(kern, dim3((unsigned)blocks), dim3(waves * kWave), smem, st,
                          timer.start(), timer.stop(), q, k, v, desc_w, desc_e, out, lse, dout, dq, stats, desc_g,
                          dcoords, dm);
    return check_launch();
}

template <typename S>
int fwd_impl(const void *q, const void *k, const void *v, const float *coords, void *out, float *lse,
             void *workspace, int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale,
             const long long *strides, void *stream, bool dense_ok)
{
    if (!q || !k || !v || !coords || !out || !lse) return DSDPA_ERR_NULL_POINTER;
    Dims dm;
    int rc = make_dims(B, V, H, Himg, Wimg, D, P, sm_scale, &dm);
    if (rc != DSDPA_OK) return rc;
    bool contiguous;
    if ((rc = apply_strides(strides, D, S::kBytes, &dm, &contiguous)) != DSDPA_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    const DescLayout dl = desc_layout(B, V, Himg, Wimg, D, P, S::kBytes);
    const DenseLayout dn = dense_ok ? dense_layout(B, V, H, Himg, Wimg, D, P, S::kBytes) : DenseLayout{0, 0, 0};
    if ((dl.bytes || dn.bytes) && !workspace) return DSDPA_ERR_NULL_POINTER;
    const int path = g_path.load();
    const bool staged = path != DSDPA_PATH_GATHER && dl.bytes != 0 &&
                        (path == DSDPA_PATH_LDS || !few_samples_prefer_gather(V, P));
    // (DSDPA_PATH_GATHER keeps its meaning: every tap, or every pixel of a query's window, read by the gather kernel)
    const bool dense = path == DSDPA_PATH_AUTO && dn.bytes != 0;
    const bool slab = path == DSDPA_PATH_AUTO && !staged && slab_path_fits(V, Himg, Wimg, D, P, S::kBytes);
    char *ws = (char *)workspace;
    if (staged && (rc = launch_plane_descriptors(coords, dm, ws, dl, false, ZeroJob{}, 4, st)) != DSDPA_OK) return rc;
    const float4 *desc_w = (const float4 *)(ws + dl.w);
    const uint32_t *desc_e = (const uint32_t *)(ws + dl.e);
    const unsigned char *todo = dense ? (const unsigned char *)(ws + dn.todo) : nullptr;
#define DSDPA_FWD_CASE(DD)                                                                        \
    case DD:                                                                                      \
        if (staged) return launch_fwd_plane<S, DD>(q, k, v, desc_w, desc_e, out, lse, dm, st);    \
        if (slab) return launch_fwd_slab<S, DD>(q, k, v, coords, out, lse, dm, st);               \
        if (dense && (rc = launch_fwd_dense<S, DD>(q, k, v, coords, out, lse, ws, dn, dm, st)) != DSDPA_OK) return rc; \
        return launch_fwd_gather<S, DD>(q, k, v, coords, out, lse, todo, dn.ntl, dm, st);
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

static inline int zero_fill(const ZeroJob &job, hipStream_t st)
{
    size_t big = 0;
    for (int i = 0; i < 4; ++i) big = job.n[i] / 4 > big ? job.n[i] / 4 : big;
    const int threads = 256;
    size_t blocks = (big + threads - 1) / threads;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(threads), 0, st, job);
    return check_launch();
}

// elements per lane in the cell kernel. fp32: 4 up to D = 128 (64 tap/accumulator registers, 5 waves per
// SIMD; 8 elements per lane at D = 32/64 were measured slower: 211 VGPRs, 2 waves per SIMD). 16-bit storage
// keeps the taps packed, so 8 elements per lane fit in ~150 VGPRs and pay off from D = 128 on, where 4 per
// lane would spread one sample over 32 lanes and repeat the per-sample scalar work in all of them.
template <typename S, int D> struct CellChunk {
    static constexpr int value = S::kBytes == 2 ? (D <= 64 ? 4 : 8) : (D <= 128 ? 4 : 8);
};

// records: the lists as 12-byte records (id and position in the cell) from wl.sorted on, through the room of
// wl.frac behind it; else plain ids in wl.sorted (the deterministic backward, which sorts them).
static inline int launch_binning(const float *coords, const Dims &dm, const WorkspaceLayout &wl, char *ws,
                                 int records, hipStream_t st)
{
    unsigned *counters = (unsigned *)(ws + wl.counters);
    unsigned *start = (unsigned *)(ws + wl.start);
    unsigned *sorted = (unsigned *)(ws + wl.sorted);
    const size_t hist_bytes = (size_t)dm.V * wl.NC * sizeof(unsigned);
    // each of the three launches carries its own pair of events: the timer's slot 3 adds up their busy time
    ScopedKernelTimer t_count(3, st), t_scan(3, st), t_fill(3, st);
    if (2 * hist_bytes <= (size_t)kLdsBytes - 1024) {
        // LDS-aggregated passes: a workgroup per run of about 4k samples of one (b, s1); more when the histogram
        // is large, since every workgroup walks all of it twice: twice its counters, between 8k and 32k samples, as
        // long as that leaves 128 workgroups (64x64, 4 views, 8.4 M samples: 0.203 ms for the three launches with
        // runs of 8k, 0.179 with 16k or 32k, 0.229 with 64k; 48x48, 6 views, 5.3 M: 0.177 / 0.174 / 0.157 / 0.221;
        // 32x32, 6 views, 0.6 M: 0.037 / 0.050 / 0.072)
        const long long hist_entries = (long long)dm.V * wl.NC, total_samples = (long long)dm.B * dm.V * dm.L * dm.N;
        long long run = 4096;
        if (hist_entries >= 4096) {
            run = 2 * hist_entries < 8192 ? 8192 : (2 * hist_entries > 32768 ? 32768 : 2 * hist_entries);
            while (run > 8192 && total_samples / run < 128) run /= 2;
            if (run < 8192) run = 8192;
        }
        int lchunk = (int)(run / dm.N);
        if (lchunk < 1) lchunk = 1;
        if (lchunk > dm.L) lchunk = dm.L;
        const int nlc = (dm.L + lchunk - 1) / lchunk;
        lchunk = (dm.L + nlc - 1) / nlc;
        const long long blocks = (long long)dm.B * dm.V * nlc;
        if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
        auto k0 = bin_samples_lds_kernel<0>;
        auto k1 = bin_samples_lds_kernel<1>;
        static std::atomic<unsigned long long> lds_set[2];
        if (int rc = allow_full_lds(k0, lds_set[0])) return rc;
        if (int rc = allow_full_lds(k1, lds_set[1])) return rc;
        DSDPA_LAUNCH(k0, dim3((unsigned)blocks), dim3(kBinLdsThreads), hist_bytes, st,
                              t_count.start(), t_count.stop(),
                           coords, dm, wl.NC, wl.NK, wl.vpg, lchunk, nlc, counters, sorted, records);
        DSDPA_LAUNCH(bin_scan_kernel, dim3((unsigned)(dm.B * dm.V)), dim3(1024), 0, st,
                              t_scan.start(), t_scan.stop(), counters, start, wl.NK, wl.NC, wl.piece, wl.wmax,
                              (uint4 *)(ws + wl.items));
        DSDPA_LAUNCH(k1, dim3((unsigned)blocks), dim3(kBinLdsThreads), 2 * hist_bytes, st,
                              t_fill.start(), t_fill.stop(),
                           coords, dm, wl.NC, wl.NK, wl.vpg, lchunk, nlc, counters, sorted, records);
        return check_launch();
    }
    const long long total = (long long)dm.B * dm.V * dm.L * dm.N;
    const long long blocks = (total + kBinThreads - 1) / kBinThreads;
    if (blocks > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;
    DSDPA_LAUNCH(bin_samples_kernel<0>, dim3((unsigned)blocks), dim3(kBinThreads), 0, st,
                          t_count.start(), t_count.stop(),
                       coords, dm, wl.NC, wl.NK, wl.vpg, counters, sorted, records);
    DSDPA_LAUNCH(bin_scan_kernel, dim3((unsigned)(dm.B * dm.V)), dim3(1024), 0, st,
                          t_scan.start(), t_scan.stop(), counters, start, wl.NK, wl.NC, wl.piece, wl.wmax,
                              (uint4 *)(ws + wl.items));
    DSDPA_LAUNCH(bin_samples_kernel<1>, dim3((unsigned)blocks), dim3(kBinThreads), 0, st,
                          t_fill.start(), t_fill.stop(),
                       coords, dm, wl.NC, wl.NK, wl.vpg, counters, sorted, records);
    return check_launch();
}

// deterministic: four launches, one per (row parity, column parity) of the cells, each with plain stores
template <typename S, int D>
int launch_bwd_dkdv_cell(const void *q, const void *k, const void *v, const float *coords,
                         const float2 *stats, const void *dout, const unsigned *start, const unsigned *sorted,
                         int records, const uint4 *items, unsigned wmax, const float2 *handed,
                         float *dk_acc, float *dv_acc, const Dims &dm, int NC, bool deterministic, int bh0, int nbh,
                         hipStream_t st)
{
    constexpr int DC = CellChunk<S, D>::value;
    ScopedKernelTimer timer(1, st);
    for (int colour = deterministic ? 0 : -1; colour < (deterministic ? 4 : 0); ++colour) {
        const int cw = dm.Wimg + 1, ch = dm.Himg + 1;
        CellGrid cg;
        cg.colour = colour;
        cg.oy = colour < 0 ? 0 : colour >> 1;
        cg.ox = colour < 0 ? 0 : colour & 1;
        cg.step = colour < 0 ? 1 : 2;
        cg.ncx = (cw - cg.ox + cg.step - 1) / cg.step;
        cg.ncells = cg.ncx * ((ch - cg.oy + cg.step - 1) / cg.step);
        if (colour < 0) cg.ncells = (int)wmax;          // work-list mode: one wave per item slot
        const long long nwork = (long long)nbh * dm.V * cg.ncells;       // the pairs [bh0, bh0 + nbh) of (batch, head)
        if (nwork >= 0x7fffffffll - kCellWaves) return DSDPA_ERR_TOO_LARGE;
        cg.bh0 = bh0;
        cg.nwork = (unsigned)nwork;
        cg.div_cells = FastDiv::make((unsigned)cg.ncells);
        cg.div_ncx = FastDiv::make((unsigned)cg.ncx);
        cg.div_v = FastDiv::make((unsigned)dm.V);
        cg.div_h = FastDiv::make((unsigned)dm.H);
        const unsigned blocks = (unsigned)((nwork + kCellWaves - 1) / kCellWaves);
        const bool first = colour <= 0, last = colour < 0 || colour == 3;
        if (handed && colour < 0 && records)
            DSDPA_LAUNCH((bwd_dkdv_cell_kernel<S, D, DC, true, true>), dim3(blocks), dim3(kCellWaves * kWave), 0, st,
                                  first ? timer.start() : nullptr, last ? timer.stop() : nullptr, q, k, v, coords,
                                  stats, dout, start, sorted, items, handed, dk_acc, dv_acc, dm, NC, cg);
        else if (records)
            DSDPA_LAUNCH((bwd_dkdv_cell_kernel<S, D, DC, false, true>), dim3(blocks), dim3(kCellWaves * kWave), 0, st,
                                  first ? timer.start() : nullptr, last ? timer.stop() : nullptr, q, k, v, coords,
                                  stats, dout, start, sorted, items, handed, dk_acc, dv_acc, dm, NC, cg);
        else
            DSDPA_LAUNCH((bwd_dkdv_cell_kernel<S, D, DC, false, false>), dim3(blocks), dim3(kCellWaves * kWave), 0, st,
                                  first ? timer.start() : nullptr, last ? timer.stop() : nullptr, q, k, v, coords,
                                  stats, dout, start, sorted, items, handed, dk_acc, dv_acc, dm, NC, cg);
    }
    return check_launch();
}

// Deterministic backward: order every cell list by sample id (the counting sort leaves the order inside a
// cell to its atomics).
static inline int launch_list_ordering(const Dims &dm, const WorkspaceLayout &wl, char *ws, hipStream_t st)
{
    const size_t M = (size_t)dm.V * dm.L * dm.P, groups = (size_t)dm.B * dm.V;
    const size_t ids = groups * M, segs = groups * (size_t)wl.NC;
    if (ids > 0xffffffffull || segs > 0x7fffffffull) return DSDPA_ERR_TOO_LARGE;
    unsigned *seg_begin = (unsigned *)(ws + wl.seg), *seg_end = seg_begin + segs;
    ScopedKernelTimer timer(3, st, /*record=*/true);      // the sort launches its own kernels
    hipLaunchKernelGGL(cell_segments_kernel, dim3((unsigned)((segs + 255) / 256)), dim3(256), 0, st,
                       (const unsigned *)(ws + wl.start), wl.NC, (unsigned)M, (unsigned)segs, seg_begin, seg_end);
    int rc = check_launch();
    if (rc != DSDPA_OK) return rc;
    unsigned bits = 1;
    while (bits < 32 && (1ull << bits) < M) ++bits;
    return sort_cell_lists(ws + wl.sorttmp, wl.sorttmp_bytes, (const unsigned *)(ws + wl.sorted),
                           (unsigned *)(ws + wl.sorted2), ids, segs, seg_begin, seg_end, bits, st);
}

// Joins the backward's side lane to the caller's stream, once: by join() on the normal path, by the
// destructor on every other way out of bwd_impl after the fork (an error return must not leave work on the
// side lane that the caller's stream does not wait for: the caller may free the buffers it writes, and a
// stream capture with an unjoined fork is invalid).
struct SideJoin {
    SideLane *side = nullptr;
    hipStream_t main = nullptr;
    bool pending = false;
    int join()
    {
        if (!pending) return DSDPA_OK;
        pending = false;
        hipError_t e = hipEventRecord(side->join, side->stream);
        if (e == hipSuccess) e = hipStreamWaitEvent(main, side->join, 0);
        if (e != hipSuccess) { g_last_hip_error = (int)e; return DSDPA_ERR_HIP; }
        return DSDPA_OK;
    }
    ~SideJoin() { (void)join(); }
};

template <typename S>
int bwd_impl(const void *q, const void *k, const void *v, const float *coords, const void *out,
             const float *lse, const void *dout, void *dq, void *dk, void *dv, float *dcoords, void *workspace,
             int B, int V, int H, int Himg, int Wimg, int D, int P, float sm_scale, const long long *strides,
             unsigned flags, void *stream)
{
    if (!q || !k || !v || !coords || !out || !lse || !dout || !dq || !dk || !dv || !workspace)
        return DSDPA_ERR_NULL_POINTER;
    if (flags & ~(unsigned)(DSDPA_FLAG_DETERMINISTIC | DSDPA_FLAG_COORDS_GRAD | DSDPA_FLAG_SINGLE_STREAM)) return DSDPA_ERR_UNSUPPORTED;
    const bool deterministic = (flags & DSDPA_FLAG_DETERMINISTIC) != 0;
    if (deterministic && dcoords) return DSDPA_ERR_UNSUPPORTED;   // dcoords sums over heads with float atomics
    Dims dm;
    int rc = make_dims(B, V, H, Himg, Wimg, D, P, sm_scale, &dm);
    if (rc != DSDPA_OK) return rc;
    if ((long long)dm.L * dm.N > 0x7fffffffll) return DSDPA_ERR_TOO_LARGE;   // sample ids are 32-bit
    bool contiguous;
    if ((rc = apply_strides(strides, D, S::kBytes, &dm, &contiguous)) != DSDPA_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    const size_t n = (size_t)dm.rows * D;
    // the staged dq kernel computes dcoords only when the caller sized the workspace for it (same flags)
    const bool cg_table = dcoords && (flags & DSDPA_FLAG_COORDS_GRAD) != 0;
    const WorkspaceLayout wl = workspace_layout(B, V, H, Himg, Wimg, D, P, S::kBytes != 4, deterministic, cg_table);
    char *ws = (char *)workspace;
    float2 *stats = (float2 *)(ws + wl.delta);          // per row: lse, delta
    const int path = deterministic ? (int)DSDPA_PATH_AUTO : g_path.load();   // only the cell-binned path has a fixed order
    // (the per-tap atomic backward, kept as the reference's scheme for measurements, takes a tap's offset in k/v
    // for its offset in dk/dv: with strided k/v the gather dq kernel and the cell-binned dk/dv take its place)
    const bool fused_atomics = path == DSDPA_PATH_GATHER && contiguous;
    const bool cell_binned = path == DSDPA_PATH_AUTO || (path == DSDPA_PATH_GATHER && !contiguous);
    // (with the coordinate gradient the layout holds a table only where the larger LDS block still fits)
    const bool staged = path != DSDPA_PATH_GATHER && wl.dl.bytes != 0 && (!dcoords || cg_table) &&
                        (path == DSDPA_PATH_LDS || !few_samples_prefer_gather(V, P));
    const float4 *desc_w = (const float4 *)(ws + wl.desc + wl.dl.w);
    const uint32_t *desc_e = (const uint32_t *)(ws + wl.desc + wl.dl.e);
    const float4 *desc_g = (const float4 *)(ws + wl.desc + wl.dl.g);
    const unsigned *start = (const unsigned *)(ws + wl.start);
    const unsigned *sorted = (const unsigned *)(ws + (deterministic ? wl.sorted2 : wl.sorted));
    // (the reordered lists of the deterministic backward are ids without positions beside them: coordinates are read again)
    const int records = deterministic ? 0 : 1;
    // (p, sm_scale * ds) per query*sample from the dq kernel to the dk/dv kernel, where the layout has room for it
    // (shapes on the gather dq kernel, which then runs before dk/dv on the same stream)
    float2 *handed = (wl.handed_bytes && cell_binned && !staged) ? (float2 *)(ws + wl.handed) : nullptr;
    // fp32 storage: dk and dv are their own accumulators; 16-bit: fp32 accumulators in the workspace
    float *dk_acc = S::kBytes == 4 ? (float *)dk : (float *)(ws + wl.acc);
    float *dv_acc = S::kBytes == 4 ? (float *)dv : dk_acc + n;
    // Two sides that do not read what the other writes: tap table -> dq on the caller's stream, and clears ->
    // (lse, delta) pairs -> binning (-> list ordering) -> dk/dv on the side lane. Forked before anything is
    // enqueued; joined after the dk/dv kernel (before the casts of 16-bit storage, which need both).
    // Only for shapes on the staged dq kernel, whose one 16-wave workgroup per CU leaves half the wave slots
    // free. The gather dq kernel (planes too large for LDS) fills every CU with small workgroups: beside it the
    // binning workgroups (1024 threads, up to 135 KB of LDS) wait until it ends, and with the binning done
    // first the dq and dk/dv kernels only take turns (measured at 64x64, D = 128: 14.2 ms against 14.5 for the
    // step, each kernel stretched to the sum of both) -- those shapes run the backward on the caller's stream.
    // So do small problems: the fork and join cost about 0.05 ms of host time per call, which a backward of
    // under two million query*samples (0.15 ms of kernels) does not win back.
    hipStream_t bst = st;
    const bool worth_forking = (long long)dm.rows * dm.N >= (2ll << 20);
    SideLane *side = cell_binned && staged && worth_forking && !(flags & DSDPA_FLAG_SINGLE_STREAM) ? side_lane() : nullptr;
    const size_t ncounters = cell_binned ? wl.counters_bytes / 4 : 0;
    SideJoin joiner;
    if (side && hipEventRecord(side->fork, st) == hipSuccess &&
        hipStreamWaitEvent(side->stream, side->fork, 0) == hipSuccess) {
        bst = side->stream;
        joiner.side = side;
        joiner.main = st;
        joiner.pending = true;
    }
    const bool side_on = bst != st;
    const size_t ndc = dcoords ? (size_t)dm.B * dm.V * dm.L * dm.N * 2 : 0;
    // what has to start at zero: on one stream everything in one job, which the tap-table launch (when
    // there is one) takes along; with the side lane the dk/dv side clears its own buffers there
    const ZeroJob zero_all{{dk_acc, dv_acc, (float *)(ws + wl.counters), dcoords}, {n, n, ncounters, ndc}};
    const ZeroJob zero_main{{dcoords, nullptr, nullptr, nullptr}, {ndc, 0, 0, 0}};
    const ZeroJob &zero = side_on ? zero_main : zero_all;
    if (staged) rc = launch_plane_descriptors(coords, dm, ws + wl.desc, wl.dl, cg_table, zero, 4, st);
    else if (!side_on || ndc) rc = zero_fill(zero, st);
    if (rc != DSDPA_OK) return rc;
    if (side_on) {
        // the dk/dv side: its clears, and the (lse, delta) pairs that the dq kernel otherwise writes on the way
        const ZeroJob zero_side{{dk_acc, dv_acc, (float *)(ws + wl.counters), nullptr}, {n, n, ncounters, 0}};
        if ((rc = zero_fill(zero_side, bst)) != DSDPA_OK) return rc;
        const size_t lanes = (size_t)dm.rows * 4;
        hipLaunchKernelGGL((delta_kernel<S>), dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, bst, out, dout, lse,
                           stats, (size_t)dm.rows, D);
        if ((rc = check_launch()) != DSDPA_OK) return rc;
    }
    if (cell_binned && (rc = launch_binning(coords, dm, wl, ws, deterministic ? 0 : 1, bst)) != DSDPA_OK) return rc;
    if (deterministic && (rc = launch_list_ordering(dm, wl, ws, bst)) != DSDPA_OK) return rc;
    float2 *dq_stats = side_on ? nullptr : stats;       // the dq kernel writes them only when dk/dv runs behind it
    // With the pairs handed over the two kernels go group by group of (batch, head) pairs: the buffer holds one
    // group's pairs (workspace_layout), and the dk/dv kernel of a group finds them where the dq kernel of the same
    // group has just left them. Otherwise one launch each covers all pairs.
    const int nbh_all = dm.B * dm.H, bh_step = handed ? wl.bh_group : nbh_all;
    const bool slab = path == DSDPA_PATH_AUTO && !staged && slab_path_fits(V, Himg, Wimg, D, P, S::kBytes);
#define DSDPA_BWD_CASE(DD)                                                                                      \
    case DD:                                                                                                    \
        if (fused_atomics && !dcoords) {                                                                        \
            rc = launch_bwd_gather<S, DD>(q, k, v, coords, out, lse, dout, dq, dk_acc, dv_acc, dm, st);         \
            break;                                                                                              \
        }                                                                                                       \
        for (int bh0 = 0; bh0 < nbh_all && rc == DSDPA_OK; bh0 += bh_step) {                                    \
            const int nbh = bh_step < nbh_all - bh0 ? bh_step : nbh_all - bh0;                                  \
            rc = staged ? launch_bwd_dq_plane<S, DD>(q, k, v, desc_w, desc_e, out, lse, dout, dq, dq_stats,     \
                                                     desc_g, dcoords, dm, st)                                   \
                 : slab ? launch_bwd_dq_slab<S, DD>(q, k, v, coords, out, lse, dout, dq, dq_stats, handed, dcoords,\
                                                    dm, bh0, nbh, st)                                           \
                        : launch_bwd_dq_gather<S, DD>(q, k, v, coords, out, lse, dout, dq, dq_stats, dcoords,   \
                                                      handed, dm, bh0, nbh, st);                                \
            if (rc == DSDPA_OK && cell_binned)                                                                  \
                rc = launch_bwd_dkdv_cell<S, DD>(q, k, v, coords, stats, dout, start, sorted, records,          \
                                                 (const uint4 *)(ws + wl.items), wl.wmax, handed, dk_acc,       \
                                                 dv_acc, dm, wl.NK, deterministic, bh0, nbh, bst);              \
            else if (rc == DSDPA_OK)                                                                            \
                rc = launch_bwd_dkdv_tile<S, DD>(q, k, v, coords, stats, dout, dk_acc, dv_acc, dm, st);         \
        }                                                                                                       \
        if (rc == DSDPA_OK) rc = joiner.join();                                                                 \
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

}  // namespace dsdpa
