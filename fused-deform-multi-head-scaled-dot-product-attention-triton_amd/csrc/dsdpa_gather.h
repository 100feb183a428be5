// "Gather" kernels: K/V taps are read straight from global memory (served by
// the XCD's L2), for shapes whose per-view K/V planes do not fit in LDS.
//
// Work split: one 64-lane wave per query row (b, s1, h, l). The wave is cut
// into NS = 64/G "slots" of G = D/DC adjacent lanes; a slot handles one sample
// at a time and its G lanes hold DC consecutive head-dim elements each, so the
// four taps of a sample are four (two when the taps are side by side)
// contiguous D-element runs read with 16-byte loads. Samples are taken 64 at a
// time: every lane first turns one coordinate pair into a tap descriptor
// (4 weights + 4 element offsets) and parks it in LDS, then the slots walk the
// 64 descriptors. Softmax is online per 64-sample chunk and per slot; slots
// are merged once per query row.
#pragma once
#include "dsdpa_common.h"

namespace dsdpa {

constexpr int kGatherWaves = 4;   // waves (= query rows) per workgroup

struct RowCtx {
    size_t row;        // linear query row in [B][V][H][L] (out, lse, dout, dq)
    size_t q_off;      // element offset of the query row in q
    size_t kv_base;    // element offset of plane (b, view 0, h) in k and v
    size_t acc_base;   // the same in the contiguous dk/dv accumulators
    size_t crow;       // float2 offset of coords[b][s1][l][0][0]
    int view_stride;   // elements between consecutive views of one (b, h) in k and v
};

// Logical work item -> query row; order (b, h, s1, l), l fastest, so that
// neighbouring work items share the K/V planes of one (b, h).
__device__ __forceinline__ RowCtx decode_row(int work, const Dims &dm, int D)
{
    int l = work % dm.L;
    int t = work / dm.L;
    int s1 = t % dm.V;
    t /= dm.V;
    int h = t % dm.H;
    int b = t / dm.H;
    RowCtx c;
    c.row = (((size_t)b * dm.V + s1) * dm.H + h) * dm.L + l;
    c.q_off = dm.q_row(b, s1, h, l);
    c.kv_base = dm.kv_plane(b, 0, h);
    c.acc_base = ((size_t)b * dm.V * dm.H + h) * (size_t)dm.L * D;
    c.crow = (((size_t)b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
    c.view_stride = dm.kv_sv;
    return c;
}

// Each lane builds the descriptor of sample c0+lane and parks it in this wave's LDS slice: the four
// weights and the four taps' BYTE offsets from plane (b, view 0, h), unsigned 32-bit (one batch item of a
// tensor stays below 2^30 elements, so below 2^32 bytes). With a wave-uniform base pointer a gather is then
// "scalar base + 32-bit lane offset", one add per tap instead of 64-bit address arithmetic.
template <int D, int BYTES>
__device__ __forceinline__ void park_descriptors(const Taps &tp, bool valid, int nc, const RowCtx &rc,
                                                 const Dims &dm, int lane, float4 *s_w, uint4 *s_e)
{
    int ebase = (nc / dm.P) * rc.view_stride;
    float4 w = valid ? make_float4(tp.w[0], tp.w[1], tp.w[2], tp.w[3]) : make_float4(0.f, 0.f, 0.f, 0.f);
    uint4 e = make_uint4((unsigned)(ebase + tp.pix[0] * dm.kv_sl) * BYTES, (unsigned)(ebase + tp.pix[1] * dm.kv_sl) * BYTES,
                         (unsigned)(ebase + tp.pix[2] * dm.kv_sl) * BYTES, (unsigned)(ebase + tp.pix[3] * dm.kv_sl) * BYTES);
    wave_lds_sync();          // the previous chunk's readers are done
    s_w[lane] = w;
    s_e[lane] = e;
    wave_lds_sync();
}

template <int D, int BYTES>
__device__ __forceinline__ void stage_descriptors(const float2 *__restrict__ coords, const RowCtx &rc,
                                                  const Dims &dm, int c0, int lane,
                                                  float4 *s_w, uint4 *s_e)
{
    int n = c0 + lane;
    bool valid = n < dm.N;
    int nc = valid ? n : dm.N - 1;
    float2 xy = coords[rc.crow + nc];
    Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
    park_descriptors<D, BYTES>(tp, valid, nc, rc, dm, lane, s_w, s_e);
}

// ------------------------------------------------------------------ window mode
// When the samples of a chunk (up to 64 samples of one query row, all in one key view) fall into a small
// window of the image -- deformable sampling around a reference point does -- the chunk is worked on per
// PIXEL of the window instead of per tap: one q.K[pixel] dot product per pixel, each sample's logit blended
// from four of those scalars, the softmax weights times the bilinear weights scattered into one
// coefficient per pixel, and one multiply-add of V[pixel] per pixel. A window of w x h pixels costs w*h
// rows of K and of V, read as contiguous runs, where the taps cost 4 per sample: about 120 against 256 for
// 64 samples with a standard deviation of two pixels. Chosen per chunk, from the bounding box of its taps.
//
// The window is laid out in UNITS of four pixels that are neighbours in a row: its rows are padded to a whole
// number of units, and it is moved left where that would cross the right edge of the image, so every pixel
// of every unit lies inside the image. Tables are indexed by entry = (row - ymin) * 4 * nu + (column - xmin).
// Only the pixels that some tap of the chunk touches are worked on, four at a time ("quads", see
// window_quads): of the 134 pixels of the padded box of such a chunk, 72 on average.
constexpr int kWinUnits = 56;                  // units per window: a window is taken only while 8 * units <= 7 * samples
                                               // (the work goes with the touched pixels, the tables with the box):
                                               // the tables of a wave hold 224 pixels
constexpr int kWinEntries = 4 * kWinUnits;
constexpr int kWinDummy = kWinEntries;         // table entry of the padding pixels of the last quad (a place of its own)

struct Window { int xmin, ymin, nu, nunits; };     // wave-uniform; nu = units per window row

// Bounding box of the clamped tap pixels of the lanes with `counted` set (a live sample with a tap inside the
// image), as padded units. Needs Wimg, Himg < 65536. nunits = 0: no window (the image is narrower than
// the padded rows).
__device__ __forceinline__ Window chunk_window(const Taps &tp, bool counted, int Wimg, int Himg)
{
    const int cx0 = min(max(tp.x0, 0), Wimg - 1), cx1 = min(max(tp.x0 + 1, 0), Wimg - 1);
    const int cy0 = min(max(tp.y0, 0), Himg - 1), cy1 = min(max(tp.y0 + 1, 0), Himg - 1);
    uint32_t lo = counted ? (uint32_t)cx0 | ((uint32_t)cy0 << 16) : 0xffffffffu;
    uint32_t hi = counted ? (uint32_t)(0xffff - cx1) | ((uint32_t)(0xffff - cy1) << 16) : 0xffffffffu;
    lo = __builtin_amdgcn_readfirstlane(wave_min_u16x2(lo));
    hi = __builtin_amdgcn_readfirstlane(wave_min_u16x2(hi));
    Window w;
    int xmax = 0, ymax = 0;
    w.xmin = 0;
    w.ymin = 0;
    if (lo != 0xffffffffu) {                   // else: no sample has a tap inside the image; any one unit will do
        w.xmin = (int)(lo & 0xffffu);
        w.ymin = (int)(lo >> 16);
        xmax = 0xffff - (int)(hi & 0xffffu);
        ymax = 0xffff - (int)(hi >> 16);
    }
    w.nu = (xmax - w.xmin + 4) >> 2;
    w.xmin = min(w.xmin, Wimg - 4 * w.nu);
    w.nunits = w.xmin >= 0 ? w.nu * (ymax - w.ymin + 1) : 0;
    return w;
}

// The four taps' entries in the window's tables (clamped pixels: inside the window whenever the sample
// counts; the others carry weight 0 and are only kept inside the tables).
__device__ __forceinline__ int4 window_entries(const Taps &tp, const Window &win, int Wimg, int Himg)
{
    const int cx0 = min(max(tp.x0, 0), Wimg - 1) - win.xmin, cx1 = min(max(tp.x0 + 1, 0), Wimg - 1) - win.xmin;
    const int cy0 = (min(max(tp.y0, 0), Himg - 1) - win.ymin) * 4 * win.nu;
    const int cy1 = (min(max(tp.y0 + 1, 0), Himg - 1) - win.ymin) * 4 * win.nu;
    const int last = 4 * win.nunits - 1;
    return make_int4(min(max(cy0 + cx0, 0), last), min(max(cy0 + cx1, 0), last), min(max(cy1 + cx0, 0), last),
                     min(max(cy1 + cx1, 0), last));
}

// The touched pixels of the window, compacted into quads. te: this lane's four table entries (every lane has
// four, the clamped taps of weight 0 included, so that every entry a sample reads is among the touched).
// Lane i looks after unit i: a bitmap in LDS tells which of its four pixels are touched, ballots rank them
// (pixel k of all units before pixel k+1), and the lane writes each one's byte offset from plane (b, view 0, h)
// to q_off[rank] and its table entry to q_ent[rank]. The last quad is padded with the window's first pixel
// (inside the image) and the dummy entry. Returns the number of quads (wave-uniform).
__device__ __forceinline__ int window_quads(const Window &win, const int4 &te, int lane, int Wimg, unsigned view_byte,
                                            float rnu, unsigned px_bytes, unsigned *bm, unsigned *q_off,
                                            unsigned *q_ent)
{
    if (lane < kWinEntries / 32) bm[lane] = 0u;
    wave_lds_sync();
    atomicOr(&bm[te.x >> 5], 1u << (te.x & 31));
    atomicOr(&bm[te.y >> 5], 1u << (te.y & 31));
    atomicOr(&bm[te.z >> 5], 1u << (te.z & 31));
    atomicOr(&bm[te.w >> 5], 1u << (te.w & 31));
    wave_lds_sync();
    const unsigned nib = lane < win.nunits ? (bm[lane >> 3] >> ((lane & 7) * 4)) & 0xFu : 0u;
    const int wy = (int)(((float)lane + 0.5f) * rnu);          // lane / nu: exact for these small numbers
    const int wxu = lane - wy * win.nu;
    const unsigned first = view_byte + (unsigned)((win.ymin + wy) * Wimg + win.xmin + 4 * wxu) * px_bytes;
    int total = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const bool set = ((nib >> k) & 1u) != 0u;
        const unsigned long long mask = __ballot(set);
        const int rank = total + (int)__builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32),
                                                                __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
        if (set) {
            q_off[rank] = first + (unsigned)k * px_bytes;
            q_ent[rank] = (unsigned)(4 * lane + k);
        }
        total += __popcll(mask);
    }
    const int nquads = (total + 3) >> 2;
    if (lane < 4 * nquads - total) {
        q_off[total + lane] = view_byte + (unsigned)(win.ymin * Wimg + win.xmin) * px_bytes;
        q_ent[total + lane] = (unsigned)kWinDummy;
    }
    wave_lds_sync();
    return nquads;
}

// x.row for the four pixels of this slot's quad (byte offsets o[k], this lane's part of the row included), summed
// over the slot.
template <typename S, int DC, int G>
__device__ __forceinline__ void window_dots(const char *__restrict__ base, const unsigned (&o)[4],
                                            const float (&xf)[DC], const uint32_t *xp, float (&d)[4])
{
    if constexpr (S::kBytes == 2) {
        uint32_t r[4][DC / 2];
#pragma unroll
        for (int k = 0; k < 4; ++k) load_packed<S, DC>(base + o[k], r[k]);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < DC / 2; ++i) {
                if constexpr (S::kBf16)
                    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(dsdpa_bf16x2, xp[i]),
                                                          __builtin_bit_cast(dsdpa_bf16x2, r[k][i]), acc, false);
                else
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(dsdpa_f16x2, xp[i]),
                                                 __builtin_bit_cast(dsdpa_f16x2, r[k][i]), acc, false);
            }
            d[k] = acc;
        }
    } else {
        float r[4][DC];
#pragma unroll
        for (int k = 0; k < 4; ++k) load_chunk<S, DC>(base + o[k], r[k]);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float acc = 0.f;
#pragma unroll
            for (int e = 0; e < DC; ++e) acc = fmaf(xf[e], r[k][e], acc);
            d[k] = acc;
        }
    }
    if constexpr (G > 0) {
#pragma unroll
        for (int k = 0; k < 4; ++k) d[k] = group_sum<G>(d[k]);
    }
}

// Sums over the 16 lanes of a slot of EIGHT values per lane, a[0..3] and b[0..3], by reduce-scatter: a step adds two
// halves of the slot and leaves each half with half of the values, so that the steps cost 8 + 4 + 2 + 2 instructions
// where butterflies over all eight values cost 32. The first two steps are vector adds whose first operand comes
// from the partner lane (row rotation by 8, then by 4 up or down) and whose bank mask -- a bank is four lanes -- makes
// them write one half of the lanes only: lanes 0-7 of the slot take a, lanes 8-15 take b; then banks 0 and 2 take
// values 0 and 1, banks 1 and 3 values 2 and 3. The last two steps are butterflies inside the banks. Afterwards
// lane 4j + i holds in (r0, r1): j = 0: (a0, a1), j = 1: (a2, a3), j = 2: (b0, b1), j = 3: (b2, b3), summed.
// (A rotation by N hands lane i the value of lane (i - N) mod 16. The s_nop covers the two wait states between a
// vector instruction's write and a cross-lane read of the same register.)
__device__ __forceinline__ void slot16_sums(const float (&a)[4], const float (&b)[4], float &r0, float &r1)
{
    float h0, h1, h2, h3;
    asm volatile("s_nop 1\n\t"
                 "v_add_f32_dpp %0, %4, %4 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                 "v_add_f32_dpp %1, %5, %5 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                 "v_add_f32_dpp %2, %6, %6 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                 "v_add_f32_dpp %3, %7, %7 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                 "v_add_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %1, %9, %9 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %2, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %3, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc"
                 : "=&v"(h0), "=&v"(h1), "=&v"(h2), "=&v"(h3)
                 : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]));
    float q0, q1;
    asm volatile("s_nop 1\n\t"
                 "v_add_f32_dpp %0, %2, %2 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
                 "v_add_f32_dpp %1, %3, %3 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
                 "v_add_f32_dpp %0, %4, %4 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
                 "v_add_f32_dpp %1, %5, %5 row_ror:4 row_mask:0xf bank_mask:0xa"
                 : "=&v"(q0), "=&v"(q1)
                 : "v"(h0), "v"(h1), "v"(h2), "v"(h3));
    r0 = group_sum<4>(q0);
    r1 = group_sum<4>(q1);
}

// The same with EIGHT lanes per pixel (16-bit storage, rows of 16 lanes): lane g2 of a slot takes DC elements of
// each half of the row (bytes o[k] + h * HALF, o[k] with the lane's offset inside a half included), so a step of the
// wave covers eight quads instead of four with three lane sums per product instead of four, and a chunk's
// pixels take about half as many steps. xp[h]: x's elements of the same two places.
template <typename S, int DC, int HALF>
__device__ __forceinline__ void window_dots_half(const char *__restrict__ base, const unsigned (&o)[4],
                                                 const uint32_t (&xp)[2][DC / 2], float (&d)[4])
{
    uint32_t r[4][2][DC / 2];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        load_packed<S, DC>(base + o[k], r[k][0]);
        load_packed<S, DC>(base + o[k] + HALF, r[k][1]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float acc = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < DC / 2; ++i) {
                if constexpr (S::kBf16)
                    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(dsdpa_bf16x2, xp[h][i]),
                                                          __builtin_bit_cast(dsdpa_bf16x2, r[k][h][i]), acc, false);
                else
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(dsdpa_f16x2, xp[h][i]),
                                                 __builtin_bit_cast(dsdpa_f16x2, r[k][h][i]), acc, false);
            }
        }
        d[k] = group_sum<8>(acc);
    }
}

// Bilinear blend of the four taps of one sample, this lane's DC elements. `e`: the taps' byte offsets from
// the (uniform) base, this lane's part of the row included.
template <typename S, int DC>
__device__ __forceinline__ void blend_taps(const char *__restrict__ base, const uint4 &e, const float4 &w,
                                           float (&dst)[DC])
{
    float t0[DC], t1[DC], t2[DC], t3[DC];
    load_chunk<S, DC>(base + e.x, t0);
    load_chunk<S, DC>(base + e.y, t1);
    load_chunk<S, DC>(base + e.z, t2);
    load_chunk<S, DC>(base + e.w, t3);
#pragma unroll
    for (int d = 0; d < DC; ++d)
        dst[d] = fmaf(w.x, t0[d], fmaf(w.y, t1[d], fmaf(w.z, t2[d], w.w * t3[d])));
}

// acc += sum_t c_t * tap_t for the four taps of one sample (no separate blend).
template <typename S, int DC>
__device__ __forceinline__ void accumulate_taps(const char *__restrict__ base, const uint4 &e, const float4 &c,
                                                float (&acc)[DC])
{
    float t0[DC], t1[DC], t2[DC], t3[DC];
    load_chunk<S, DC>(base + e.x, t0);
    load_chunk<S, DC>(base + e.y, t1);
    load_chunk<S, DC>(base + e.z, t2);
    load_chunk<S, DC>(base + e.w, t3);
#pragma unroll
    for (int d = 0; d < DC; ++d)
        acc[d] = fmaf(c.x, t0[d], fmaf(c.y, t1[d], fmaf(c.z, t2[d], fmaf(c.w, t3[d], acc[d]))));
}

// ------------------------------------------------------------------ forward
// WIN: chunks are cut per key view (up to 64 samples of one view each) and every chunk may take the window
// mode above; chosen by the host for P >= 64, where a view's samples fill whole chunks. Without WIN the
// chunks are 64 consecutive samples of the row, whatever views they belong to, and always gather.
template <typename S, int D, int DC, bool WIN>
__global__ __launch_bounds__(kGatherWaves *kWave, (WIN && DC <= 8) ? 4 : 1) void fwd_gather_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, void *__restrict__ out_, float *__restrict__ lse_,
    const unsigned char *__restrict__ todo_, int ntl, Dims dm)
{
    constexpr int G = D / DC;        // lanes per sample
    constexpr int NS = kWave / G;    // samples in flight per wave
    constexpr int ITS = G;           // slot iterations per 64-sample chunk
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    __shared__ float4 s_w[kGatherWaves][kWave];
    __shared__ uint4 s_e[kGatherWaves][kWave];
    constexpr int kTab = WIN ? kGatherWaves : 1, kTabUnits = WIN ? kWinUnits : 1;
    __shared__ __attribute__((aligned(16))) float s_dot[kTab][4 * kTabUnits + 4];     // window mode: q.K per pixel (+ the dummy entry)
    __shared__ __attribute__((aligned(16))) double s_coef[kTab][4 * kTabUnits + 4];   // window mode: coefficient of V per pixel
    __shared__ uint4 s_blend[kTab][2 * kTabUnits];                                  // ... per quad, as the V pass reads them
    __shared__ __attribute__((aligned(16))) unsigned s_qoff[kTab][4 * kTabUnits + 4]; // window mode: byte offsets of the quads' pixels
    __shared__ __attribute__((aligned(16))) unsigned s_qent[kTab][4 * kTabUnits + 4]; // ... and their table entries
    __shared__ unsigned s_bitmap[kTab][kWinEntries / 32];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    const int work = xcd_logical_block(blockIdx.x, gridDim.x) * kGatherWaves + wave;
    if (work >= dm.rows) return;
    // todo_ (may be null): one flag per tile of 16 consecutive pixels of a (b, h, s1), ntl tiles each; a tile
    // whose flag is 0 has been worked on by fwd_dense_kernel
    if (todo_) {
        const int bhs = work / dm.L, l = work - bhs * dm.L;
        if (!todo_[(size_t)bhs * ntl + (l >> 4)]) return;
    }
    const RowCtx rc = decode_row(work, dm, D);
    const int g = lane % G, slot = lane / G, lane_elem = g * DC;
    const unsigned lane_byte = (unsigned)lane_elem * S::kBytes;
    const char *kb = (const char *)k_ + rc.kv_base * S::kBytes;
    const char *vb = (const char *)v_ + rc.kv_base * S::kBytes;
    const float2 *coords = (const float2 *)coords_;

    // fp32 storage: q widened and pre-scaled; 16-bit storage: q kept as packed pairs for the dot-product
    // instructions and the scale applied to the logit
    constexpr bool kPacked = S::kBytes == 2;
    float qf[DC];
    uint32_t qp[kPacked ? DC / 2 : 1];
    const float qscale = dm.sm_scale * kLog2e;
    if constexpr (kPacked) {
        load_packed<S, DC>((const char *)q_ + (rc.q_off + lane_elem) * S::kBytes, qp);
    } else {
        load_chunk<S, DC>((const char *)q_ + (rc.q_off + lane_elem) * S::kBytes, qf);
#pragma unroll
        for (int d = 0; d < DC; ++d) qf[d] *= qscale;
    }

    // window chunks with 16 lanes per row take their dot products with 8 lanes per pixel (window_dots_half); the
    // q row is kept in LDS for that and read in that layout per chunk (no registers to spare for it between chunks)
    constexpr bool kHalf = WIN && kPacked && G == 16;
    constexpr unsigned kHalfBytes = D * S::kBytes / 2;
    __shared__ uint4 s_xq[kHalf ? kGatherWaves : 1][kHalf ? D / 8 : 1];
    if constexpr (kHalf) {
        if (lane < D / 8) s_xq[wave][lane] = reinterpret_cast<const uint4 *>((const char *)q_ + rc.q_off * S::kBytes)[lane];
    }

    float m = kNegBig, lsum = 0.f, acc[DC];
#pragma unroll
    for (int d = 0; d < DC; ++d) acc[d] = 0.f;
    // WIN: m is kept the same in all slots from chunk to chunk, and the window chunks add their samples' weights
    // per lane to lwin (same reference m), summed over the wave once, after the last chunk
    float lwin = 0.f;
    (void)lwin;

    const bool window_ok = WIN && dm.Wimg < 65536 && dm.Himg < 65536;
    const int view_chunks = (dm.P + kWave - 1) / kWave;
    const int nchunks = WIN ? dm.V * view_chunks : (dm.N + kWave - 1) / kWave;
    int next_view = 0, next_p0 = 0;                      // WIN: key view and first sample in it of the next chunk
    // the coordinates of a chunk are requested a chunk ahead (they come from HBM, once each)
    float2 xy_next = coords[rc.crow + min(lane, min(kWave, WIN ? dm.P : dm.N) - 1)];
    for (int ci = 0; ci < nchunks; ++ci) {
        const int s2c = next_view, p0 = next_p0;         // WIN: this chunk's
        const int c0 = WIN ? s2c * dm.P + p0 : ci * kWave;
        const int cnt = WIN ? min(kWave, dm.P - p0) : min(kWave, dm.N - c0);
        if (WIN) {
            next_p0 += kWave;
            if (next_p0 >= dm.P) { next_p0 = 0; ++next_view; }
        }
        // this lane's sample of the chunk
        const bool live = lane < cnt;
        const int nc = c0 + (live ? lane : cnt - 1);
        const float2 xy = xy_next;
        {
            const int c0n = WIN ? next_view * dm.P + next_p0 : c0 + kWave;
            const int cntn = WIN ? min(kWave, dm.P - next_p0) : min(kWave, dm.N - c0n);
            xy_next = coords[rc.crow + min(c0n + min(lane, cntn - 1), dm.N - 1)];     // (after the last chunk: any valid one)
        }
        const Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
        if (window_ok) {                                 // (the chunk lies in one key view)
            const bool counted = live && ((tp.w[0] != 0.f) | (tp.w[1] != 0.f) | (tp.w[2] != 0.f) | (tp.w[3] != 0.f));
            const Window win = chunk_window(tp, counted, dm.Wimg, dm.Himg);
            if (win.nunits > 0 && win.nunits <= kWinUnits && 8 * win.nunits <= 7 * cnt) {
                const unsigned kRow = (unsigned)dm.kv_sl * S::kBytes;       // bytes between neighbouring pixels of K and V
                constexpr bool kBlock = kPacked && G >= 4;         // V rows blended by the block matrix instruction
                float *tS = s_dot[wave];
                double *tA = s_coef[wave];
                uint4 *tC = s_blend[wave];
                const float rnu = 1.0f / (float)win.nu;
                const unsigned view_byte = (unsigned)s2c * (unsigned)rc.view_stride * S::kBytes;
                // one q.K dot product per touched pixel of the window
                const int4 te = window_entries(tp, win, dm.Wimg, dm.Himg);
                const unsigned *q_off = s_qoff[wave], *q_ent = s_qent[wave];
                const int nquads = window_quads(win, te, lane, dm.Wimg, view_byte, rnu, kRow, s_bitmap[wave],
                                                s_qoff[wave], s_qent[wave]);
                if constexpr (kHalf) {
                    const unsigned lb2 = (unsigned)(lane & 7) * DC * S::kBytes;
                    uint32_t xq[2][DC / 2];
                    load_packed<S, DC>((const char *)s_xq[wave] + lb2, xq[0]);
                    load_packed<S, DC>((const char *)s_xq[wave] + lb2 + kHalfBytes, xq[1]);
                    for (int q0 = 0; q0 < nquads; q0 += 2 * NS) {
                        const int qd = min(q0 + (lane >> 3), nquads - 1);
                        const uint4 off = *reinterpret_cast<const uint4 *>(q_off + 4 * qd);
                        const uint4 ent = *reinterpret_cast<const uint4 *>(q_ent + 4 * qd);
                        const unsigned o[4] = { off.x + lb2, off.y + lb2, off.z + lb2, off.w + lb2 };
                        float d4[4];
                        window_dots_half<S, DC, kHalfBytes>(kb, o, xq, d4);
                        if ((lane & 7) == 0) {
                            tS[ent.x] = d4[0];
                            tS[ent.y] = d4[1];
                            tS[ent.z] = d4[2];
                            tS[ent.w] = d4[3];
                        }
                    }
                } else {
                    for (int q0 = 0; q0 < nquads; q0 += NS) {
                        const int qd = min(q0 + slot, nquads - 1);
                        const uint4 off = *reinterpret_cast<const uint4 *>(q_off + 4 * qd);
                        const uint4 ent = *reinterpret_cast<const uint4 *>(q_ent + 4 * qd);
                        const unsigned o[4] = { off.x + lane_byte, off.y + lane_byte, off.z + lane_byte, off.w + lane_byte };
                        float d4[4];
                        window_dots<S, DC, G>(kb, o, qf, qp, d4);
                        if (g == 0) {
                            tS[ent.x] = d4[0];
                            tS[ent.y] = d4[1];
                            tS[ent.z] = d4[2];
                            tS[ent.w] = d4[3];
                        }
                    }
                }
                if (lane == 0) tA[kWinDummy] = 0.0;
                for (int e = lane; e < 4 * win.nunits; e += kWave) tA[e] = 0.0;
                wave_lds_sync();
                // the samples, one per lane: logit from four of the pixel scalars, then the softmax bookkeeping
                // of the chunk with the one running maximum that all slots share
                const float w0 = live ? tp.w[0] : 0.f, w1 = live ? tp.w[1] : 0.f;
                const float w2 = live ? tp.w[2] : 0.f, w3 = live ? tp.w[3] : 0.f;
                float logit = fmaf(w0, tS[te.x], fmaf(w1, tS[te.y], fmaf(w2, tS[te.z], w3 * tS[te.w])));
                if constexpr (kPacked) logit *= qscale;
                const float m_new = fmaxf(m, wave_max(live ? logit : kNegBig));
                const float alpha = __builtin_amdgcn_exp2f(m - m_new);
                m = m_new;
                lsum *= alpha;
#pragma unroll
                for (int d = 0; d < DC; ++d) acc[d] *= alpha;
                const float p = live ? __builtin_amdgcn_exp2f(logit - m_new) : 0.f;
                lwin = fmaf(lwin, alpha, p);
                // coefficient of every pixel: sum over the samples of p times the tap's bilinear weight
                // (every lane adds all four: a tap of weight 0 or a lane beyond the chunk adds 0 to an entry of the tables)
                atomicAdd(&tA[te.x], (double)(p * w0));
                atomicAdd(&tA[te.y], (double)(p * w1));
                atomicAdd(&tA[te.z], (double)(p * w2));
                atomicAdd(&tA[te.w], (double)(p * w3));
                wave_lds_sync();
                // the coefficients of each quad in the form the V pass wants them (one quad per lane)
                if (lane < nquads) {
                    const uint4 ent = *reinterpret_cast<const uint4 *>(q_ent + 4 * lane);
                    const float c0 = (float)tA[ent.x], c1 = (float)tA[ent.y];
                    const float c2 = (float)tA[ent.z], c3 = (float)tA[ent.w];
                    if constexpr (kBlock) {
                        tC[2 * lane] = split_coefficients<S>(c0, c1, c2, c3);      // rows 0, 1: high and low parts
                        tC[2 * lane + 1] = make_uint4(0u, 0u, 0u, 0u);             // rows 2, 3
                    } else {
                        tC[2 * lane] = make_uint4(__float_as_uint(c0), __float_as_uint(c1), __float_as_uint(c2), __float_as_uint(c3));
                    }
                }
                wave_lds_sync();
                // one weighted sum of V rows per quad
                if constexpr (kBlock) {
                    floatx4 macc[DC];
                    // (the first step starts the sums from the instruction's constant 0: there is always one)
                    auto step = [&](int q0, auto first) {
                        const int qd = min(q0 + slot, nquads - 1);
                        const uint4 off = *reinterpret_cast<const uint4 *>(q_off + 4 * qd);
                        uint2 cf = reinterpret_cast<const uint2 *>(tC)[4 * qd + (lane & 3)];
                        if (q0 + slot >= nquads) cf = make_uint2(0u, 0u);
                        uint32_t r[4][DC / 2];
                        load_packed<S, DC>(vb + (off.x + lane_byte), r[0]);
                        load_packed<S, DC>(vb + (off.y + lane_byte), r[1]);
                        load_packed<S, DC>(vb + (off.z + lane_byte), r[2]);
                        load_packed<S, DC>(vb + (off.w + lane_byte), r[3]);
                        block_blend4<S, DC, decltype(first)::value>(r, __builtin_bit_cast(shortx4, cf), macc);
                    };
                    step(0, std::true_type{});
                    for (int q0 = NS; q0 < nquads; q0 += NS) step(q0, std::false_type{});
#pragma unroll
                    for (int d = 0; d < DC; ++d) acc[d] += macc[d][0] + macc[d][1];
                } else {
                    for (int q0 = 0; q0 < nquads; q0 += NS) {
                        const int qd = min(q0 + slot, nquads - 1);
                        const uint4 off = *reinterpret_cast<const uint4 *>(q_off + 4 * qd);
                        uint4 cu = tC[2 * qd];
                        if (q0 + slot >= nquads) cu = make_uint4(0u, 0u, 0u, 0u);
                        const float cf[4] = { __uint_as_float(cu.x), __uint_as_float(cu.y), __uint_as_float(cu.z), __uint_as_float(cu.w) };
                        float r[4][DC];
                        load_chunk<S, DC>(vb + (off.x + lane_byte), r[0]);
                        load_chunk<S, DC>(vb + (off.y + lane_byte), r[1]);
                        load_chunk<S, DC>(vb + (off.z + lane_byte), r[2]);
                        load_chunk<S, DC>(vb + (off.w + lane_byte), r[3]);
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
#pragma unroll
                            for (int d = 0; d < DC; ++d) acc[d] = fmaf(cf[k], r[k][d], acc[d]);
                        }
                    }
                }
                wave_lds_sync();
                continue;
            }
        }
        park_descriptors<D, S::kBytes>(tp, live, nc, rc, dm, lane, s_w[wave], s_e[wave]);
        float sv[ITS];
        float mc = kNegBig;
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            sv[it] = kNegBig;
            if (it * NS < cnt) {
                int j = it * NS + slot;
                float4 w = s_w[wave][j];
                const uint4 e = lane_offsets(s_e[wave][j], lane_byte);
                float dot = 0.f;
                if constexpr (kPacked) {
                    dot = qscale * tap_dot16<S, DC>(kb + e.x, kb + e.y, kb + e.z, kb + e.w, w, qp);
                } else {
                    float kk[DC];
                    blend_taps<S, DC>(kb, e, w, kk);
#pragma unroll
                    for (int d = 0; d < DC; ++d) dot = fmaf(qf[d], kk[d], dot);
                }
                dot = group_sum<G>(dot);
                sv[it] = (j < cnt) ? dot : kNegBig;
                mc = fmaxf(mc, sv[it]);
            }
        }
        const float m_new = fmaxf(m, mc);
        const float alpha = __builtin_amdgcn_exp2f(m - m_new);
        m = m_new;
        lsum *= alpha;
        if constexpr (WIN) lwin *= alpha;
#pragma unroll
        for (int d = 0; d < DC; ++d) acc[d] *= alpha;
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            if (it * NS < cnt) {
                int j = it * NS + slot;
                float p = (j < cnt) ? __builtin_amdgcn_exp2f(sv[it] - m) : 0.f;
                lsum += p;
                float4 w = s_w[wave][j];
                const uint4 e = lane_offsets(s_e[wave][j], lane_byte);
                float4 c = make_float4(p * w.x, p * w.y, p * w.z, p * w.w);
                accumulate_taps<S, DC>(vb, e, c, acc);
            }
        }
        if constexpr (WIN) {                             // back to one running maximum for all slots
            const float mu = wave_max(m);
            const float a = __builtin_amdgcn_exp2f(m - mu);
            m = mu;
            lsum *= a;
            lwin *= a;
#pragma unroll
            for (int d = 0; d < DC; ++d) acc[d] *= a;
        }
    }
    if constexpr (WIN) {
        const float lw = wave_sum(lwin);
        if (slot == 0) lsum += lw;
    }

    // merge the NS slots (each has its own running max / sum / accumulator)
#pragma unroll
    for (int off = G; off < kWave; off <<= 1) {
        float mo = __shfl_xor(m, off, kWave);
        float lo = __shfl_xor(lsum, off, kWave);
        float mn = fmaxf(m, mo);
        float a = __builtin_amdgcn_exp2f(m - mn), bsc = __builtin_amdgcn_exp2f(mo - mn);
        lsum = lsum * a + lo * bsc;
#pragma unroll
        for (int d = 0; d < DC; ++d) {
            float ao = __shfl_xor(acc[d], off, kWave);
            acc[d] = acc[d] * a + ao * bsc;
        }
        m = mn;
    }
    if (slot == 0) {
        const float inv = 1.0f / lsum;
#pragma unroll
        for (int d = 0; d < DC; ++d) acc[d] *= inv;
        store_chunk<S, DC>((char *)out_ + (rc.row * D + lane_elem) * S::kBytes, acc);
        if (g == 0) lse_[rc.row] = m + __log2f(lsum);
    }
}

// ------------------------------------------------------------------ backward
// dq is written directly; dk/dv contributions go to fp32 accumulators
// (dk_acc/dv_acc, same [B][V][H][L][D] layout) with hardware float atomics.
template <typename S, int D, int DC>
__global__ __launch_bounds__(kGatherWaves *kWave) void bwd_gather_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, const void *__restrict__ out_, const float *__restrict__ lse_,
    const void *__restrict__ dout_, void *__restrict__ dq_, float *__restrict__ dk_acc,
    float *__restrict__ dv_acc, Dims dm)
{
    constexpr int G = D / DC;
    constexpr int NS = kWave / G;
    constexpr int ITS = G;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    __shared__ float4 s_w[kGatherWaves][kWave];
    __shared__ uint4 s_e[kGatherWaves][kWave];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    const int work = xcd_logical_block(blockIdx.x, gridDim.x) * kGatherWaves + wave;
    if (work >= dm.rows) return;
    const RowCtx rc = decode_row(work, dm, D);
    const int g = lane % G, slot = lane / G, lane_elem = g * DC;
    const unsigned lane_byte = (unsigned)lane_elem * S::kBytes;
    const char *kb = (const char *)k_ + rc.kv_base * S::kBytes;
    const char *vb = (const char *)v_ + rc.kv_base * S::kBytes;
    float *dkb = dk_acc + rc.acc_base + lane_elem;        // (this kernel runs on contiguous k/v only: the taps'
    float *dvb = dv_acc + rc.acc_base + lane_elem;        //  offsets in k/v are then their offsets in dk/dv too)
    const float2 *coords = (const float2 *)coords_;

    float qf[DC], dof[DC], of[DC];
    const size_t roff = (rc.row * D + lane_elem) * S::kBytes;
    const size_t q_roff = (rc.q_off + lane_elem) * S::kBytes;
    load_chunk<S, DC>((const char *)q_ + q_roff, qf);
    load_chunk<S, DC>((const char *)dout_ + roff, dof);
    load_chunk<S, DC>((const char *)out_ + roff, of);
    // delta = dout . out  (the reference's _bwd_preprocess, fused here)
    float delta = 0.f;
#pragma unroll
    for (int d = 0; d < DC; ++d) delta = fmaf(dof[d], of[d], delta);
    delta = group_sum<G>(delta);
    const float qscale = dm.sm_scale * kLog2e;
    const float lse = lse_[rc.row];

    float dqa[DC];
#pragma unroll
    for (int d = 0; d < DC; ++d) dqa[d] = 0.f;

    for (int c0 = 0; c0 < dm.N; c0 += kWave) {
        stage_descriptors<D, S::kBytes>(coords, rc, dm, c0, lane, s_w[wave], s_e[wave]);
        const int cnt = min(kWave, dm.N - c0);
#pragma unroll 2
        for (int it = 0; it < ITS; ++it) {
            if (it * NS < cnt) {
                int j = it * NS + slot;
                float4 w = s_w[wave][j];
                const uint4 eb = s_e[wave][j];
                const uint4 e = lane_offsets(eb, lane_byte);
                float kk[DC], vv[DC];
                blend_taps<S, DC>(kb, e, w, kk);
                blend_taps<S, DC>(vb, e, w, vv);
                float dot = 0.f, dp = 0.f;
#pragma unroll
                for (int d = 0; d < DC; ++d) {
                    dot = fmaf(qf[d], kk[d], dot);
                    dp = fmaf(dof[d], vv[d], dp);
                }
                dot = group_sum<G>(dot);
                dp = group_sum<G>(dp);
                float p = (j < cnt) ? __builtin_amdgcn_exp2f(dot * qscale - lse) : 0.f;
                float ds = p * (dp - delta);
#pragma unroll
                for (int d = 0; d < DC; ++d) dqa[d] = fmaf(ds, kk[d], dqa[d]);
                const float dss = ds * dm.sm_scale;
                const float wt[4] = { w.x, w.y, w.z, w.w };
                const unsigned et[4] = { eb.x / S::kBytes, eb.y / S::kBytes, eb.z / S::kBytes, eb.w / S::kBytes };
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    if (wt[t] != 0.f) {
                        const float ck = wt[t] * dss, cv = wt[t] * p;
#pragma unroll
                        for (int d = 0; d < DC; ++d) {
                            atomicAdd(dkb + et[t] + d, ck * qf[d]);
                            atomicAdd(dvb + et[t] + d, cv * dof[d]);
                        }
                    }
                }
            }
        }
    }
    // sum dq over slots
#pragma unroll
    for (int off = G; off < kWave; off <<= 1) {
#pragma unroll
        for (int d = 0; d < DC; ++d) dqa[d] += __shfl_xor(dqa[d], off, kWave);
    }
    if (slot == 0) {
#pragma unroll
        for (int d = 0; d < DC; ++d) dqa[d] *= dm.sm_scale;
        store_chunk<S, DC>((char *)dq_ + roff, dqa);
    }
}

// ------------------------------------------------------------------ backward, dq only
// Same walk as bwd_gather_kernel without the dk/dv scatter: writes dq and the
// per-row delta = dout.out (consumed by the kernels that produce dk/dv).
//
// CG: also the gradient of the coordinates (the reference's fused operator returns None there,
// ops/triton.py:464; its eager operator gets it through grid_sample, ops/torch.py:14-15). With
// g_t = sm_scale*ds*(q.K_t) + p*(dout.V_t) per tap, dL/dx = sum_t (d w_t/dx) g_t, likewise y. The per-tap
// dot products replace the blend-then-dot of the plain kernel; a lane keeps partial sums over its DC
// elements, combines them with the (slot-uniform) ds, p and tap derivatives and only the two results
// are reduced over the slot. The H heads share the coordinates: float atomics into dcoords (zeroed by
// the caller of the kernel).
// WIN: chunks per key view and the window mode, as in the forward: q.K and dout.V per pixel of the window, each
// sample's logit and dp blended from those scalars, ds times the bilinear weights scattered into one coefficient
// per pixel, dq += coefficient * K[pixel] per pixel. With CG the per-pixel scalars are all the coordinate gradient
// needs as well: a sample's g_t is sm_scale*ds*(q.K) + p*(dout.V) of its tap's pixel, four table reads it has
// made already.
template <typename S, int D, int DC, bool CG, bool WIN>
__global__ __launch_bounds__(kGatherWaves *kWave, (WIN && !CG && DC <= 8) ? 4 : 1) void bwd_dq_gather_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, const void *__restrict__ out_, const float *__restrict__ lse_,
    const void *__restrict__ dout_, void *__restrict__ dq_, float2 *__restrict__ stats_,
    float *__restrict__ dcoords_, float2 *__restrict__ handed_, Dims dm, int work0, int work_end)
{
    constexpr int G = D / DC;
    constexpr int NS = kWave / G;
    constexpr int ITS = G;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    __shared__ float4 s_w[kGatherWaves][kWave];
    __shared__ uint4 s_e[kGatherWaves][kWave];
    __shared__ float4 s_gx[CG ? kGatherWaves : 1][CG ? kWave : 1];
    __shared__ float4 s_gy[CG ? kGatherWaves : 1][CG ? kWave : 1];
    __shared__ float2 s_hand[kGatherWaves][kWave];                               // (p, sm_scale * ds) of the chunk's samples
    constexpr int kTab = WIN ? kGatherWaves : 1, kTabUnits = WIN ? kWinUnits : 1;
    __shared__ __attribute__((aligned(16))) float s_dotk[kTab][4 * kTabUnits + 4];    // window mode: q.K per pixel (+ the dummy entry)
    __shared__ __attribute__((aligned(16))) float s_dotv[kTab][4 * kTabUnits + 4];    // window mode: dout.V per pixel
    __shared__ __attribute__((aligned(16))) double s_coef[kTab][4 * kTabUnits + 4];   // window mode: coefficient of K per pixel
    __shared__ uint4 s_blend[kTab][2 * kTabUnits];                                  // ... per quad, as the last pass reads them
    __shared__ __attribute__((aligned(16))) unsigned s_qoff[kTab][4 * kTabUnits + 4]; // window mode: byte offsets of the quads' pixels
    __shared__ __attribute__((aligned(16))) unsigned s_qent[kTab][4 * kTabUnits + 4]; // ... and their table entries
    __shared__ unsigned s_bitmap[kTab][kWinEntries / 32];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    // a launch covers the query rows [work0, work_end) of the (b, h, s1, l) order: a group of (batch, head) pairs
    const int work = work0 + xcd_logical_block(blockIdx.x, gridDim.x) * kGatherWaves + wave;
    if (work >= work_end) return;
    const RowCtx rc = decode_row(work, dm, D);
    const int g = lane % G, slot = lane / G, lane_elem = g * DC;
    const unsigned lane_byte = (unsigned)lane_elem * S::kBytes;
    const char *kb = (const char *)k_ + rc.kv_base * S::kBytes;
    const char *vb = (const char *)v_ + rc.kv_base * S::kBytes;
    const float2 *coords = (const float2 *)coords_;

    // 16-bit storage: packed pairs for the dot-product instructions -- in the window mode always, tap by tap only
    // without the coordinate gradient (whose per-tap products take the widened rows)
    constexpr bool kPackedWin = S::kBytes == 2 && WIN;
    constexpr bool kPacked = S::kBytes == 2 && !CG;
    float qf[DC], dof[DC], of[DC];
    uint32_t dop[(kPacked || kPackedWin) ? DC / 2 : 1], qp[kPackedWin ? DC / 2 : 1];
    const size_t roff = (rc.row * D + lane_elem) * S::kBytes;
    const size_t q_roff = (rc.q_off + lane_elem) * S::kBytes;
    load_chunk<S, DC>((const char *)q_ + q_roff, qf);
    load_chunk<S, DC>((const char *)dout_ + roff, dof);
    load_chunk<S, DC>((const char *)out_ + roff, of);
    if constexpr (kPacked || kPackedWin) load_packed<S, DC>((const char *)dout_ + roff, dop);
    if constexpr (kPackedWin) load_packed<S, DC>((const char *)q_ + q_roff, qp);
    float delta = 0.f;
#pragma unroll
    for (int d = 0; d < DC; ++d) delta = fmaf(dof[d], of[d], delta);
    delta = group_sum<G>(delta);
    const float qscale = dm.sm_scale * kLog2e;
    const float lse = lse_[rc.row];
    if (stats_ && lane == 0) stats_[rc.row] = make_float2(lse, delta);     // null: a launch of its own does it
    // handed_ (may be null): per sample, (p, sm_scale * ds) for the dk/dv kernel, which then need
    // not recompute them from the taps: [pair (b, h) of this launch][s1][l][sample], i.e. in the order of the work
    // items of this launch and, inside a row, of its coordinates
    float2 *handed_row = handed_ ? handed_ + (size_t)(work - work0) * dm.N : nullptr;

    float dqa[DC];
#pragma unroll
    for (int d = 0; d < DC; ++d) dqa[d] = 0.f;

    const bool window_ok = WIN && dm.Wimg < 65536 && dm.Himg < 65536;
    const int view_chunks = (dm.P + kWave - 1) / kWave;
    const int nchunks = WIN ? dm.V * view_chunks : (dm.N + kWave - 1) / kWave;
    int next_view = 0, next_p0 = 0;                      // WIN: key view and first sample in it of the next chunk
    // the coordinates of a chunk are requested a chunk ahead (they come from HBM, once each)
    float2 xy_next = coords[rc.crow + min(lane, min(kWave, WIN ? dm.P : dm.N) - 1)];
    for (int ci = 0; ci < nchunks; ++ci) {
        const int s2c = next_view, p0 = next_p0;         // WIN: this chunk's
        const int c0 = WIN ? s2c * dm.P + p0 : ci * kWave;
        const int cnt = WIN ? min(kWave, dm.P - p0) : min(kWave, dm.N - c0);
        if (WIN) {
            next_p0 += kWave;
            if (next_p0 >= dm.P) { next_p0 = 0; ++next_view; }
        }
        // this lane's sample of the chunk
        const bool live = lane < cnt;
        const int nc = c0 + (live ? lane : cnt - 1);
        const float2 xy0 = xy_next;
        {
            const int c0n = WIN ? next_view * dm.P + next_p0 : c0 + kWave;
            const int cntn = WIN ? min(kWave, dm.P - next_p0) : min(kWave, dm.N - c0n);
            xy_next = coords[rc.crow + min(c0n + min(lane, cntn - 1), dm.N - 1)];     // (after the last chunk: any valid one)
        }
        const Taps tp = make_taps(xy0.x, xy0.y, dm.Wimg, dm.Himg);
        if constexpr (WIN) {
            const bool counted = live && ((tp.w[0] != 0.f) | (tp.w[1] != 0.f) | (tp.w[2] != 0.f) | (tp.w[3] != 0.f));
            const Window win = window_ok ? chunk_window(tp, counted, dm.Wimg, dm.Himg) : Window{0, 0, 0, 0};
            if (win.nunits > 0 && win.nunits <= kWinUnits && 8 * win.nunits <= 7 * cnt) {
                const unsigned kRow = (unsigned)dm.kv_sl * S::kBytes;       // bytes between neighbouring pixels of K and V
                constexpr bool kBlock = kPackedWin && G >= 4;
                float *tS = s_dotk[wave], *tT = s_dotv[wave];
                double *tA = s_coef[wave];
                uint4 *tC = s_blend[wave];
                const float rnu = 1.0f / (float)win.nu;
                const unsigned view_byte = (unsigned)s2c * (unsigned)rc.view_stride * S::kBytes;
                // q.K and dout.V per touched pixel of the window
                const int4 te = window_entries(tp, win, dm.Wimg, dm.Himg);
                const unsigned *q_off = s_qoff[wave], *q_ent = s_qent[wave];
                const int nquads = window_quads(win, te, lane, dm.Wimg, view_byte, rnu, kRow, s_bitmap[wave],
                                                s_qoff[wave], s_qent[wave]);
                for (int q0 = 0; q0 < nquads; q0 += NS) {
                    const int qd = min(q0 + slot, nquads - 1);
                    const uint4 off = *reinterpret_cast<const uint4 *>(q_off + 4 * qd);
                    const uint4 ent = *reinterpret_cast<const uint4 *>(q_ent + 4 * qd);
                    const unsigned o[4] = { off.x + lane_byte, off.y + lane_byte, off.z + lane_byte, off.w + lane_byte };
                    float dk4[4], dv4[4];
                    if constexpr (G == 16) {
                        // the eight sums over the slot by reduce-scatter: every bank of four lanes ends up with two of
                        // them, which its first lane stores
                        window_dots<S, DC, 0>(kb, o, qf, qp, dk4);
                        window_dots<S, DC, 0>(vb, o, dof, dop, dv4);
                        float r0, r1;
                        slot16_sums(dk4, dv4, r0, r1);
                        float *tab = (g & 8) ? tT : tS;
                        const unsigned e0 = (g & 4) ? ent.z : ent.x, e1 = (g & 4) ? ent.w : ent.y;
                        if ((g & 3) == 0) { tab[e0] = r0; tab[e1] = r1; }
                    } else {
                        window_dots<S, DC, G>(kb, o, qf, qp, dk4);
                        window_dots<S, DC, G>(vb, o, dof, dop, dv4);
                        if (g == 0) {
                            tS[ent.x] = dk4[0]; tS[ent.y] = dk4[1]; tS[ent.z] = dk4[2]; tS[ent.w] = dk4[3];
                            tT[ent.x] = dv4[0]; tT[ent.y] = dv4[1]; tT[ent.z] = dv4[2]; tT[ent.w] = dv4[3];
                        }
                    }
                }
                if (lane == 0) tA[kWinDummy] = 0.0;
                for (int e = lane; e < 4 * win.nunits; e += kWave) tA[e] = 0.0;
                wave_lds_sync();
                // the samples, one per lane
                const float w0 = live ? tp.w[0] : 0.f, w1 = live ? tp.w[1] : 0.f;
                const float w2 = live ? tp.w[2] : 0.f, w3 = live ? tp.w[3] : 0.f;
                const float sk0 = tS[te.x], sk1 = tS[te.y], sk2 = tS[te.z], sk3 = tS[te.w];
                const float sv0 = tT[te.x], sv1 = tT[te.y], sv2 = tT[te.z], sv3 = tT[te.w];
                const float dot = fmaf(w0, sk0, fmaf(w1, sk1, fmaf(w2, sk2, w3 * sk3)));
                const float dp = fmaf(w0, sv0, fmaf(w1, sv1, fmaf(w2, sv2, w3 * sv3)));
                const float p = live ? __builtin_amdgcn_exp2f(dot * qscale - lse) : 0.f;
                const float ds = p * (dp - delta);
                if (handed_row && live) handed_row[nc] = make_float2(p, ds * dm.sm_scale);
                if constexpr (CG) {
                    // one sample per lane: the tap derivatives (zero for a tap outside the image, and for a dead
                    // lane through p = ds = 0) times g_t of the four pixels
                    const TapGrads tg = make_tap_grads(xy0.x, xy0.y, dm.Wimg, dm.Himg);
                    const float a = ds * dm.sm_scale;
                    const float g0 = fmaf(a, sk0, p * sv0), g1 = fmaf(a, sk1, p * sv1);
                    const float g2 = fmaf(a, sk2, p * sv2), g3 = fmaf(a, sk3, p * sv3);
                    if (live) {
                        float *dst = dcoords_ + 2 * (rc.crow + (size_t)nc);
                        atomicAdd(dst, fmaf(tg.gx[0], g0, fmaf(tg.gx[1], g1, fmaf(tg.gx[2], g2, tg.gx[3] * g3))));
                        atomicAdd(dst + 1, fmaf(tg.gy[0], g0, fmaf(tg.gy[1], g1, fmaf(tg.gy[2], g2, tg.gy[3] * g3))));
                    }
                }
                atomicAdd(&tA[te.x], (double)(ds * w0));
                atomicAdd(&tA[te.y], (double)(ds * w1));
                atomicAdd(&tA[te.z], (double)(ds * w2));
                atomicAdd(&tA[te.w], (double)(ds * w3));
                wave_lds_sync();
                if (lane < nquads) {
                    const uint4 ent = *reinterpret_cast<const uint4 *>(q_ent + 4 * lane);
                    const float c0f = (float)tA[ent.x], c1f = (float)tA[ent.y];
                    const float c2f = (float)tA[ent.z], c3f = (float)tA[ent.w];
                    if constexpr (kBlock) {
                        tC[2 * lane] = split_coefficients<S>(c0f, c1f, c2f, c3f);
                        tC[2 * lane + 1] = make_uint4(0u, 0u, 0u, 0u);
                    } else {
                        tC[2 * lane] = make_uint4(__float_as_uint(c0f), __float_as_uint(c1f), __float_as_uint(c2f), __float_as_uint(c3f));
                    }
                }
                wave_lds_sync();
                // dq += coefficient * K per touched pixel
                if constexpr (kBlock) {
                    floatx4 macc[DC];
                    // (the first step starts the sums from the instruction's constant 0: there is always one)
                    auto step = [&](int q0, auto first) {
                        const int qd = min(q0 + slot, nquads - 1);
                        const uint4 off = *reinterpret_cast<const uint4 *>(q_off + 4 * qd);
                        uint2 cf = reinterpret_cast<const uint2 *>(tC)[4 * qd + (lane & 3)];
                        if (q0 + slot >= nquads) cf = make_uint2(0u, 0u);
                        uint32_t r[4][DC / 2];
                        load_packed<S, DC>(kb + (off.x + lane_byte), r[0]);
                        load_packed<S, DC>(kb + (off.y + lane_byte), r[1]);
                        load_packed<S, DC>(kb + (off.z + lane_byte), r[2]);
                        load_packed<S, DC>(kb + (off.w + lane_byte), r[3]);
                        block_blend4<S, DC, decltype(first)::value>(r, __builtin_bit_cast(shortx4, cf), macc);
                    };
                    step(0, std::true_type{});
                    for (int q0 = NS; q0 < nquads; q0 += NS) step(q0, std::false_type{});
#pragma unroll
                    for (int d = 0; d < DC; ++d) dqa[d] += macc[d][0] + macc[d][1];
                } else {
                    for (int q0 = 0; q0 < nquads; q0 += NS) {
                        const int qd = min(q0 + slot, nquads - 1);
                        const uint4 off = *reinterpret_cast<const uint4 *>(q_off + 4 * qd);
                        uint4 cu = tC[2 * qd];
                        if (q0 + slot >= nquads) cu = make_uint4(0u, 0u, 0u, 0u);
                        const float cf[4] = { __uint_as_float(cu.x), __uint_as_float(cu.y), __uint_as_float(cu.z), __uint_as_float(cu.w) };
                        float r[4][DC];
                        load_chunk<S, DC>(kb + (off.x + lane_byte), r[0]);
                        load_chunk<S, DC>(kb + (off.y + lane_byte), r[1]);
                        load_chunk<S, DC>(kb + (off.z + lane_byte), r[2]);
                        load_chunk<S, DC>(kb + (off.w + lane_byte), r[3]);
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
#pragma unroll
                            for (int d = 0; d < DC; ++d) dqa[d] = fmaf(cf[k], r[k][d], dqa[d]);
                        }
                    }
                }
                wave_lds_sync();
                continue;
            }
        }
        park_descriptors<D, S::kBytes>(tp, live, nc, rc, dm, lane, s_w[wave], s_e[wave]);
        if constexpr (CG) {
            // (stage_descriptors ends with a wave-level LDS sync; these two arrays are read after the
            // next one, and their previous readers finished before the sync at its start)
            const TapGrads tg = make_tap_grads(xy0.x, xy0.y, dm.Wimg, dm.Himg);
            s_gx[wave][lane] = make_float4(tg.gx[0], tg.gx[1], tg.gx[2], tg.gx[3]);
            s_gy[wave][lane] = make_float4(tg.gy[0], tg.gy[1], tg.gy[2], tg.gy[3]);
            wave_lds_sync();
        }
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            if (it * NS < cnt) {
                int j = it * NS + slot;
                float4 w = s_w[wave][j];
                const uint4 e = lane_offsets(s_e[wave][j], lane_byte);
                float kk[DC];
                float dot = 0.f, dp = 0.f;
                if constexpr (CG) {
                    float t[4][DC], u[4][DC];
                    const unsigned eo[4] = { e.x, e.y, e.z, e.w };
                    const float wt[4] = { w.x, w.y, w.z, w.w };
                    float dk_t[4], dv_t[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        load_chunk<S, DC>(kb + eo[i], t[i]);
                        load_chunk<S, DC>(vb + eo[i], u[i]);
                    }
#pragma unroll
                    for (int d = 0; d < DC; ++d) kk[d] = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        dk_t[i] = 0.f;
                        dv_t[i] = 0.f;
#pragma unroll
                        for (int d = 0; d < DC; ++d) {
                            dk_t[i] = fmaf(qf[d], t[i][d], dk_t[i]);
                            dv_t[i] = fmaf(dof[d], u[i][d], dv_t[i]);
                            kk[d] = fmaf(wt[i], t[i][d], kk[d]);
                        }
                        dot = fmaf(wt[i], dk_t[i], dot);
                        dp = fmaf(wt[i], dv_t[i], dp);
                    }
                    dot = group_sum<G>(dot);
                    dp = group_sum<G>(dp);
                    const float p = (j < cnt) ? __builtin_amdgcn_exp2f(dot * qscale - lse) : 0.f;
                    const float ds = p * (dp - delta);
                    s_hand[wave][j] = make_float2(p, ds * dm.sm_scale);          // (all lanes of the slot: same value, same place)
#pragma unroll
                    for (int d = 0; d < DC; ++d) dqa[d] = fmaf(ds, kk[d], dqa[d]);
                    const float4 ax = s_gx[wave][j], ay = s_gy[wave][j];
                    const float a = ds * dm.sm_scale;
                    const float g0 = fmaf(a, dk_t[0], p * dv_t[0]), g1 = fmaf(a, dk_t[1], p * dv_t[1]);
                    const float g2 = fmaf(a, dk_t[2], p * dv_t[2]), g3 = fmaf(a, dk_t[3], p * dv_t[3]);
                    float gx = fmaf(ax.x, g0, fmaf(ax.y, g1, fmaf(ax.z, g2, ax.w * g3)));
                    float gy = fmaf(ay.x, g0, fmaf(ay.y, g1, fmaf(ay.z, g2, ay.w * g3)));
                    gx = group_sum<G>(gx);
                    gy = group_sum<G>(gy);
                    if (g == 0 && j < cnt) {
                        float *dst = dcoords_ + 2 * (rc.crow + (size_t)(c0 + j));
                        atomicAdd(dst, gx);
                        atomicAdd(dst + 1, gy);
                    }
                    continue;
                }
                blend_taps<S, DC>(kb, e, w, kk);
#pragma unroll
                for (int d = 0; d < DC; ++d) dot = fmaf(qf[d], kk[d], dot);
                if constexpr (kPacked) {
                    // dout . v~ needs no widened v~: four packed dot products on the raw taps
                    dp = tap_dot16<S, DC>(vb + e.x, vb + e.y, vb + e.z, vb + e.w, w, dop);
                } else {
                    float vv[DC];
                    blend_taps<S, DC>(vb, e, w, vv);
#pragma unroll
                    for (int d = 0; d < DC; ++d) dp = fmaf(dof[d], vv[d], dp);
                }
                dot = group_sum<G>(dot);
                dp = group_sum<G>(dp);
                float p = (j < cnt) ? __builtin_amdgcn_exp2f(dot * qscale - lse) : 0.f;
                float ds = p * (dp - delta);
                if constexpr (!CG) s_hand[wave][j] = make_float2(p, ds * dm.sm_scale);   // (all lanes of the slot: same value, same place)
#pragma unroll
                for (int d = 0; d < DC; ++d) dqa[d] = fmaf(ds, kk[d], dqa[d]);
            }
        }
        // the chunk's pairs, one sample per lane, in one coalesced store (plain stores and loads: streaming
        // ones keep the pairs out of L2, where the dk/dv kernel finds them: 2.44 -> 2.64 ms at 64x64, D = 128)
        if (handed_row) {
            wave_lds_sync();
            if (live) handed_row[c0 + lane] = s_hand[wave][lane];
            wave_lds_sync();
        }
    }
#pragma unroll
    for (int off = G; off < kWave; off <<= 1) {
#pragma unroll
        for (int d = 0; d < DC; ++d) dqa[d] += __shfl_xor(dqa[d], off, kWave);
    }
    if (slot == 0) {
#pragma unroll
        for (int d = 0; d < DC; ++d) dqa[d] *= dm.sm_scale;
        store_chunk<S, DC>((char *)dq_ + roff, dqa);
    }
}

}  // namespace dsdpa
