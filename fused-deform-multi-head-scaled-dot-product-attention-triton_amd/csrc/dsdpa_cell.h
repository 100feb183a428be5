// Cell-binned dk/dv: scatter turned into register accumulation.
//
// A sample's four bilinear taps are the 2x2 pixel block whose top-left pixel is
// (y0, x0) = floor of its pixel coordinate -- its "cell". Which cell a sample
// falls in depends on the coordinates only, not on the head, so one counting
// sort per (batch, key view) -- bin_count / bin_scan / bin_fill below -- orders
// the samples (s1, l, p) of every key view by cell, and all H heads reuse it.
//
// The dk/dv kernel then gives one wave to one (plane (b, h, s2), cell): the
// cell's four K and four V tap rows are loaded ONCE into registers; for every
// sample in the cell's list the wave gathers the sample's query row (q, dout,
// log-sum-exp, delta), recomputes p and ds, and adds w_t*ds*scale*q and
// w_t*p*dout into register accumulators for the four pixels. Only the cell's
// final sums go to memory: 8*D float atomics per non-empty cell instead of 8*D
// per sample (each pixel is shared by four cells, hence atomics for that last
// step). Heavy cells (clustered coordinates) are the best case, not the worst.
//
// Cells are indexed on a (Himg+1) x (Wimg+1) grid, y0 in [-1, Himg-1] and x0 in
// [-1, Wimg-1]: border cells hold the samples with some taps outside the image
// (weight 0 there, zero padding per tap). Samples with all four taps outside
// contribute nothing to dk/dv and are left out of the lists.
#pragma once
#include "dsdpa_common.h"

namespace dsdpa {

constexpr int kBinThreads = 256;
// Waves per workgroup of the dk/dv kernel. One: items differ in length by orders of magnitude (a heavy
// list's piece beside lists of a few entries), and a workgroup keeps its LDS and its place on the CU until
// its longest wave ends -- with four waves a workgroup the SIMDs held 2.1 waves on average where the
// registers allow 3 (64x64, 64 samples per view, clustered: 4.88 ms with four, 4.13 ms with one).
constexpr int kCellWaves = 1;

__device__ __forceinline__ int cell_of(const Taps &tp, int Wimg) { return (tp.y0 + 1) * (Wimg + 1) + (tp.x0 + 1); }

// Fractional position of a sample inside its cell: the bilinear weights are (1-fx)(1-fy), fx(1-fy), (1-fx)fy, fx*fy.
// The binning pass stores it beside the sample id (same order), so that the dk/dv kernel reads it in list order
// instead of gathering the coordinate pair again (a random 8-byte read per entry, per head).
__device__ __forceinline__ float2 cell_fraction(float2 xy, const Dims &dm)
{
    const float x = ((xy.x * 2.0f - 1.0f) + 1.0f) * ((float)(dm.Wimg - 1) * 0.5f);
    const float y = ((xy.y * 2.0f - 1.0f) + 1.0f) * ((float)(dm.Himg - 1) * 0.5f);
    return make_float2(x - floorf(x), y - floorf(y));
}

__device__ __forceinline__ bool taps_any(const Taps &tp)
{
    return (tp.w[0] != 0.f) | (tp.w[1] != 0.f) | (tp.w[2] != 0.f) | (tp.w[3] != 0.f);
}

// Lists are kept per key = (group of query views s1 / vpg, cell), NK = groups * NC keys per (batch, key view).
// With more than one group the dk/dv kernel works through a key view's lists one group of query views at a
// time, so that the query rows it gathers (q and dout of that group only) stay in the XCD's L2.
//
// One thread per coordinate pair, in memory order (b, s1, l, s2, p).
// mode 0: count[(b*V+s2)*NK + key] += 1
// mode 1: the sample's list entry at place (b*V+s2)*M + cursor[(b*V+s2)*NK + key]++: with `records` a 12-byte
//         record (id = (s1*L + l)*P + p, then its position (fx, fy) inside the cell as two floats) in `sorted` taken
//         as an array of records -- one scattered store per sample, and the dk/dv kernel reads id and position in
//         list order instead of gathering the coordinate pair again; without, the id alone as sorted[place] (the
//         deterministic backward sorts the ids of every list before use).
struct CellEntry { unsigned id; float fx, fy; };
__device__ __forceinline__ void store_cell_entry(unsigned *sorted, size_t place, unsigned id, const float2 &ff, int records)
{
    if (records) {
        unsigned *r = sorted + 3 * place;
        r[0] = id;
        r[1] = __float_as_uint(ff.x);
        r[2] = __float_as_uint(ff.y);
    } else {
        sorted[place] = id;
    }
}

template <int MODE>
__global__ __launch_bounds__(kBinThreads) void bin_samples_kernel(const float *__restrict__ coords_, Dims dm,
                                                                  int NC, int NK, int vpg,
                                                                  unsigned *__restrict__ counters,
                                                                  unsigned *__restrict__ sorted, int records)
{
    const long long total = (long long)dm.B * dm.V * dm.L * dm.N;
    const long long i = (long long)blockIdx.x * kBinThreads + threadIdx.x;
    if (i >= total) return;
    const float2 xy = reinterpret_cast<const float2 *>(coords_)[i];
    const Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
    if (!taps_any(tp)) return;
    const int p = (int)(i % dm.P);
    long long t = i / dm.P;
    const int s2 = (int)(t % dm.V);
    t /= dm.V;                                   // t = (b*V + s1)*L + l
    const int ql = (int)(t % ((long long)dm.V * dm.L));   // s1*L + l
    const int b = (int)(t / ((long long)dm.V * dm.L));
    const size_t grp = (size_t)b * dm.V + s2;
    unsigned *ctr = counters + grp * NK + (ql / dm.L / vpg) * NC + cell_of(tp, dm.Wimg);
    if (MODE == 0) {
        atomicAdd(ctr, 1u);
    } else {
        const unsigned pos = atomicAdd(ctr, 1u);
        const size_t M = (size_t)dm.V * dm.L * dm.P;
        store_cell_entry(sorted, grp * M + pos, (unsigned)ql * (unsigned)dm.P + (unsigned)p, cell_fraction(xy, dm), records);
    }
}

// LDS-aggregated variant of the two passes above, used when the V*NC counters of
// one batch item fit in LDS. A workgroup takes a contiguous run of query rows of
// one (b, s1) -- whose coordinates are one contiguous block covering all V key
// views -- and histograms it in LDS first, so the contended global atomics drop
// from one per sample to one per (workgroup, non-empty cell).
// mode 0: global count[cell] += local count
// mode 1: reserve [base, base+local count) from the global cursor of each cell,
//         then place every sample at base + its local rank.
constexpr int kBinLdsThreads = 1024;

template <int MODE>
__global__ __launch_bounds__(kBinLdsThreads) void bin_samples_lds_kernel(
    const float *__restrict__ coords_, Dims dm, int NC, int NK, int vpg, int lchunk, int nlc,
    unsigned *__restrict__ counters, unsigned *__restrict__ sorted, int records)
{
    extern __shared__ unsigned s_hist[];                 // [V][NC]; mode 1 adds [V][NC] bases
    unsigned *s_base = s_hist + (size_t)dm.V * NC;
    const int lc = blockIdx.x % nlc;
    const int s1 = (blockIdx.x / nlc) % dm.V;
    const int b = blockIdx.x / (nlc * dm.V);
    const int l0 = lc * lchunk, l1 = min(dm.L, l0 + lchunk);
    const int nhist = dm.V * NC;
    for (int i = threadIdx.x; i < nhist; i += kBinLdsThreads) s_hist[i] = 0u;
    __syncthreads();
    const float2 *crd = reinterpret_cast<const float2 *>(coords_) + (((size_t)b * dm.V + s1) * dm.L + l0) * dm.N;
    const int total = (l1 - l0) * dm.N;                  // samples of this workgroup, all key views
    for (int i = threadIdx.x; i < total; i += kBinLdsThreads) {
        const float2 xy = crd[i];
        const Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
        if (taps_any(tp)) atomicAdd(&s_hist[((i / dm.P) % dm.V) * NC + cell_of(tp, dm.Wimg)], 1u);
    }
    __syncthreads();
    // [s2][key] of this batch item, at this workgroup's group of query views
    unsigned *gctr = counters + (size_t)b * dm.V * NK + (size_t)(s1 / vpg) * NC;
    if (MODE == 0) {
        for (int i = threadIdx.x; i < nhist; i += kBinLdsThreads) {
            const unsigned c = s_hist[i];
            if (c) atomicAdd(gctr + (size_t)(i / NC) * NK + i % NC, c);
        }
    } else {
        for (int i = threadIdx.x; i < nhist; i += kBinLdsThreads) {
            const unsigned c = s_hist[i];
            s_base[i] = c ? atomicAdd(gctr + (size_t)(i / NC) * NK + i % NC, c) : 0u;
            s_hist[i] = 0u;
        }
        __syncthreads();
        const size_t M = (size_t)dm.V * dm.L * dm.P;
        for (int i = threadIdx.x; i < total; i += kBinLdsThreads) {
            const float2 xy = crd[i];
            const Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
            if (!taps_any(tp)) continue;
            const int p = i % dm.P, s2 = (i / dm.P) % dm.V, l = l0 + i / dm.N;
            const int hidx = s2 * NC + cell_of(tp, dm.Wimg);
            const unsigned pos = s_base[hidx] + atomicAdd(&s_hist[hidx], 1u);
            store_cell_entry(sorted, ((size_t)b * dm.V + s2) * M + pos, ((unsigned)s1 * dm.L + l) * (unsigned)dm.P + (unsigned)p,
                             cell_fraction(xy, dm), records);
        }
    }
}

// One workgroup per (b, s2): exclusive scan of the list lengths (NC here = the number of keys, group-major). Writes
// start[grp*(NC+1) + c] (with the total at c = NC) and resets counters to the
// same starts, so that the fill pass can use them as cursors.
//
// It also makes the dk/dv kernel's work list of this (b, s2): one item (cell, first entry, end) per run of at
// most `piece` consecutive entries of a non-empty list, in list order -- items[grp*wmax + i]; the slots after
// the last item are marked empty (first = end). Empty lists get no item (clustered coordinates leave most
// of the grid empty), and a list much longer than the average is cut into pieces that different waves take,
// so that the longest list no longer sets the kernel's duration. wmax >= NC + M/piece bounds the number of
// items (M = entries of all lists). An item carries all a wave needs to start on it: one read, where the
// list's bounds would be a second, dependent one.
static __global__ __launch_bounds__(1024) void bin_scan_kernel(unsigned *__restrict__ counters,
                                                        unsigned *__restrict__ start, int NC, int grid_cells,
                                                        unsigned piece, unsigned wmax, uint4 *__restrict__ items)
{
    __shared__ unsigned s_part[1024], s_pcs[1024];
    __shared__ unsigned s_carry, s_pcarry;
    unsigned *cnt = counters + (size_t)blockIdx.x * NC;
    unsigned *st = start + (size_t)blockIdx.x * (NC + 1);
    uint4 *it = items + (size_t)blockIdx.x * wmax;
    if (threadIdx.x == 0) { s_carry = 0; s_pcarry = 0; }
    __syncthreads();
    for (int base = 0; base < NC; base += 1024) {
        const int c = base + threadIdx.x;
        const unsigned v = c < NC ? cnt[c] : 0u;
        const unsigned np = (v + piece - 1) / piece;               // pieces of this list
        s_part[threadIdx.x] = v;
        s_pcs[threadIdx.x] = np;
        __syncthreads();
        for (int off = 1; off < 1024; off <<= 1) {             // Hillis-Steele inclusive scans, both at once
            const bool take = threadIdx.x >= (unsigned)off;
            const unsigned add = take ? s_part[threadIdx.x - off] : 0u;
            const unsigned padd = take ? s_pcs[threadIdx.x - off] : 0u;
            __syncthreads();
            s_part[threadIdx.x] += add;
            s_pcs[threadIdx.x] += padd;
            __syncthreads();
        }
        const unsigned excl = s_carry + s_part[threadIdx.x] - v;
        const unsigned pexcl = s_pcarry + s_pcs[threadIdx.x] - np;
        if (c < NC) {
            st[c] = excl;
            cnt[c] = excl;
            const unsigned cell = (unsigned)(c % grid_cells);
            for (unsigned i = 0; i < np; ++i)
                if (pexcl + i < wmax) it[pexcl + i] = make_uint4(cell, excl + i * piece, min(excl + v, excl + (i + 1) * piece), 0u);
        }
        __syncthreads();
        if (threadIdx.x == 1023) { s_carry += s_part[1023]; s_pcarry += s_pcs[1023]; }
        __syncthreads();
    }
    if (threadIdx.x == 0) st[NC] = s_carry;
    for (unsigned i = min(s_pcarry, wmax) + threadIdx.x; i < wmax; i += 1024) it[i] = make_uint4(0u, 0u, 0u, 0u);
}

// Deterministic backward: begin / end of every cell list as positions in the flat id array
// [B*V][M] (one thread per (group, cell)), the segment bounds of the sort that orders each list.
static __global__ void cell_segments_kernel(const unsigned *__restrict__ start, int NC, unsigned M, unsigned nseg,
                                            unsigned *__restrict__ seg_begin, unsigned *__restrict__ seg_end)
{
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nseg) return;
    const unsigned grp = i / (unsigned)NC, cell = i - grp * (unsigned)NC;
    const unsigned *st = start + (size_t)grp * (NC + 1) + cell;
    seg_begin[i] = grp * M + st[0];
    seg_end[i] = grp * M + st[1];
}

template <typename S, int DC>
__device__ __forceinline__ void load_tap_or_zero(const char *base, int pix, int D, int lane_elem, bool valid,
                                                 float (&dst)[DC])
{
    if (valid) {
        load_chunk<S, DC>(base + ((size_t)pix * D + lane_elem) * S::kBytes, dst);
    } else {
#pragma unroll
        for (int d = 0; d < DC; ++d) dst[d] = 0.f;
    }
}

// A lane's part of one query row as it comes from memory: q and dout words (storage type), and the row's
// (lse, delta) pair.
template <int WORDS> struct RowFetch { uint32_t qw[WORDS], dw[WORDS]; float2 ld; };

template <int WORDS>
__device__ __forceinline__ void load_words(const void *p, uint32_t (&w)[WORDS])
{
    static_assert(WORDS == 2 || WORDS % 4 == 0, "8 bytes, or multiples of 16");
    if constexpr (WORDS == 2) {
        const uint2 t = *reinterpret_cast<const uint2 *>(p);
        w[0] = t.x; w[1] = t.y;
    } else {
#pragma unroll
        for (int i = 0; i < WORDS / 4; ++i) {
            const uint4 t = reinterpret_cast<const uint4 *>(p)[i];
            w[4 * i + 0] = t.x; w[4 * i + 1] = t.y; w[4 * i + 2] = t.z; w[4 * i + 3] = t.w;
        }
    }
}

// the words of load_words as DC fp32 values
template <typename S, int DC>
__device__ __forceinline__ void widen_words(const uint32_t (&w)[DC * S::kBytes / 4], float (&dst)[DC])
{
    if constexpr (S::kBytes == 4) {
#pragma unroll
        for (int d = 0; d < DC; ++d) dst[d] = __uint_as_float(w[d]);
    } else {
#pragma unroll
        for (int j = 0; j < DC / 2; ++j) {
            if constexpr (S::kBf16) {
                dst[2 * j + 0] = __uint_as_float(w[j] << 16);
                dst[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
            } else {
                union { uint32_t u; _Float16 h[2]; } cv;
                cv.u = w[j];
                dst[2 * j + 0] = (float)cv.h[0];
                dst[2 * j + 1] = (float)cv.h[1];
            }
        }
    }
}

// Which cells one launch of the dk/dv kernel covers, and the divisors that decode a work index into
// (b, h, s2, cell) with multiply-shift instead of integer division (the decode is scalar code every
// wave runs before it knows whether its cell is empty).
// colour < 0: all cells, per-cell sums flushed with float atomics (a pixel belongs to four cells).
// colour 0..3 (deterministic backward): only the cells with (row parity, column parity) = colour; no
// two of them share a pixel, so the flush is a plain read-add-write, and the four launches, one
// after the other, add every pixel's four contributions in a fixed order.
// colour < 0 also switches the decode to the work list made by bin_scan_kernel: work index -> (b, h, s2, item),
// `ncells` then being the list's capacity wmax per (b, s2); empty slots leave at once.
struct CellGrid {
    int colour, oy, ox, step, ncx, ncells;
    int bh0;                                // first (batch, head) pair of this launch (b * H + h)
    unsigned nwork;                         // pairs of this launch * V * ncells < 2^31
    FastDiv div_cells, div_ncx, div_v, div_h;
};

// HANDED: the dq kernel has left (p, sm_scale * ds) of every sample in `handed_` (per query row of this head,
// in the order of the row's coordinates): an entry then costs a gather of that pair and the two rank-1 updates --
// no taps in registers, no dot products, no exponential. Only with the work list (colour < 0) and with
// records (the positions beside the ids).
// RECORDS: the lists hold 12-byte records (sample id and position in the cell); without, ids alone, and every
// entry's coordinate pair is read again (the deterministic backward, whose lists are sorted id arrays).
template <typename S, int D, int DC, bool HANDED, bool RECORDS>
__global__ __launch_bounds__(kCellWaves *kWave, HANDED ? (DC <= 4 ? 5 : (S::kBytes == 2 ? 3 : 4))
                                                       : DC <= 4 ? (S::kBytes == 2 && D >= 64 ? 5 : 4) : (S::kBytes == 2 ? 3 : 2))
void bwd_dkdv_cell_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, const float2 *__restrict__ stats_,
    const void *__restrict__ dout_, const unsigned *__restrict__ start, const unsigned *__restrict__ sorted,
    const uint4 *__restrict__ items, const float2 *__restrict__ handed_,
    float *__restrict__ dk_acc, float *__restrict__ dv_acc, Dims dm, int NC, CellGrid cg)
{
    constexpr int G = D / DC;
    constexpr int NS = kWave / G;
    static_assert(G >= 4 && G <= 64 && G * DC == D, "lane split (a block of four lanes must not straddle two samples)");
    __shared__ float4 s_w[kCellWaves][2 * kWave];           // two sets of entry tables, used in turn
    __shared__ unsigned s_row[kCellWaves][2 * kWave];       // byte offset of the entry's query row in dout (and its (lse, delta))
    __shared__ unsigned s_qrow[kCellWaves][2 * kWave];      // ... in q (which may be strided)
    __shared__ float2 s_f[S::kBytes == 2 ? kCellWaves : 1][2 * kWave];      // 16-bit storage: (fx, fy) of the entry
    __shared__ __attribute__((aligned(16))) float s_flush[kCellWaves][4 * D];                 // the flush: four rows of dk, then of dv
    constexpr bool kQuad = HANDED && S::kBytes == 2 && DC >= 8;            // four-entry trips (below)
    // kQuad: a ring of merged entries; the coefficients as [tap][place]
    __shared__ __attribute__((aligned(16))) float s_ckq[kQuad ? kCellWaves : 1][2 * 4 * kWave], s_cvq[kQuad ? kCellWaves : 1][2 * 4 * kWave];
    __shared__ __attribute__((aligned(16))) unsigned s_rowq[kQuad ? kCellWaves : 1][2 * kWave], s_qrowq[kQuad ? kCellWaves : 1][2 * kWave];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    const unsigned work = (unsigned)xcd_logical_block(blockIdx.x, gridDim.x) * kCellWaves + wave;
    if (work >= cg.nwork) return;
    const int colour = cg.colour;
    // plane-major: (b, h, s2, cell or work item)
    unsigned t = cg.div_cells.div(work);
    const int ci = (int)(work - t * (unsigned)cg.ncells);
    const unsigned bhl = cg.div_v.div(t);                      // pair within this launch
    const int s2 = (int)(t - bhl * (unsigned)dm.V);
    const unsigned bh = (unsigned)cg.bh0 + bhl;
    const int b = (int)cg.div_h.div(bh);
    const int h = (int)(bh - (unsigned)b * (unsigned)dm.H);
    const size_t grp = (size_t)b * dm.V + s2;
    int cy, cx, cell;
    unsigned lo, hi;
    if (colour < 0) {
        const uint4 item = items[grp * (size_t)cg.ncells + ci];              // (cell, first entry, end)
        cell = (int)item.x;
        cy = (int)cg.div_ncx.div(item.x);                      // div_ncx: by Wimg + 1 in this mode
        cx = cell - cy * (dm.Wimg + 1);
        lo = item.y;
        hi = item.z;
    } else {
        const int cyi = (int)cg.div_ncx.div((unsigned)ci);
        cy = cyi * cg.step + cg.oy;
        cx = (ci - cyi * cg.ncx) * cg.step + cg.ox;            // on the (Himg+1) x (Wimg+1) grid
        cell = cy * (dm.Wimg + 1) + cx;
        lo = start[grp * (NC + 1) + cell];
        hi = start[grp * (NC + 1) + cell + 1];
    }
    if (lo >= hi) return;

    const int g = lane % G, slot = lane / G, lane_elem = g * DC;
    const int y0 = cy - 1, x0 = cx - 1;
    const bool vy0 = y0 >= 0, vy1 = y0 + 1 < dm.Himg, vx0 = x0 >= 0, vx1 = x0 + 1 < dm.Wimg;
    const bool tv[4] = { vy0 && vx0, vy0 && vx1, vy1 && vx0, vy1 && vx1 };
    const int tpix[4] = { y0 * dm.Wimg + x0, y0 * dm.Wimg + x0 + 1, (y0 + 1) * dm.Wimg + x0,
                          (y0 + 1) * dm.Wimg + x0 + 1 };
    const size_t plane_base = ((grp * dm.H) + h) * (size_t)dm.L * D;          // elements in dk/dv; grp = b*V + s2
    const size_t kv_base = dm.kv_plane(b, s2, h);                               // ... in k and v
    const char *kb = (const char *)k_ + kv_base * S::kBytes;
    const char *vb = (const char *)v_ + kv_base * S::kBytes;
    // fp32 storage: the taps widened in registers; 16-bit storage: the taps as packed pairs (half the
    // registers) feeding the packed dot-product instructions
    constexpr bool kPacked = S::kBytes == 2;
    float kt[4][kPacked ? 1 : DC], vt[4][kPacked ? 1 : DC], aK[4][DC], aV[4][DC];
    uint32_t ktp[4][kPacked ? DC / 2 : 1], vtp[4][kPacked ? DC / 2 : 1];
    // The per-sample rank-1 updates aK[t][d] += c_t * q[d], aV[t][d] += c'_t * dout[d] run on the 4x4 block
    // matrix instruction (see block_outer_fma): mK[d][t] / mV[d][t] are the same sums as aK[t][d] / aV[t][d].
    floatx4 mK[DC], mV[DC];
    // The row of the update that lane (lane & 3) supplies is a product a_x(fx) * a_y(fy) of two linear forms
    // with per-lane constants, so no lane ever selects among the four: packed (the bilinear weight of tap
    // lane & 3): a_x = 1 - fx or fx, a_y = 1 - fy or fy; fp32 (the moment 1, fx, fy, fx*fy): a_x = 1 or fx,
    // a_y = 1 or fy.
    const float row_sx = (lane & 1) ? 1.0f : (kPacked ? -1.0f : 0.0f), row_ox = (lane & 1) ? 0.0f : 1.0f;
    const float row_sy = (lane & 2) ? 1.0f : (kPacked ? -1.0f : 0.0f), row_oy = (lane & 2) ? 0.0f : 1.0f;
#pragma unroll
    for (int tpi = 0; tpi < (HANDED ? 0 : 4); ++tpi) {
        if constexpr (kPacked) {
#pragma unroll
            for (int i = 0; i < DC / 2; ++i) { ktp[tpi][i] = 0u; vtp[tpi][i] = 0u; }
            if (tv[tpi]) {
                load_packed<S, DC>(kb + ((size_t)tpix[tpi] * dm.kv_sl + lane_elem) * S::kBytes, ktp[tpi]);
                load_packed<S, DC>(vb + ((size_t)tpix[tpi] * dm.kv_sl + lane_elem) * S::kBytes, vtp[tpi]);
            }
        } else {
            load_tap_or_zero<S, DC>(kb, tpix[tpi], dm.kv_sl, lane_elem, tv[tpi], kt[tpi]);
            load_tap_or_zero<S, DC>(vb, tpix[tpi], dm.kv_sl, lane_elem, tv[tpi], vt[tpi]);
        }
    }
#pragma unroll
    for (int d = 0; d < DC; ++d) { mK[d] = floatx4{0.f, 0.f, 0.f, 0.f}; mV[d] = floatx4{0.f, 0.f, 0.f, 0.f}; }
    // fp32 storage: the cell's taps are turned, once, into the coefficients of the bilinear form
    //   blend(fx, fy) = T00 + fx*(T01 - T00) + fy*(T10 - T00) + fx*fy*(T00 - T01 - T10 + T11)
    // so that a sample's blend costs 3 multiply-adds per element instead of 4, and the sums are kept as the
    // matching moments (sum c, sum c*fx, sum c*fy, sum c*fx*fy times the query row), turned back into the
    // four pixels' sums after the loop. (Taps outside the image were loaded as zero rows.)
    if constexpr (!kPacked && !HANDED) {
#pragma unroll
        for (int d = 0; d < DC; ++d) {
            kt[3][d] = (kt[3][d] - kt[2][d]) - (kt[1][d] - kt[0][d]);
            kt[1][d] -= kt[0][d];
            kt[2][d] -= kt[0][d];
            vt[3][d] = (vt[3][d] - vt[2][d]) - (vt[1][d] - vt[0][d]);
            vt[1][d] -= vt[0][d];
            vt[2][d] -= vt[0][d];
        }
    }
    const float qscale = dm.sm_scale * kLog2e;
    const size_t M = (size_t)dm.V * dm.L * dm.P;
    static_assert(RECORDS || !HANDED, "the pairs are handed over to lists of records only");
    const unsigned *list = sorted + grp * M * (RECORDS ? 3u : 1u);      // ids, or 12-byte records (id, fx, fy)
    // Query rows of this wave's (b, h) are addressed as a uniform base plus a 32-bit byte offset
    // (s1*H*L + l) * ROW < V*H*L*D*e <= 2^32 (the shape limits keep one batch item of a tensor below 2^30
    // elements): one add per gather instead of 64-bit address arithmetic per lane.
    constexpr unsigned kRowBytes = D * S::kBytes;
    constexpr int kRowWords = DC * S::kBytes / 4;                           // 32-bit words of a row held by one lane
    constexpr int kRowToPairShift = __builtin_ctz(kRowBytes) - 3;          // row byte offset -> offset of the row's (lse, delta)
    const size_t bh_row0 = ((size_t)b * dm.V * dm.H + h) * dm.L;              // row of (b, s1 = 0, h, l = 0)
    const char *q_bh = (const char *)q_ + dm.q_row(b, 0, h, 0) * S::kBytes;
    const char *do_bh = (const char *)dout_ + bh_row0 * kRowBytes;
    const char *stats_bh = (const char *)(stats_ + bh_row0);                 // (lse, delta) per row
    const unsigned lane_byte = (unsigned)lane_elem * S::kBytes;
    const unsigned view_rows = (unsigned)dm.H * (unsigned)dm.L;
    const float2 *coords = reinterpret_cast<const float2 *>(coords_);

    // HANDED: the entry's pair, gathered one chunk ahead (so the ids are fetched two chunks ahead). The pairs of
    // this launch's (batch, head) pairs lie as [pair][s1][l][sample]; those of this wave's pair are a uniform base
    // plus a 32-bit byte offset (the host checks V*L*N*8 < 2^32).
    const char *handed_bh = (const char *)(handed_ + (size_t)bhl * dm.V * dm.L * (size_t)dm.N);
    auto load_pair = [&](unsigned sid) -> float2 {
        const unsigned qlx = dm.divP.div(sid), px = sid - qlx * (unsigned)dm.P;       // qlx = s1*L + l
        const unsigned off = (qlx * (unsigned)dm.N + (unsigned)s2 * (unsigned)dm.P + px) * 8u;
        return *reinterpret_cast<const float2 *>(handed_bh + off);
    };
    if constexpr (kQuad) {
        // 16-bit storage with the pairs handed over, eight elements per lane (at four the trips are too short for
        // the requests to arrive in time: 1.14 -> 1.22 ms at 48x48, D = 64): FOUR entries per slot and trip on the
        // 4x4x4 block matrix instruction. k runs over the four entries, i over the four taps (lane 4b+i supplies
        // the four entries' coefficients of tap i, high and low parts in two instructions), j over the block's
        // lanes with their elements of the four query rows -- as stored, regrouped by two byte permutes per pair
        // of rows. 4 * DC instructions do what 4 * 2 * DC rank-1 updates and as many bf16 -> fp32 conversions did.
        //
        // Entries of ONE query in one cell are merged before their rows are requested: a query's samples cluster,
        // the fill pass of the binning leaves the samples that one wave places in one list next to each other (the
        // ranks that one returning LDS atomic hands out), and the sums are linear in the coefficients -- so a run
        // of up to four neighbouring entries with the same query row becomes one entry with the summed tap
        // coefficients: one gather of q and dout and one set of matrix instructions instead of up to four.
        //
        // The merged entries of the list's 64-entry blocks are appended to a ring of kRing places in LDS (tables
        // [tap][place] of coefficients and [place] of row offsets); trips of QT merged entries are taken off its
        // head. Everything is requested ahead: the q and dout rows of the next trip while this trip is worked on
        // (one set of registers each), which needs the next trip's places filled -- so blocks are merged two ahead
        // of the trips, and trips run while two whole trips are in the ring (all of them once the last block is in;
        // the places after the last entry then hold zero coefficients and the row of a live entry).
        constexpr int QT = 4 * NS, kRing = 2 * kWave;
        static_assert(QT % 4 == 0 && kRing % QT == 0 && kRing >= 2 * kWave && kRing >= kWave + 3 * QT,
                      "two blocks fit before the first trip; places written by one block never reach the trips in flight");
        // (requests past the end of the list repeat its last entry: no request sits under a branch, and the number
        // of requests in flight at any point is the same on every path -- the compiler's waits are exact then)
        auto load_entry_q = [&](unsigned cstart) -> CellEntry {
            const unsigned *r = list + 3u * min(cstart + (unsigned)lane, hi - 1u);
            return CellEntry{r[0], __uint_as_float(r[1]), __uint_as_float(r[2])};
        };
        auto prepare = [&](unsigned cstart, int tail, unsigned sid, float2 ff, float2 pdv) -> int {
            const unsigned ql = dm.divP.div(sid);                                  // ql = s1*L + l
            const unsigned s1 = dm.divL.div(ql), l = ql - s1 * (unsigned)dm.L;
            const bool live = cstart + (unsigned)lane < hi;                        // a dead entry adds nothing
            const unsigned before = (unsigned)__shfl_up((int)ql, 1, kWave);
            const unsigned long long below = (1ull << lane) - 1ull;                // the lanes under this one
            const unsigned long long first = __ballot(lane == 0 || ql != before);  // first entries of the runs of one row
            const int run0 = 63 - __builtin_clzll(first & (below | (1ull << lane)));
            const bool lead = live && ((lane - run0) & 3) == 0;                    // runs are cut into merged entries of up to four
            const unsigned long long leads = __ballot(lead);
            const int idx = __builtin_popcountll(leads & below);                   // a leader's place after the tail
            const int n = __builtin_popcountll(leads);
            // the entries after this one that belong to the same merged entry: the lanes up to the next leader
            const bool f1 = lane < 63 && !((leads >> (lane + 1)) & 1ull);
            const bool f2 = f1 && lane < 62 && !((leads >> (lane + 2)) & 1ull);
            const float m1 = f1 ? 1.0f : 0.0f, m2 = f2 ? 1.0f : 0.0f;
            const float pn = live ? pdv.x : 0.f, dsn = live ? pdv.y : 0.f;
            const float gx = 1.0f - ff.x, gy = 1.0f - ff.y;
            const float wt[4] = { gx * gy, ff.x * gy, gx * ff.y, ff.x * ff.y };
            float c[8];
#pragma unroll
            for (int tpi = 0; tpi < 4; ++tpi) { c[tpi] = wt[tpi] * dsn; c[4 + tpi] = wt[tpi] * pn; }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float pairsum = fmaf(m1, __shfl_down(c[i], 1, kWave), c[i]);
                c[i] = fmaf(m2, __shfl_down(pairsum, 2, kWave), pairsum);
            }
            const unsigned row = (s1 * view_rows + l) * kRowBytes;
            const unsigned qrow = (s1 * (unsigned)dm.q_sv + l * (unsigned)dm.q_sl) * S::kBytes;
            float *ck = s_ckq[wave], *cv = s_cvq[wave];
            if (lead) {
                const int at = (tail + idx) & (kRing - 1);
#pragma unroll
                for (int tpi = 0; tpi < 4; ++tpi) { ck[tpi * kRing + at] = c[tpi]; cv[tpi * kRing + at] = c[4 + tpi]; }
                s_rowq[wave][at] = row;
                s_qrowq[wave][at] = qrow;
            }
            // the places up to the end of a last, partial trip: no coefficients, and a row that is in this list
            // (no further: the two blocks merged before the first trip may fill the ring to its last place)
            if (tail + n + lane < ((tail + n + QT - 1) & ~(QT - 1))) {
                const int at = (tail + n + lane) & (kRing - 1);
#pragma unroll
                for (int tpi = 0; tpi < 4; ++tpi) { ck[tpi * kRing + at] = 0.f; cv[tpi * kRing + at] = 0.f; }
                s_rowq[wave][at] = (unsigned)__builtin_amdgcn_readfirstlane((int)row);
                s_qrowq[wave][at] = (unsigned)__builtin_amdgcn_readfirstlane((int)qrow);
            }
            return n;
        };
        uint32_t rq[4][kRowWords], rd[4][kRowWords];
        auto issue_q = [&](int at0) {
            const uint4 r = reinterpret_cast<const uint4 *>(s_qrowq[wave])[((at0 >> 2) + slot) & (kRing / 4 - 1)];
            load_words<kRowWords>(q_bh + (r.x + lane_byte), rq[0]);
            load_words<kRowWords>(q_bh + (r.y + lane_byte), rq[1]);
            load_words<kRowWords>(q_bh + (r.z + lane_byte), rq[2]);
            load_words<kRowWords>(q_bh + (r.w + lane_byte), rq[3]);
        };
        auto issue_d = [&](int at0) {
            const uint4 r = reinterpret_cast<const uint4 *>(s_rowq[wave])[((at0 >> 2) + slot) & (kRing / 4 - 1)];
            load_words<kRowWords>(do_bh + (r.x + lane_byte), rd[0]);
            load_words<kRowWords>(do_bh + (r.y + lane_byte), rd[1]);
            load_words<kRowWords>(do_bh + (r.z + lane_byte), rd[2]);
            load_words<kRowWords>(do_bh + (r.w + lane_byte), rd[3]);
        };
        // (places that were never written are read for requests that nothing uses: any row of the pair will do)
        s_rowq[wave][lane] = 0u;
        s_rowq[wave][kWave + lane] = 0u;
        s_qrowq[wave][lane] = 0u;
        s_qrowq[wave][kWave + lane] = 0u;
        int head = 0, tail;
        CellEntry e_a;
        {
            const CellEntry e0 = load_entry_q(lo), e1 = load_entry_q(lo + kWave);
            e_a = load_entry_q(lo + 2 * kWave);
            const float2 pd0 = load_pair(e0.id), pd1 = load_pair(e1.id);
            tail = prepare(lo, 0, e0.id, make_float2(e0.fx, e0.fy), pd0);
            tail += prepare(lo + kWave, tail, e1.id, make_float2(e1.fx, e1.fy), pd1);
        }
        wave_lds_sync();
        issue_q(0);
        issue_d(0);
        const int tap_lane = (lane & 3) * (kRing / 4) + slot;                       // this lane's tap, its slot's four entries (in float4 units)
        for (unsigned cnext = lo + 2 * kWave;; cnext += kWave) {
            const bool more = cnext < hi;                      // a block is left to merge
            const float2 pd_a = load_pair(e_a.id);
            const CellEntry e_n = load_entry_q(cnext + kWave);
            __builtin_amdgcn_sched_barrier(0);                 // (requested here, not where they are used)
            // (at least one trip: a whole block adds QT merged entries or more to the QT or more that the trips before left)
            const int stop = more ? tail - 2 * QT : tail - 1;
            do {
                const int at = (head & (kRing - 1)) >> 2;
                const float4 ck4 = reinterpret_cast<const float4 *>(s_ckq[wave])[tap_lane + at];
                const float4 cv4 = reinterpret_cast<const float4 *>(s_cvq[wave])[tap_lane + at];
                const uint4 sk = split_coefficients<S>(ck4.x, ck4.y, ck4.z, ck4.w);
                const uint4 sv = split_coefficients<S>(cv4.x, cv4.y, cv4.z, cv4.w);
                __builtin_amdgcn_sched_barrier(0);
                block_blend4_pair<S, DC>(rq, __builtin_bit_cast(shortx4, make_uint2(sk.x, sk.y)),
                                         __builtin_bit_cast(shortx4, make_uint2(sk.z, sk.w)), mK);
                __builtin_amdgcn_sched_barrier(0);
                issue_q(head + QT);
                __builtin_amdgcn_sched_barrier(0);
                block_blend4_pair<S, DC>(rd, __builtin_bit_cast(shortx4, make_uint2(sv.x, sv.y)),
                                         __builtin_bit_cast(shortx4, make_uint2(sv.z, sv.w)), mV);
                __builtin_amdgcn_sched_barrier(0);
                issue_d(head + QT);
                __builtin_amdgcn_sched_barrier(0);
                head += QT;
            } while (head <= stop);
            if (!more) break;
            wave_lds_sync();
            tail += prepare(cnext, tail, e_a.id, make_float2(e_a.fx, e_a.fy), pd_a);
            wave_lds_sync();
            e_a = e_n;
        }
    }
    if constexpr (!kQuad) {
        // One list entry per lane and 64-entry block: weights and query row go into tables in LDS, which the slots
        // walk NS entries a trip. Two sets of tables, used in turn: the next block's are made while this block is
        // worked on, so that the last trip of a block can request the rows of the next block's first. The NS
        // samples of a trip need their query rows (q, dout, lse, delta) from memory, a round trip of several
        // hundred nanoseconds that the other waves of the SIMD do not cover: the rows of trip t+1 are requested
        // before trip t is worked on (two sets of row registers, the loop unrolled by two so that no set is ever
        // copied). Every request is unconditional -- entries past the end of the list repeat its last one, with
        // zero weights, and the last request of a list is never used -- and the trip loop runs at least once: the
        // number of requests in flight is the same on every path, so the compiler's waits name exactly the
        // younger requests instead of "everything" (a request under a branch, or a loop that may run zero times,
        // makes the wait at the join a wait for all outstanding loads, which undoes the overlap).
        auto load_entry_c = [&](unsigned cstart) -> CellEntry {
            const unsigned at = min(cstart + (unsigned)lane, hi - 1u);
            if constexpr (RECORDS) {
                const unsigned *r = list + 3u * at;
                return CellEntry{r[0], __uint_as_float(r[1]), __uint_as_float(r[2])};
            } else {
                return CellEntry{list[at], 0.f, 0.f};
            }
        };
        auto tables = [&](unsigned cstart, int buf, const CellEntry &e, const float2 &pdv) {
            const unsigned ql = dm.divP.div(e.id), p = e.id - ql * (unsigned)dm.P;     // ql = s1*L + l
            const unsigned s1 = dm.divL.div(ql), l = ql - s1 * (unsigned)dm.L;
            float2 ff = make_float2(e.fx, e.fy);
            if constexpr (!RECORDS) {
                const size_t ci = (((size_t)b * dm.V * dm.L + ql) * dm.V + s2) * (size_t)dm.P + p;
                ff = cell_fraction(coords[ci], dm);
            }
            // Plain bilinear weights, not masked: every sample of this list lies in this cell, whose taps
            // outside the image were loaded as zeros above and are skipped by the flush below.
            const float fx = ff.x, fy = ff.y;
            const float gx = 1.0f - fx, gy = 1.0f - fy;
            const bool live = cstart + (unsigned)lane < hi;           // a dead entry adds nothing
            const int at = buf * kWave + lane;
            if constexpr (HANDED) {
                s_w[wave][at] = make_float4(fx, fy, live ? pdv.x : 0.f, live ? pdv.y : 0.f);     // (fx, fy, p, sm_scale * ds)
            } else if constexpr (kPacked) {
                s_w[wave][at] = live ? make_float4(gx * gy, fx * gy, gx * fy, fx * fy) : make_float4(0.f, 0.f, 0.f, 0.f);
                s_f[wave][at] = make_float2(fx, live ? fy : __int_as_float(0x7fc00000));          // NaN marks a dead entry
            } else {
                s_w[wave][at] = make_float4(fx, fy, fx * fy, live ? 1.0f : 0.0f);
            }
            s_row[wave][at] = (s1 * view_rows + l) * kRowBytes;
            s_qrow[wave][at] = (s1 * (unsigned)dm.q_sv + l * (unsigned)dm.q_sl) * S::kBytes;
        };
        auto issue = [&](int buf, int j0, RowFetch<kRowWords> &f) {
            const unsigned r = s_row[wave][buf * kWave + j0 + slot];
            const unsigned roff = r + lane_byte, soff = r >> kRowToPairShift;
            load_words<kRowWords>(q_bh + (s_qrow[wave][buf * kWave + j0 + slot] + lane_byte), f.qw);
            load_words<kRowWords>(do_bh + roff, f.dw);
            if constexpr (!HANDED) f.ld = *(const float2 *)(stats_bh + soff);
        };
        auto consume = [&](int buf, int j0, const RowFetch<kRowWords> &f) {
            float qf[DC], dof[DC];
            widen_words<S, DC>(f.qw, qf);
            widen_words<S, DC>(f.dw, dof);
            if constexpr (HANDED) {
                const float4 w4 = s_w[wave][buf * kWave + j0 + slot];                 // (fx, fy, p, sm_scale * ds)
                const float cl = fmaf(w4.x, row_sx, row_ox) * fmaf(w4.y, row_sy, row_oy);
                const float ck = cl * w4.w, cv = cl * w4.z;
#pragma unroll
                for (int d = 0; d < DC; ++d) {
                    mK[d] = block_outer_fma(ck, qf[d], mK[d]);
                    mV[d] = block_outer_fma(cv, dof[d], mV[d]);
                }
            } else {
            const float4 w = s_w[wave][buf * kWave + j0 + slot];
            const float lse = f.ld.x, delta = f.ld.y;
            float dot = 0.f, dp = 0.f;
            if constexpr (kPacked) {
                // q . k~ = sum_t w_t (q . K_t): packed dot products on the raw 16-bit pairs
                dot = fmaf(w.x, packed_dot<S, DC>(f.qw, ktp[0]),
                           fmaf(w.y, packed_dot<S, DC>(f.qw, ktp[1]),
                                fmaf(w.z, packed_dot<S, DC>(f.qw, ktp[2]), w.w * packed_dot<S, DC>(f.qw, ktp[3]))));
                dp = fmaf(w.x, packed_dot<S, DC>(f.dw, vtp[0]),
                          fmaf(w.y, packed_dot<S, DC>(f.dw, vtp[1]),
                               fmaf(w.z, packed_dot<S, DC>(f.dw, vtp[2]), w.w * packed_dot<S, DC>(f.dw, vtp[3]))));
            } else {
                // w = (fx, fy, fx*fy, live)
#pragma unroll
                for (int d = 0; d < DC; ++d) {
                    const float kk = fmaf(w.z, kt[3][d], fmaf(w.y, kt[2][d], fmaf(w.x, kt[1][d], kt[0][d])));
                    const float vv = fmaf(w.z, vt[3][d], fmaf(w.y, vt[2][d], fmaf(w.x, vt[1][d], vt[0][d])));
                    dot = fmaf(qf[d], kk, dot);
                    dp = fmaf(dof[d], vv, dp);
                }
            }
            dot = group_sum<G>(dot);
            dp = group_sum<G>(dp);
            float p_n = __builtin_amdgcn_exp2f(dot * qscale - lse);
            if constexpr (!kPacked) p_n *= w.w;                    // entries past the end of the list
            const float dss = p_n * (dp - delta) * dm.sm_scale;
            // this lane's row of the update: packed: the weight of tap (lane & 3); fp32: the moment
            // (1, fx, fy, fx*fy)[lane & 3]. The four lanes of a block sit in one slot (G is a multiple of 4),
            // so they share the sample and supply its four coefficients between them.
            float fxs, fys;
            if constexpr (kPacked) {
                const float2 ff = s_f[wave][buf * kWave + j0 + slot];
                fxs = ff.x;
                fys = ff.y;
            } else {
                fxs = w.x;
                fys = w.y;
            }
            float cl = fmaf(fxs, row_sx, row_ox) * fmaf(fys, row_sy, row_oy);
            if constexpr (kPacked) cl = (fys == fys) ? cl : 0.0f;       // dead entry: p_n is finite, the row is 0
            const float ck = cl * dss, cv = cl * p_n;
#pragma unroll
            for (int d = 0; d < DC; ++d) {
                mK[d] = block_outer_fma(ck, qf[d], mK[d]);
                mV[d] = block_outer_fma(cv, dof[d], mV[d]);
            }
            }
        };
        static_assert(kWave % (2 * NS) == 0, "a block of 64 entries is a whole number of trip pairs");
        // entries are fetched one block ahead of their tables; with the pairs handed over two, and the pairs -- whose
        // addresses come from the ids -- one
        CellEntry e_a, e_b{0u, 0.f, 0.f};
        float2 pd_a = make_float2(0.f, 0.f);
        {
            const CellEntry e0 = load_entry_c(lo);
            e_a = load_entry_c(lo + kWave);
            float2 pd0 = make_float2(0.f, 0.f);
            if constexpr (HANDED) {
                e_b = load_entry_c(lo + 2 * kWave);
                pd0 = load_pair(e0.id);
                pd_a = load_pair(e_a.id);
            }
            tables(lo, 0, e0, pd0);
        }
        wave_lds_sync();
        RowFetch<kRowWords> fa, fb;
        issue(0, 0, fa);
        int cur = 0;
        for (unsigned c0 = lo;; c0 += kWave) {
            const bool has_next = c0 + kWave < hi;
            CellEntry e_c;
            float2 pd_b = make_float2(0.f, 0.f);
            if constexpr (HANDED) {
                pd_b = load_pair(e_b.id);
                e_c = load_entry_c(c0 + 3 * kWave);
            } else {
                e_c = load_entry_c(c0 + 2 * kWave);
            }
            __builtin_amdgcn_sched_barrier(0);         // (requested here, not where they are used)
            wave_lds_sync();
            tables(c0 + kWave, cur ^ 1, e_a, pd_a);
            wave_lds_sync();
            const int cnt = (int)min((unsigned)kWave, hi - c0);
            int j0 = 0;
            do {
                issue(cur, j0 + NS, fb);
                __builtin_amdgcn_sched_barrier(0);     // (keeps the requests where they are written)
                consume(cur, j0, fa);
                __builtin_amdgcn_sched_barrier(0);
                // the next pair of trips: of this block, or the first of the next block
                const bool over = j0 + 2 * NS >= kWave && has_next;
                issue(over ? cur ^ 1 : cur, (j0 + 2 * NS) & (kWave - 1), fa);
                __builtin_amdgcn_sched_barrier(0);
                consume(cur, j0 + NS, fb);
                __builtin_amdgcn_sched_barrier(0);
                j0 += 2 * NS;
            } while (j0 < cnt);
            if (!has_next) break;
            if constexpr (HANDED) {
                e_a = e_b;
                pd_a = pd_b;
                e_b = e_c;
            } else {
                e_a = e_c;
            }
            cur ^= 1;
        }
    }
#pragma unroll
    for (int tpi = 0; tpi < 4; ++tpi) {
#pragma unroll
        for (int d = 0; d < DC; ++d) { aK[tpi][d] = mK[d][tpi]; aV[tpi][d] = mV[d][tpi]; }
    }
    if constexpr (!kPacked) {
        // moments -> pixels (linear, so it can be done on the slots' partial sums):
        // w00 = 1 - fx - fy + fx*fy, w01 = fx - fx*fy, w10 = fy - fx*fy, w11 = fx*fy
#pragma unroll
        for (int d = 0; d < DC; ++d) {
            aK[0][d] = (aK[0][d] - aK[1][d]) - (aK[2][d] - aK[3][d]);
            aK[1][d] -= aK[3][d];
            aK[2][d] -= aK[3][d];
            aV[0][d] = (aV[0][d] - aV[1][d]) - (aV[2][d] - aV[3][d]);
            aV[1][d] -= aV[3][d];
            aV[2][d] -= aV[3][d];
        }
    }
    // Sum the NS slots. Slots that differ in lane bits below 16 are summed by butterflies (every lane ends
    // up with the sum); the last two steps (lane bits 16 and 32) are reduce-scatters on the lane-swap
    // instructions: a step adds the two halves and leaves each half with one half of the taps, so that in
    // the end lane bit 16 and lane bit 32 select the tap a lane holds (G <= 16), or bit 32 the tap pair
    // (G = 32), and all 64 lanes carry sums that go to memory.
#pragma unroll
    for (int off = G; off < 16; off <<= 1) {
#pragma unroll
        for (int tpi = 0; tpi < 4; ++tpi) {
#pragma unroll
            for (int d = 0; d < DC; ++d) {
                aK[tpi][d] += __shfl_xor(aK[tpi][d], off, kWave);
                aV[tpi][d] += __shfl_xor(aV[tpi][d], off, kWave);
            }
        }
    }
    static_assert(G <= 32, "at least two slots");
    constexpr int kTapsHeld = G <= 16 ? 1 : 2;             // taps a lane holds after the reduce-scatters
    float hK[kTapsHeld][DC], hV[kTapsHeld][DC];
    if constexpr (G <= 16) {
#pragma unroll
        for (int d = 0; d < DC; ++d) {
            // bit 16: rows {0, 1} | {2, 3}; then bit 32: first | second of the pair
            const float k0 = swap_add_16(aK[0][d], aK[2][d]), k1 = swap_add_16(aK[1][d], aK[3][d]);
            const float v0 = swap_add_16(aV[0][d], aV[2][d]), v1 = swap_add_16(aV[1][d], aV[3][d]);
            hK[0][d] = swap_add_32(k0, k1);
            hV[0][d] = swap_add_32(v0, v1);
        }
    } else {
#pragma unroll
        for (int d = 0; d < DC; ++d) {
            hK[0][d] = swap_add_32(aK[0][d], aK[2][d]);
            hK[1][d] = swap_add_32(aK[1][d], aK[3][d]);
            hV[0][d] = swap_add_32(aV[0][d], aV[2][d]);
            hV[1][d] = swap_add_32(aV[1][d], aV[3][d]);
        }
    }
    // tap of hK[i] / hV[i] in this lane
    const int held0 = G <= 16 ? ((lane >> 4) & 1) * 2 + (lane >> 5) : (lane >> 5) * 2;
    // Through LDS into memory order: the four rows of dk (then of dv) as 4*D consecutive floats, which the
    // wave then adds to memory 64 consecutive floats per instruction (one or two cache lines a request,
    // where a lane adding its own DC consecutive floats would touch 64 / G lines with every instruction).
    const bool writer = (lane & 15) < G;                     // (lanes that differ below bit 16 hold copies)
    float *fl = s_flush[wave];
    constexpr int kLog2D = __builtin_ctz(D);
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        wave_lds_sync();
        if (writer) {
#pragma unroll
            for (int i = 0; i < kTapsHeld; ++i) {
                float *dst = fl + (held0 + i) * D + lane_elem;
#pragma unroll
                for (int d = 0; d < DC; d += 4)
                    *reinterpret_cast<float4 *>(dst + d) = which == 0
                        ? make_float4(hK[i][d], hK[i][d + 1], hK[i][d + 2], hK[i][d + 3])
                        : make_float4(hV[i][d], hV[i][d + 1], hV[i][d + 2], hV[i][d + 3]);
            }
        }
        wave_lds_sync();
        float *acc = (which == 0 ? dk_acc : dv_acc) + plane_base;
#pragma unroll
        for (int idx0 = 0; idx0 < 4 * D; idx0 += kWave) {
            const int idx = idx0 + lane;
            const int r = idx >> kLog2D, dd = idx & (D - 1);
            const bool ok = ((r & 2) ? vy1 : vy0) && ((r & 1) ? vx1 : vx0);
            const int pix = (y0 + (r >> 1)) * dm.Wimg + x0 + (r & 1);
            const float val = fl[idx];
            if (ok) {
                float *pa = acc + (size_t)pix * D + dd;
                if (colour < 0) atomicAdd(pa, val);
                else *pa += val;
            }
        }
    }
}

}  // namespace dsdpa
