// Forward and dq for fp32 storage and 16 or 32 samples per view on images whose K/V planes do not fit in LDS but
// whose planes cut to 16 columns do, twice: "slabs" of 64 bytes per pixel (`ops/triton.py:118-170` is the sampling
// and softmax loop this replaces; the reference gathers every tap from global memory).
//
// A workgroup owns a block of query rows of one (batch, head). For every key view it walks the column slabs of K
// and then those of V, each the whole image at 64 bytes per pixel, in two LDS buffers: the slab of the next step
// is loaded straight into the other buffer (global_load_lds_dwordx4) while the present one is worked on, one
// barrier per step. One lane owns one (query row, sample) pair for a whole view: it reads its four tap rows from
// the slab in 16-byte pieces and keeps the partial dot product (K slabs) in a register, so the tap weights and
// addresses are computed once per sample and view and nothing is summed across lanes for the logits. For the V
// slabs the 16 samples of a block sit in 16 neighbouring lanes, whose weighted sums are combined by a
// reduce-scatter over those lanes: every lane ends up with one column of the slab.
//
// LDS banks (64 banks of 4 bytes; a 16-byte read is served 16 lanes a clock): the piece a lane reads at step c is
// (c + lane) mod 4, so four neighbouring lanes cover the 16 banks of one slab row; which quarter of the banks a
// row lies in is its index mod 4. Image rows are stored with a pitch of 2 mod 4 pixels, which gives the four
// taps of a sample (x, x+1, x+pitch, x+pitch+1) four different quarters, and lanes 4g .. 4g+3 of every 16 read
// their taps in the order that starts in quarter g: the 16 lanes of a clock then touch all 64 banks once,
// whatever the coordinates (a tap outside the image reads a row of the quarter it would have had: slab_sample).
#pragma once
#include "dsdpa_common.h"

namespace dsdpa {

constexpr int kSlabBytes = 64;             // bytes of one pixel in a slab: 16 fp32 columns
constexpr int kSlabCols = 16;
constexpr int kSlabSamples = 16;           // samples of a (query row, view) per block: the 16 lanes of a DPP row

// slab rows between two image rows: the width rounded up to 2 mod 4
__host__ __device__ inline int slab_pitch(int Wimg) { return Wimg + ((6 - (Wimg & 3)) & 3); }

// maximum over aligned groups of 16 lanes; every lane gets it
__device__ __forceinline__ float group16_max(float x)
{
    x = fmaxf(x, dpp_f32<0xB1>(x));
    x = fmaxf(x, dpp_f32<0x4E>(x));
    x = fmaxf(x, dpp_f32<0x141>(x));
    x = fmaxf(x, dpp_f32<0x140>(x));
    return x;
}

// The four tap rows of a sample, made opaque to the compiler at the place they are used: the addresses formed
// from them (16 per sample and slab) are then computed there, next to their reads, and not once for all slabs.
__device__ __forceinline__ void keep_here(unsigned (&o)[4])
{
    asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]));
}

__device__ __forceinline__ void pin_here(float (&o)[4])
{
    asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]));
}

// rows of 16 lanes rotated: lane i of a row receives the value of lane (i - N) mod 16
#define DSDPA_ROW_ROR(N) (0x120 + (N))

// the value of lane i ^ 4: a rotation by 12 for the lanes with bit 2 clear (banks 0 and 2 of a row), by 4 for the others
__device__ __forceinline__ float dpp_xor4(float x)
{
    int r = __builtin_amdgcn_update_dpp(0, __float_as_int(x), DSDPA_ROW_ROR(12), 0xf, 0x5, false);
    r = __builtin_amdgcn_update_dpp(r, __float_as_int(x), DSDPA_ROW_ROR(4), 0xf, 0xa, false);
    return __int_as_float(r);
}

// ------------------------------------------------------------------ pieces shared by the forward and dq kernels
// What a lane keeps of one of its samples for a view: the slab rows of the four taps (in 16-byte units, in this
// lane's read order) and their weights in the same order.
// Slab rows: image row y at y * pitch. The taps 00, 01, 10, 11 of a sample inside the image lie in the quarters
// r, r+1, r+2, r+3 (mod 4) with r that of tap 00. A tap outside the image has weight 0 and may read any row: it
// reads one of the first four, the one in the quarter it would have had (clamped into the image it would share a
// row with its neighbour, and the 16 lanes of a clock would collide).
// Returns the rotation: place k of the lane's order holds tap (k + rot) mod 4.
__device__ __forceinline__ int slab_sample(float2 xy, const Dims &dm, int pitch, int g4, unsigned (&off)[4], float (&w)[4])
{
    const Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
    const int n0 = tp.y0 * pitch + tp.x0;
    const bool vx0 = (unsigned)tp.x0 < (unsigned)dm.Wimg, vx1 = (unsigned)(tp.x0 + 1) < (unsigned)dm.Wimg;
    const bool vy0 = (unsigned)tp.y0 < (unsigned)dm.Himg, vy1 = (unsigned)(tp.y0 + 1) < (unsigned)dm.Himg;
    unsigned o[4] = { (unsigned)((vx0 && vy0) ? n0 : (n0 & 3)), (unsigned)((vx1 && vy0) ? n0 + 1 : ((n0 + 1) & 3)),
                      (unsigned)((vx0 && vy1) ? n0 + pitch : ((n0 + pitch) & 3)),
                      (unsigned)((vx1 && vy1) ? n0 + pitch + 1 : ((n0 + pitch + 1) & 3)) };
    float ww[4] = { tp.w[0], tp.w[1], tp.w[2], tp.w[3] };
    const int rot = (g4 - n0) & 3;                 // read order: tap (k + rot) mod 4 at step k
    if (rot & 1) {
        const unsigned t0 = o[0]; o[0] = o[1]; o[1] = o[2]; o[2] = o[3]; o[3] = t0;
        const float f0 = ww[0]; ww[0] = ww[1]; ww[1] = ww[2]; ww[2] = ww[3]; ww[3] = f0;
    }
    if (rot & 2) {
        const unsigned t0 = o[0], t1 = o[1]; o[0] = o[2]; o[1] = o[3]; o[2] = t0; o[3] = t1;
        const float f0 = ww[0], f1 = ww[1]; ww[0] = ww[2]; ww[1] = ww[3]; ww[2] = f0; ww[3] = f1;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        off[k] = o[k] * (kSlabBytes / 16);
        w[k] = ww[k];
    }
    return rot;
}

// four values in tap order 00, 01, 10, 11 into a lane's read order (place k: tap (k + rot) mod 4)
__device__ __forceinline__ void slab_rotate(float (&a)[4], int rot)
{
    if (rot & 1) {
        const float f0 = a[0]; a[0] = a[1]; a[1] = a[2]; a[2] = a[3]; a[3] = f0;
    }
    if (rot & 2) {
        const float f0 = a[0], f1 = a[1]; a[0] = a[2]; a[1] = a[3]; a[2] = f0; a[3] = f1;
    }
}

// x . (sum_t w_t * row_t) over the 16 columns of the slab in buffer `cur`: x is the wave's parked vector of the
// sample's query row (q or dout), read from LDS in the same rotated pieces as the taps.
// d: x . row_t of the four taps (the lane's order), for the caller that needs them one by one.
__device__ __forceinline__ float slab_dot(const float4 *slab4, const float4 *xrow, const unsigned (&off)[4], unsigned cur,
                                          const unsigned (&chv)[4], const float (&w)[4], float (&d)[4])
{
    unsigned ob[4] = { off[0] + cur, off[1] + cur, off[2] + cur, off[3] + cur };
    keep_here(ob);
    d[0] = d[1] = d[2] = d[3] = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const float4 x = xrow[chv[c]];
        float4 t[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) t[k] = slab4[ob[k] + chv[c]];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            d[k] = fmaf(x.x, t[k].x, fmaf(x.y, t[k].y, fmaf(x.z, t[k].z, fmaf(x.w, t[k].w, d[k]))));
        pin_here(d);                      // (the arithmetic on a piece stays next to its reads)
        __builtin_amdgcn_sched_barrier(0);
    }
    return fmaf(w[0], d[0], fmaf(w[1], d[1], fmaf(w[2], d[2], w[3] * d[3])));
}

// sum over the 16 lanes of a query row of (sum_t w_t * row_t) on the slab in buffer `cur`; lane j of the 16 gets
// column 4 (j & 3) + 2 * bit 3 + bit 2 of the slab.
// Register c of lane j holds piece (c + j) mod 4: the same piece is in register c + 2 of lane j + 2 and in
// register c + 1 of lane j - 1 (lanes mod 16); the lanes j ^ 8, j ^ 4, j ^ 12 then hold the other twelve lanes'
// sums of piece j mod 4, and two halving steps leave one column each.
__device__ __forceinline__ float slab_axpy(const float4 *slab4, const unsigned (&off)[4], unsigned cur,
                                           const unsigned (&chv)[4], const float (&w)[4], int lane)
{
    unsigned ob[4] = { off[0] + cur, off[1] + cur, off[2] + cur, off[3] + cur };
    keep_here(ob);
    float o[2][4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float4 t[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) t[k] = slab4[ob[k] + chv[c]];
        const float x0 = fmaf(w[0], t[0].x, fmaf(w[1], t[1].x, fmaf(w[2], t[2].x, w[3] * t[3].x)));
        const float x1 = fmaf(w[0], t[0].y, fmaf(w[1], t[1].y, fmaf(w[2], t[2].y, w[3] * t[3].y)));
        const float x2 = fmaf(w[0], t[0].z, fmaf(w[1], t[1].z, fmaf(w[2], t[2].z, w[3] * t[3].z)));
        const float x3 = fmaf(w[0], t[0].w, fmaf(w[1], t[1].w, fmaf(w[2], t[2].w, w[3] * t[3].w)));
        if (c < 2) {
            o[c][0] = x0; o[c][1] = x1; o[c][2] = x2; o[c][3] = x3;
        } else {
            o[c - 2][0] += dpp_f32<DSDPA_ROW_ROR(14)>(x0);
            o[c - 2][1] += dpp_f32<DSDPA_ROW_ROR(14)>(x1);
            o[c - 2][2] += dpp_f32<DSDPA_ROW_ROR(14)>(x2);
            o[c - 2][3] += dpp_f32<DSDPA_ROW_ROR(14)>(x3);
        }
        pin_here(o[c & 1]);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) o[0][e] += dpp_f32<DSDPA_ROW_ROR(1)>(o[1][e]);
    const bool b8 = (lane & 8) != 0, b4 = (lane & 4) != 0;
    const float k0 = b8 ? o[0][2] : o[0][0], k1 = b8 ? o[0][3] : o[0][1];
    const float g0 = b8 ? o[0][0] : o[0][2], g1 = b8 ? o[0][1] : o[0][3];
    const float h0 = k0 + dpp_f32<DSDPA_ROW_ROR(8)>(g0), h1 = k1 + dpp_f32<DSDPA_ROW_ROR(8)>(g1);
    const float kk = b4 ? h1 : h0, gg = b4 ? h0 : h1;
    return kk + dpp_xor4(gg);
}

// Staging of the slabs: a wave moves runs of 16 pixels of one image row (four lanes per pixel, 16 bytes each), run
// wave + 16 j of the image's Himg * nxb runs at its step j: where a run starts is the same for all lanes (scalar
// registers), a lane adds its own place in the run. Offsets inside one (batch, head) fit 32 bits. The slab goes
// from memory to LDS without passing through registers (global_load_lds_dwordx4: lane i of a wave writes 16 bytes
// at the wave's LDS base + 16 i, which is the layout of a run); fetch() only issues the loads, wait() -- before the
// barrier that ends a step -- waits for this wave's.
template <int NW>
struct SlabStager {
    static constexpr int kStage = (64 + NW - 1) / NW;       // runs of 16 pixels a wave moves per slab (an image has at most 64)
    int pix[kStage], dst[kStage], x0[kStage];       // per wave: scalar registers
    __device__ __forceinline__ void init(int wave, const Dims &dm, int pitch)
    {
        const int nxb = (dm.Wimg + 15) >> 4, nruns = dm.Himg * nxb;
#pragma unroll
        for (int j = 0; j < kStage; ++j) {
            const int run = min(wave + NW * j, nruns - 1);           // (a run past the image: the last one once more)
            const int y = run / nxb, xs = (run - y * nxb) * 16;
            pix[j] = __builtin_amdgcn_readfirstlane(y * dm.Wimg + xs);
            dst[j] = __builtin_amdgcn_readfirstlane((y * pitch + xs) * kSlabBytes);
            x0[j] = __builtin_amdgcn_readfirstlane(xs);
        }
    }
    // columns [col, col + 16) of `plane` into the LDS buffer at byte offset lds_base
    __device__ __forceinline__ void fetch(const float *plane, int col, unsigned lds_base, int lane, const Dims &dm) const
    {
        const float *src = plane + col + (lane & 3) * 4;
#pragma unroll
        for (int j = 0; j < kStage; ++j) {
            if (x0[j] + (lane >> 2) < dm.Wimg) {       // (lanes past the end of the image row stay out)
                const unsigned px = (unsigned)(pix[j] + (lane >> 2));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + px * (unsigned)dm.kv_sl),
                                                 (__attribute__((address_space(3))) void *)(uintptr_t)(lds_base + (unsigned)dst[j]),
                                                 16, 0, 0);
            }
        }
    }
    __device__ __forceinline__ static void wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
};

// ------------------------------------------------------------------ forward
// KB: blocks of 16 samples per (query row, view), P = 16 KB. A lane's IT samples of a view are the KB blocks of IT / KB
// query rows: the blocks of one row sit in the same 16 lanes, so what a row's blocks share (running maximum, sum,
// output columns) is combined inside a lane.
template <int D, int IT, int NW, int KB>
__global__ __launch_bounds__(NW *kWave) void fwd_slab_kernel(
    const float *__restrict__ q_, const float *__restrict__ k_, const float *__restrict__ v_,
    const float *__restrict__ coords_, float *__restrict__ out_, float *__restrict__ lse_, Dims dm, int nblk,
    int pitch, unsigned buf_bytes)
{
    constexpr int NSLAB = D / kSlabCols;
    constexpr int NR = IT / KB;                      // query rows a lane works on
    constexpr int RW = 4 * NR;                       // query rows per wave
    constexpr int RB = NW * RW;                      // query rows per workgroup
    static_assert(NR * KB == IT, "whole rows per lane");
    extern __shared__ __attribute__((aligned(16))) char slab[];
    const float4 *slab4 = reinterpret_cast<const float4 *>(slab);
    const unsigned slab_base = (unsigned)(uintptr_t)slab;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i3 = lane & 3, g4 = (lane >> 2) & 3, smp = lane & 15, rg = lane >> 4;
    const int blk = xcd_logical_block(blockIdx.x, gridDim.x);
    const int bh = blk / nblk, rb = blk - bh * nblk;
    const int b = bh / dm.H, h = bh - b * dm.H;
    const int VL = dm.V * dm.L;
    const float *qb = q_ + (size_t)((long long)b * dm.q_sb + (long long)h * dm.q_sh);
    const size_t kvb = dm.kv_plane(b, 0, h);
    const float2 *cb = reinterpret_cast<const float2 *>(coords_) + (size_t)b * VL * dm.N;
    const float qscale = dm.sm_scale * kLog2e;

    // the pieces of a 64-byte slab row in this lane's order (in 16-byte units)
    unsigned chv[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) chv[c] = (unsigned)((c + i3) & 3);

    // row r of this lane: query row rb * RB + wave * RW + 4 r + rg of the (batch, head); sample it: block it % KB of
    // row it / KB
    bool live[NR];
    unsigned coff[NR];
    float m[NR], lsum[NR], acc[NR][NSLAB];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int rr = rb * RB + wave * RW + 4 * r + rg;
        live[r] = rr < VL;
        const int rc = min(rr, VL - 1);
        coff[r] = (unsigned)rc * (unsigned)dm.N + (unsigned)smp;
        m[r] = kNegBig;
        lsum[r] = 0.f;
#pragma unroll
        for (int s = 0; s < NSLAB; ++s) acc[r][s] = 0.f;
    }

    // q goes through LDS too, 16 columns of the wave's RW rows at a time (a region per wave: no barrier): a load
    // issued behind the slab's loads would only return after them (loads return in order), at the start of
    // every K step. The piece for the next K step is requested before that step's slab and parked after the work
    // on the present step; lane i moves piece i & 3 of row i >> 2.
    float4 *qlds = reinterpret_cast<float4 *>(slab + 2 * buf_bytes) + wave * (RW * 4);
    unsigned qst_off;
    {
        const int rc = min(rb * RB + wave * RW + min(lane >> 2, RW - 1), VL - 1);
        const int s1 = rc / dm.L, l = rc - s1 * dm.L;
        qst_off = (unsigned)s1 * (unsigned)dm.q_sv + (unsigned)l * (unsigned)dm.q_sl + (unsigned)(lane & 3) * 4;
    }
    float4 qnext = *reinterpret_cast<const float4 *>(qb + qst_off);          // K slab 0 of the first view
    if (lane < 4 * RW) qlds[lane] = qnext;

    SlabStager<NW> stg;
    stg.init(wave, dm, pitch);
    // step ph of the walk: view ph / (2 NSLAB), K slabs first, then V slabs
    const int nsteps = dm.V * 2 * NSLAB;
    auto stage_fetch = [&](int ph) {
        const int s2 = ph / (2 * NSLAB), r = ph - s2 * (2 * NSLAB);
        stg.fetch((r < NSLAB ? k_ : v_) + kvb + (size_t)s2 * dm.kv_sv, (r % NSLAB) * kSlabCols,
                  slab_base + (unsigned)(ph & 1) * buf_bytes, lane, dm);
    };
    stage_fetch(0);
    SlabStager<NW>::wait();
    __syncthreads();

    int ph = 0;
    for (int s2 = 0; s2 < dm.V; ++s2) {
        // this lane's samples of the view
        unsigned off[IT][4];
        float w[IT][4], part[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            slab_sample(cb[coff[it / KB] + (unsigned)s2 * (unsigned)dm.P + (unsigned)(it % KB) * kSlabSamples], dm, pitch, g4,
                        off[it], w[it]);
            part[it] = 0.f;
        }
        // ---- logits: K slab by slab
#pragma unroll 1
        for (int s = 0; s < NSLAB; ++s, ++ph) {
            if (s + 1 < NSLAB) qnext = *reinterpret_cast<const float4 *>(qb + qst_off + (s + 1) * kSlabCols);
            stage_fetch(ph + 1);                      // (a K step is never the last one)
            const unsigned cur = (unsigned)(ph & 1) * (buf_bytes / 16);
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                float d[4];
                part[it] += slab_dot(slab4, qlds + ((it / KB) * 4 + rg) * 4, off[it], cur, chv, w[it], d);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (s + 1 < NSLAB && lane < 4 * RW) qlds[lane] = qnext;      // (this wave has read the present piece)
            SlabStager<NW>::wait();
            __syncthreads();
        }
        // ---- softmax bookkeeping of the view, row by row; the weights become p * w
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            float mx = kNegBig;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) mx = fmaxf(mx, part[r * KB + kb] * qscale);
            const float m_new = fmaxf(m[r], group16_max(mx));
            const float alpha = __builtin_amdgcn_exp2f(m[r] - m_new);
            m[r] = m_new;
            lsum[r] *= alpha;
#pragma unroll
            for (int s = 0; s < NSLAB; ++s) acc[r][s] *= alpha;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const int it = r * KB + kb;
                const float p = __builtin_amdgcn_exp2f(part[it] * qscale - m_new);
                lsum[r] += p;
#pragma unroll
                for (int t = 0; t < 4; ++t) w[it][t] *= p;
            }
        }
        // ---- out: V slab by slab
#pragma unroll
        for (int s = 0; s < NSLAB; ++s, ++ph) {
            if (s == NSLAB - 1) qnext = *reinterpret_cast<const float4 *>(qb + qst_off);      // the next view starts with K slab 0
            if (ph + 1 < nsteps) stage_fetch(ph + 1);
            const unsigned cur = (unsigned)(ph & 1) * (buf_bytes / 16);
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                acc[it / KB][s] += slab_axpy(slab4, off[it], cur, chv, w[it], lane);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (s == NSLAB - 1 && lane < 4 * RW) qlds[lane] = qnext;
            SlabStager<NW>::wait();
            __syncthreads();
        }
    }

    // ---- epilogue: lane j of a row's 16 lanes holds column 16 s + 4 (j & 3) + 2 * bit 3 + bit 2 of the row
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const float l16 = group_sum<16>(lsum[r]);
        if (!live[r]) continue;
        const int rr = rb * RB + wave * RW + 4 * r + rg;
        const int s1 = rr / dm.L, l = rr - s1 * dm.L;
        const size_t row = (((size_t)b * dm.V + s1) * dm.H + h) * dm.L + l;
        const float inv = 1.0f / l16;
        const int col = 4 * i3 + 2 * ((lane >> 3) & 1) + ((lane >> 2) & 1);
#pragma unroll
        for (int s = 0; s < NSLAB; ++s) out_[row * D + s * kSlabCols + col] = acc[r][s] * inv;
        if (smp == 0) lse_[row] = m[r] + __log2f(l16);
    }
}

// ------------------------------------------------------------------ backward, dq (`ops/triton.py:219-365` computes
// dq, dk and dv in one kernel; here dk/dv come from the cell-binned kernel, which takes (p, sm_scale * ds) of
// every sample from this one).
// Three walks per key view: the K slabs for the logits (q parked in LDS), the V slabs for dp = dout . v~ (dout
// parked the same way), then p = 2^(s - lse), ds = p (dp - delta), and the K slabs again for dq += ds * k~, the
// 16 samples of a row combined as in the forward's V walk. Covers the query rows of the (batch, head) pairs
// [bh0, bh0 + gridDim.x / nblk).
// CG: also the gradient of the coordinates (see bwd_dq_gather_kernel): the per-tap products q . K_t and dout . V_t
// are kept tap by tap over the slabs, and g_t = sm_scale * ds * (q . K_t) + p * (dout . V_t) meets the tap
// derivatives once per sample and view; two float atomics per sample (the heads share the coordinates).
template <int D, int IT, int NW, int KB, bool CG>
__global__ __launch_bounds__(NW *kWave) void bwd_dq_slab_kernel(
    const float *__restrict__ q_, const float *__restrict__ k_, const float *__restrict__ v_,
    const float *__restrict__ coords_, const float *__restrict__ out_, const float *__restrict__ lse_,
    const float *__restrict__ dout_, float *__restrict__ dq_, float2 *__restrict__ stats_,
    float2 *__restrict__ handed_, float *__restrict__ dcoords_, Dims dm, int bh0, int nblk, int pitch, unsigned buf_bytes)
{
    constexpr int NSLAB = D / kSlabCols;
    constexpr int NR = IT / KB, RW = 4 * NR, RB = NW * RW;       // query rows per lane, wave, workgroup (see the forward)
    static_assert(NR * KB == IT, "whole rows per lane");
    extern __shared__ __attribute__((aligned(16))) char slab[];
    const float4 *slab4 = reinterpret_cast<const float4 *>(slab);
    const unsigned slab_base = (unsigned)(uintptr_t)slab;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i3 = lane & 3, g4 = (lane >> 2) & 3, smp = lane & 15, rg = lane >> 4;
    const int blk = xcd_logical_block(blockIdx.x, gridDim.x);
    const int bhl = blk / nblk, rb = blk - bhl * nblk, bh = bh0 + bhl;
    const int b = bh / dm.H, h = bh - b * dm.H;
    const int VL = dm.V * dm.L;
    const float *qb = q_ + (size_t)((long long)b * dm.q_sb + (long long)h * dm.q_sh);
    const size_t kvb = dm.kv_plane(b, 0, h);
    const float2 *cb = reinterpret_cast<const float2 *>(coords_) + (size_t)b * VL * dm.N;
    const float qscale = dm.sm_scale * kLog2e;
    const int col = 4 * i3 + 2 * ((lane >> 3) & 1) + ((lane >> 2) & 1);      // this lane's column of a slab after slab_axpy

    unsigned chv[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) chv[c] = (unsigned)((c + i3) & 3);

    // contiguous row (out, dout, dq, lse) of query row rr of this (batch, head)
    auto row_of = [&](int rr) {
        const int s1 = rr / dm.L, l = rr - s1 * dm.L;
        return (((size_t)b * dm.V + s1) * dm.H + h) * dm.L + l;
    };
    bool live[NR];
    unsigned coff[NR];
    float lse[NR], delta[NR], acc[NR][NSLAB];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int rr = rb * RB + wave * RW + 4 * r + rg;
        live[r] = rr < VL;
        const int rc = min(rr, VL - 1);
        coff[r] = (unsigned)rc * (unsigned)dm.N + (unsigned)smp;
        const size_t row = row_of(rc);
        lse[r] = lse_[row];
        // delta = dout . out (the reference's _bwd_preprocess, ops/triton.py:197-215): 4 columns a lane
        float dl = 0.f;
#pragma unroll
        for (int j = 0; j < D / 64; ++j) {
            const float4 a = *reinterpret_cast<const float4 *>(dout_ + row * D + j * 64 + smp * 4);
            const float4 o = *reinterpret_cast<const float4 *>(out_ + row * D + j * 64 + smp * 4);
            dl = fmaf(a.x, o.x, fmaf(a.y, o.y, fmaf(a.z, o.z, fmaf(a.w, o.w, dl))));
        }
        if constexpr (D < 64) {
            if (smp < D / 4) {
                const float4 a = *reinterpret_cast<const float4 *>(dout_ + row * D + smp * 4);
                const float4 o = *reinterpret_cast<const float4 *>(out_ + row * D + smp * 4);
                dl = fmaf(a.x, o.x, fmaf(a.y, o.y, fmaf(a.z, o.z, a.w * o.w)));
            }
        }
        delta[r] = group_sum<16>(dl);
        if (stats_ && live[r] && smp == 0) stats_[row] = make_float2(lse[r], delta[r]);
#pragma unroll
        for (int s = 0; s < NSLAB; ++s) acc[r][s] = 0.f;
    }

    // q and dout through LDS, a slab ahead (see the forward): lane i moves piece i & 3 of the wave's row i >> 2
    float4 *xlds = reinterpret_cast<float4 *>(slab + 2 * buf_bytes) + wave * (RW * 4);
    unsigned qst_off;
    size_t dst_off;
    {
        const int rc = min(rb * RB + wave * RW + min(lane >> 2, RW - 1), VL - 1);
        const int s1 = rc / dm.L, l = rc - s1 * dm.L;
        qst_off = (unsigned)s1 * (unsigned)dm.q_sv + (unsigned)l * (unsigned)dm.q_sl + (unsigned)(lane & 3) * 4;
        dst_off = row_of(rc) * D + (size_t)(lane & 3) * 4;
    }
    float4 xnext = *reinterpret_cast<const float4 *>(qb + qst_off);
    if (lane < 4 * RW) xlds[lane] = xnext;

    SlabStager<NW> stg;
    stg.init(wave, dm, pitch);
    // step ph of the walk: view ph / (3 NSLAB): K slabs, V slabs, K slabs
    const int nsteps = dm.V * 3 * NSLAB;
    auto stage_fetch = [&](int ph) {
        const int s2 = ph / (3 * NSLAB), r = ph - s2 * (3 * NSLAB);
        stg.fetch(((r >= NSLAB && r < 2 * NSLAB) ? v_ : k_) + kvb + (size_t)s2 * dm.kv_sv, (r % NSLAB) * kSlabCols,
                  slab_base + (unsigned)(ph & 1) * buf_bytes, lane, dm);
    };
    stage_fetch(0);
    SlabStager<NW>::wait();
    __syncthreads();

    int ph = 0;
    for (int s2 = 0; s2 < dm.V; ++s2) {
        unsigned off[IT][4];
        float w[IT][4], ps[IT], pd[IT];
        constexpr int ITG = CG ? IT : 1;
        float dkt[ITG][4], dvt[ITG][4];          // CG: q . K_t and dout . V_t, tap by tap (the lane's order)
        float2 xy[ITG];
        int rot[ITG];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const float2 c = cb[coff[it / KB] + (unsigned)s2 * (unsigned)dm.P + (unsigned)(it % KB) * kSlabSamples];
            const int r = slab_sample(c, dm, pitch, g4, off[it], w[it]);
            ps[it] = 0.f;
            pd[it] = 0.f;
            if constexpr (CG) {
                xy[it] = c;
                rot[it] = r;
#pragma unroll
                for (int k = 0; k < 4; ++k) dkt[it][k] = dvt[it][k] = 0.f;
            }
        }
        // ---- logits: K slabs, q parked
#pragma unroll 1
        for (int s = 0; s < NSLAB; ++s, ++ph) {
            xnext = (s + 1 < NSLAB) ? *reinterpret_cast<const float4 *>(qb + qst_off + (s + 1) * kSlabCols)
                                    : *reinterpret_cast<const float4 *>(dout_ + dst_off);
            stage_fetch(ph + 1);
            const unsigned cur = (unsigned)(ph & 1) * (buf_bytes / 16);
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                float d[4];
                ps[it] += slab_dot(slab4, xlds + ((it / KB) * 4 + rg) * 4, off[it], cur, chv, w[it], d);
                if constexpr (CG) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) dkt[it][k] += d[k];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (lane < 4 * RW) xlds[lane] = xnext;
            SlabStager<NW>::wait();
            __syncthreads();
        }
        // ---- dp = dout . v~: V slabs, dout parked
#pragma unroll 1
        for (int s = 0; s < NSLAB; ++s, ++ph) {
            if (s + 1 < NSLAB) xnext = *reinterpret_cast<const float4 *>(dout_ + dst_off + (s + 1) * kSlabCols);
            stage_fetch(ph + 1);
            const unsigned cur = (unsigned)(ph & 1) * (buf_bytes / 16);
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                float d[4];
                pd[it] += slab_dot(slab4, xlds + ((it / KB) * 4 + rg) * 4, off[it], cur, chv, w[it], d);
                if constexpr (CG) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) dvt[it][k] += d[k];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (s + 1 < NSLAB && lane < 4 * RW) xlds[lane] = xnext;
            SlabStager<NW>::wait();
            __syncthreads();
        }
        // ---- p, ds; the pair goes to the dk/dv kernel ([pair of this launch][s1][l][sample]); the weights become ds * w
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int r = it / KB;
            const float p = __builtin_amdgcn_exp2f(ps[it] * qscale - lse[r]);
            const float ds = p * (pd[it] - delta[r]);
            if (handed_ && live[r])
                handed_[(size_t)bhl * VL * dm.N + coff[r] + (unsigned)s2 * (unsigned)dm.P + (unsigned)(it % KB) * kSlabSamples] =
                    make_float2(p, ds * dm.sm_scale);
            if constexpr (CG) {
                // the tap derivatives (zero for a tap outside the image) in the lane's tap order, times g_t
                TapGrads tg = make_tap_grads(xy[it].x, xy[it].y, dm.Wimg, dm.Himg);
                slab_rotate(tg.gx, rot[it]);
                slab_rotate(tg.gy, rot[it]);
                const float a = ds * dm.sm_scale;
                float gx = 0.f, gy = 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float gk = fmaf(a, dkt[it][k], p * dvt[it][k]);
                    gx = fmaf(tg.gx[k], gk, gx);
                    gy = fmaf(tg.gy[k], gk, gy);
                }
                if (live[r]) {
                    float *dst = dcoords_ + 2 * ((size_t)b * VL * dm.N + coff[r] + (unsigned)s2 * (unsigned)dm.P + (unsigned)(it % KB) * kSlabSamples);
                    atomicAdd(dst, gx);
                    atomicAdd(dst + 1, gy);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) w[it][t] *= ds;
        }
        // ---- dq += ds * k~: K slabs again
#pragma unroll
        for (int s = 0; s < NSLAB; ++s, ++ph) {
            if (s == NSLAB - 1) xnext = *reinterpret_cast<const float4 *>(qb + qst_off);      // the next view starts with q, slab 0
            if (ph + 1 < nsteps) stage_fetch(ph + 1);
            const unsigned cur = (unsigned)(ph & 1) * (buf_bytes / 16);
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                acc[it / KB][s] += slab_axpy(slab4, off[it], cur, chv, w[it], lane);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (s == NSLAB - 1 && lane < 4 * RW) xlds[lane] = xnext;
            SlabStager<NW>::wait();
            __syncthreads();
        }
    }

#pragma unroll
    for (int r = 0; r < NR; ++r) {
        if (!live[r]) continue;
        const size_t row = row_of(rb * RB + wave * RW + 4 * r + rg);
#pragma unroll
        for (int s = 0; s < NSLAB; ++s) dq_[row * D + s * kSlabCols + col] = acc[r][s] * dm.sm_scale;
    }
}

}  // namespace dsdpa
