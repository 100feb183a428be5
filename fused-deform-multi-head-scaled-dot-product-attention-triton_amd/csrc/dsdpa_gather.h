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
    size_t row;        // linear query row in [B][V][H][L]
    size_t kv_base;    // element offset of plane (b, view 0, h) in k/v/dk/dv
    size_t crow;       // float2 offset of coords[b][s1][l][0][0]
    int view_stride;   // elements between consecutive views of one (b, h)
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
    c.kv_base = ((size_t)b * dm.V * dm.H + h) * (size_t)dm.L * D;
    c.crow = (((size_t)b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
    c.view_stride = dm.H * dm.L * D;
    return c;
}

// Each lane builds the descriptor of sample c0+lane and parks it in this wave's LDS slice: the four
// weights and the four taps' BYTE offsets from plane (b, view 0, h), unsigned 32-bit (one batch item of a
// tensor stays below 2^30 elements, so below 2^32 bytes). With a wave-uniform base pointer a gather is then
// "scalar base + 32-bit lane offset", one add per tap instead of 64-bit address arithmetic.
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
    int ebase = (nc / dm.P) * rc.view_stride;
    float4 w = valid ? make_float4(tp.w[0], tp.w[1], tp.w[2], tp.w[3]) : make_float4(0.f, 0.f, 0.f, 0.f);
    uint4 e = make_uint4((unsigned)(ebase + tp.pix[0] * D) * BYTES, (unsigned)(ebase + tp.pix[1] * D) * BYTES,
                         (unsigned)(ebase + tp.pix[2] * D) * BYTES, (unsigned)(ebase + tp.pix[3] * D) * BYTES);
    wave_lds_sync();          // the previous chunk's readers are done
    s_w[lane] = w;
    s_e[lane] = e;
    wave_lds_sync();
}

__device__ __forceinline__ uint4 lane_offsets(const uint4 &e, unsigned lane_byte)
{
    return make_uint4(e.x + lane_byte, e.y + lane_byte, e.z + lane_byte, e.w + lane_byte);
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
template <typename S, int D, int DC>
__global__ __launch_bounds__(kGatherWaves *kWave) void fwd_gather_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, void *__restrict__ out_, float *__restrict__ lse_, Dims dm)
{
    constexpr int G = D / DC;        // lanes per sample
    constexpr int NS = kWave / G;    // samples in flight per wave
    constexpr int ITS = G;           // slot iterations per 64-sample chunk
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
    const float2 *coords = (const float2 *)coords_;

    // fp32 storage: q widened and pre-scaled; 16-bit storage: q kept as packed pairs for the dot-product
    // instructions and the scale applied to the logit
    constexpr bool kPacked = S::kBytes == 2;
    float qf[DC];
    uint32_t qp[kPacked ? DC / 2 : 1];
    const float qscale = dm.sm_scale * kLog2e;
    if constexpr (kPacked) {
        load_packed<S, DC>((const char *)q_ + (rc.row * D + lane_elem) * S::kBytes, qp);
    } else {
        load_chunk<S, DC>((const char *)q_ + (rc.row * D + lane_elem) * S::kBytes, qf);
#pragma unroll
        for (int d = 0; d < DC; ++d) qf[d] *= qscale;
    }

    float m = kNegBig, lsum = 0.f, acc[DC];
#pragma unroll
    for (int d = 0; d < DC; ++d) acc[d] = 0.f;

    for (int c0 = 0; c0 < dm.N; c0 += kWave) {
        stage_descriptors<D, S::kBytes>(coords, rc, dm, c0, lane, s_w[wave], s_e[wave]);
        const int cnt = min(kWave, dm.N - c0);
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
    float *dkb = dk_acc + rc.kv_base + lane_elem;
    float *dvb = dv_acc + rc.kv_base + lane_elem;
    const float2 *coords = (const float2 *)coords_;

    float qf[DC], dof[DC], of[DC];
    const size_t roff = (rc.row * D + lane_elem) * S::kBytes;
    load_chunk<S, DC>((const char *)q_ + roff, qf);
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
template <typename S, int D, int DC, bool CG>
__global__ __launch_bounds__(kGatherWaves *kWave) void bwd_dq_gather_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, const void *__restrict__ out_, const float *__restrict__ lse_,
    const void *__restrict__ dout_, void *__restrict__ dq_, float2 *__restrict__ stats_,
    float *__restrict__ dcoords_, Dims dm)
{
    constexpr int G = D / DC;
    constexpr int NS = kWave / G;
    constexpr int ITS = G;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    __shared__ float4 s_w[kGatherWaves][kWave];
    __shared__ uint4 s_e[kGatherWaves][kWave];
    __shared__ float4 s_gx[CG ? kGatherWaves : 1][kWave];
    __shared__ float4 s_gy[CG ? kGatherWaves : 1][kWave];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    const int work = xcd_logical_block(blockIdx.x, gridDim.x) * kGatherWaves + wave;
    if (work >= dm.rows) return;
    const RowCtx rc = decode_row(work, dm, D);
    const int g = lane % G, slot = lane / G, lane_elem = g * DC;
    const unsigned lane_byte = (unsigned)lane_elem * S::kBytes;
    const char *kb = (const char *)k_ + rc.kv_base * S::kBytes;
    const char *vb = (const char *)v_ + rc.kv_base * S::kBytes;
    const float2 *coords = (const float2 *)coords_;

    constexpr bool kPacked = S::kBytes == 2 && !CG;
    float qf[DC], dof[DC], of[DC];
    uint32_t dop[kPacked ? DC / 2 : 1];
    const size_t roff = (rc.row * D + lane_elem) * S::kBytes;
    load_chunk<S, DC>((const char *)q_ + roff, qf);
    load_chunk<S, DC>((const char *)dout_ + roff, dof);
    load_chunk<S, DC>((const char *)out_ + roff, of);
    if constexpr (kPacked) load_packed<S, DC>((const char *)dout_ + roff, dop);
    float delta = 0.f;
#pragma unroll
    for (int d = 0; d < DC; ++d) delta = fmaf(dof[d], of[d], delta);
    delta = group_sum<G>(delta);
    const float qscale = dm.sm_scale * kLog2e;
    const float lse = lse_[rc.row];
    if (stats_ && lane == 0) stats_[rc.row] = make_float2(lse, delta);     // null: a launch of its own does it

    float dqa[DC];
#pragma unroll
    for (int d = 0; d < DC; ++d) dqa[d] = 0.f;

    for (int c0 = 0; c0 < dm.N; c0 += kWave) {
        stage_descriptors<D, S::kBytes>(coords, rc, dm, c0, lane, s_w[wave], s_e[wave]);
        if constexpr (CG) {
            // (stage_descriptors ends with a wave-level LDS sync; these two arrays are read after the
            // next one, and their previous readers finished before the sync at its start)
            const int n = min(c0 + lane, dm.N - 1);
            const float2 xy = coords[rc.crow + n];
            const TapGrads tg = make_tap_grads(xy.x, xy.y, dm.Wimg, dm.Himg);
            s_gx[wave][lane] = make_float4(tg.gx[0], tg.gx[1], tg.gx[2], tg.gx[3]);
            s_gy[wave][lane] = make_float4(tg.gy[0], tg.gy[1], tg.gy[2], tg.gy[3]);
            wave_lds_sync();
        }
        const int cnt = min(kWave, dm.N - c0);
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
#pragma unroll
                for (int d = 0; d < DC; ++d) dqa[d] = fmaf(ds, kk[d], dqa[d]);
            }
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
