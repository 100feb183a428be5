// "Plane" kernels: query-stationary forward and dq with the current key view's
// K and V planes staged in LDS, for shapes where one (b, s2, h) plane pair
// (2 * L * D * element size) fits next to the per-wave tap descriptors.
//
// A workgroup of 16 waves owns 16*QW consecutive query rows of one (b, h) (rows
// are counted over (s1, l), so a workgroup may straddle two query views) and
// walks the V key views: stage K_s2 and V_s2 (coalesced 16-byte loads, kept in
// the storage type), barrier, every wave runs its QW rows against the staged
// planes -- the 4-tap gathers are ds_read_b128 of D-contiguous runs, G lanes per
// sample as in the gather kernels -- barrier, next view. The online-softmax
// state (forward) or dq accumulator (backward) of each row stays in registers
// across the views.
#pragma once
#include "dsdpa_common.h"
#include "dsdpa_gather.h"

namespace dsdpa {

constexpr int kPlaneWaves = 16;
constexpr int kPlaneDescBytes = kPlaneWaves * kWave * 32;   // float4 weights + int4 offsets per sample slot

__device__ __forceinline__ void stage_plane(unsigned char *dst, const char *src, int bytes)
{
    const uint4 *s4 = reinterpret_cast<const uint4 *>(src);
    uint4 *d4 = reinterpret_cast<uint4 *>(dst);
    const int n16 = bytes >> 4;
    for (int i = threadIdx.x; i < n16; i += kPlaneWaves * kWave) d4[i] = s4[i];
}

// Tap descriptors of one (query row, key view): lane n handles sample c0+n.
// Offsets are BYTE offsets into the staged plane.
template <typename S, int D>
__device__ __forceinline__ void stage_plane_descriptors(float2 xy, bool valid, int lane,
                                                        int Wimg, int Himg, float4 *s_w, int4 *s_e)
{
    const Taps tp = make_taps(xy.x, xy.y, Wimg, Himg);
    constexpr int kRow = D * S::kBytes;
    const float4 w = valid ? make_float4(tp.w[0], tp.w[1], tp.w[2], tp.w[3]) : make_float4(0.f, 0.f, 0.f, 0.f);
    const int4 e = make_int4(tp.pix[0] * kRow, tp.pix[1] * kRow, tp.pix[2] * kRow, tp.pix[3] * kRow);
    wave_lds_sync();
    s_w[lane] = w;
    s_e[lane] = e;
    wave_lds_sync();
}

template <typename S, int DC>
__device__ __forceinline__ void blend_taps_lds(const unsigned char *base, const int4 &e, const float4 &w,
                                               int lane_byte, float (&dst)[DC])
{
    float t0[DC], t1[DC], t2[DC], t3[DC];
    load_chunk<S, DC>(base + e.x + lane_byte, t0);
    load_chunk<S, DC>(base + e.y + lane_byte, t1);
    load_chunk<S, DC>(base + e.z + lane_byte, t2);
    load_chunk<S, DC>(base + e.w + lane_byte, t3);
#pragma unroll
    for (int d = 0; d < DC; ++d)
        dst[d] = fmaf(w.x, t0[d], fmaf(w.y, t1[d], fmaf(w.z, t2[d], w.w * t3[d])));
}

template <typename S, int DC>
__device__ __forceinline__ void accumulate_taps_lds(const unsigned char *base, const int4 &e, const float4 &c,
                                                    int lane_byte, float (&acc)[DC])
{
    float t0[DC], t1[DC], t2[DC], t3[DC];
    load_chunk<S, DC>(base + e.x + lane_byte, t0);
    load_chunk<S, DC>(base + e.y + lane_byte, t1);
    load_chunk<S, DC>(base + e.z + lane_byte, t2);
    load_chunk<S, DC>(base + e.w + lane_byte, t3);
#pragma unroll
    for (int d = 0; d < DC; ++d)
        acc[d] = fmaf(c.x, t0[d], fmaf(c.y, t1[d], fmaf(c.z, t2[d], fmaf(c.w, t3[d], acc[d]))));
}

struct PlaneBlock {
    int b, h, qbase;     // first query row (index over (s1, l)) of this workgroup
};

__device__ __forceinline__ PlaneBlock decode_plane_block(const Dims &dm, int rows_per_block)
{
    const int nq = dm.V * dm.L;
    const int chunks = (nq + rows_per_block - 1) / rows_per_block;
    const int bid = xcd_logical_block(blockIdx.x, gridDim.x);
    PlaneBlock pb;
    const int bh = bid / chunks;
    pb.qbase = (bid % chunks) * rows_per_block;
    pb.h = bh % dm.H;
    pb.b = bh / dm.H;
    return pb;
}

// ------------------------------------------------------------------ forward
template <typename S, int D, int DC, int QW>
__global__ __launch_bounds__(kPlaneWaves *kWave) void fwd_plane_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, void *__restrict__ out_, float *__restrict__ lse_, Dims dm)
{
    constexpr int G = D / DC;
    constexpr int NS = kWave / G;
    constexpr int ITS = G;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int plane_bytes = dm.L * D * S::kBytes;
    unsigned char *sK = smem, *sV = smem + plane_bytes;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float4 *s_w = reinterpret_cast<float4 *>(smem + 2 * plane_bytes) + wave * kWave;
    int4 *s_e = reinterpret_cast<int4 *>(smem + 2 * plane_bytes + kPlaneWaves * kWave * 16) + wave * kWave;

    const PlaneBlock pb = decode_plane_block(dm, kPlaneWaves * QW);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const float2 *coords = reinterpret_cast<const float2 *>(coords_);

    float qf[QW][DC], acc[QW][DC], m[QW], lsum[QW];
    size_t row[QW], crow[QW];
    bool have[QW];
#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
        const int qidx = pb.qbase + wave * QW + qi;
        have[qi] = qidx < nq;
        const int qc = have[qi] ? qidx : nq - 1;
        const int s1 = qc / dm.L, l = qc % dm.L;
        row[qi] = (((size_t)pb.b * dm.V + s1) * dm.H + pb.h) * dm.L + l;
        crow[qi] = (((size_t)pb.b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
        load_chunk<S, DC>((const char *)q_ + (row[qi] * D + lane_elem) * S::kBytes, qf[qi]);
        m[qi] = kNegBig;
        lsum[qi] = 0.f;
#pragma unroll
        for (int d = 0; d < DC; ++d) { qf[qi][d] *= qscale; acc[qi][d] = 0.f; }
    }

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = (((size_t)pb.b * dm.V + s2) * dm.H + pb.h) * (size_t)dm.L * D * S::kBytes;
        __syncthreads();                                       // the previous view's readers are done
        stage_plane(sK, (const char *)k_ + plane, plane_bytes);
        stage_plane(sV, (const char *)v_ + plane, plane_bytes);
        __syncthreads();
#pragma unroll
        for (int qi = 0; qi < QW; ++qi) {
            if (!have[qi]) continue;                           // wave-uniform
            const float2 *cq = coords + crow[qi] + (size_t)s2 * dm.P;
            for (int c0 = 0; c0 < dm.P; c0 += kWave) {
                const float2 xy = cq[min(c0 + lane, dm.P - 1)];
                stage_plane_descriptors<S, D>(xy, c0 + lane < dm.P, lane, dm.Wimg, dm.Himg, s_w, s_e);
                const int cnt = min(kWave, dm.P - c0);
                float sv[ITS];
                float mc = kNegBig;
#pragma unroll
                for (int it = 0; it < ITS; ++it) {
                    sv[it] = kNegBig;
                    if (it * NS < cnt) {
                        const int j = it * NS + slot;
                        const float4 w = s_w[j];
                        const int4 e = s_e[j];
                        float kk[DC];
                        blend_taps_lds<S, DC>(sK, e, w, lane_byte, kk);
                        float dot = 0.f;
#pragma unroll
                        for (int d = 0; d < DC; ++d) dot = fmaf(qf[qi][d], kk[d], dot);
                        dot = group_sum<G>(dot);
                        sv[it] = (j < cnt) ? dot : kNegBig;
                        mc = fmaxf(mc, sv[it]);
                    }
                }
                const float m_new = fmaxf(m[qi], mc);
                const float alpha = __builtin_amdgcn_exp2f(m[qi] - m_new);
                m[qi] = m_new;
                lsum[qi] *= alpha;
#pragma unroll
                for (int d = 0; d < DC; ++d) acc[qi][d] *= alpha;
#pragma unroll
                for (int it = 0; it < ITS; ++it) {
                    if (it * NS < cnt) {
                        const int j = it * NS + slot;
                        const float p = (j < cnt) ? __builtin_amdgcn_exp2f(sv[it] - m_new) : 0.f;
                        lsum[qi] += p;
                        const float4 w = s_w[j];
                        const int4 e = s_e[j];
                        const float4 c = make_float4(p * w.x, p * w.y, p * w.z, p * w.w);
                        accumulate_taps_lds<S, DC>(sV, e, c, lane_byte, acc[qi]);
                    }
                }
            }
        }
    }

#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
        if (!have[qi]) continue;
        float mm = m[qi], ll = lsum[qi];
#pragma unroll
        for (int off = G; off < kWave; off <<= 1) {
            const float mo = __shfl_xor(mm, off, kWave);
            const float lo = __shfl_xor(ll, off, kWave);
            const float mn = fmaxf(mm, mo);
            const float a = __builtin_amdgcn_exp2f(mm - mn), bsc = __builtin_amdgcn_exp2f(mo - mn);
            ll = ll * a + lo * bsc;
#pragma unroll
            for (int d = 0; d < DC; ++d) {
                const float ao = __shfl_xor(acc[qi][d], off, kWave);
                acc[qi][d] = acc[qi][d] * a + ao * bsc;
            }
            mm = mn;
        }
        if (slot == 0) {
            const float inv = 1.0f / ll;
#pragma unroll
            for (int d = 0; d < DC; ++d) acc[qi][d] *= inv;
            store_chunk<S, DC>((char *)out_ + (row[qi] * D + lane_elem) * S::kBytes, acc[qi]);
            if (g == 0) lse_[row[qi]] = mm + __log2f(ll);
        }
    }
}

// ------------------------------------------------------------------ backward: dq and delta
template <typename S, int D, int DC, int QW>
__global__ __launch_bounds__(kPlaneWaves *kWave) void bwd_dq_plane_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, const void *__restrict__ out_, const float *__restrict__ lse_,
    const void *__restrict__ dout_, void *__restrict__ dq_, float *__restrict__ delta_, Dims dm)
{
    constexpr int G = D / DC;
    constexpr int NS = kWave / G;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int plane_bytes = dm.L * D * S::kBytes;
    unsigned char *sK = smem, *sV = smem + plane_bytes;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float4 *s_w = reinterpret_cast<float4 *>(smem + 2 * plane_bytes) + wave * kWave;
    int4 *s_e = reinterpret_cast<int4 *>(smem + 2 * plane_bytes + kPlaneWaves * kWave * 16) + wave * kWave;

    const PlaneBlock pb = decode_plane_block(dm, kPlaneWaves * QW);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const float2 *coords = reinterpret_cast<const float2 *>(coords_);

    float qf[QW][DC], dof[QW][DC], dqa[QW][DC], lse[QW], delta[QW];
    size_t row[QW], crow[QW];
    bool have[QW];
#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
        const int qidx = pb.qbase + wave * QW + qi;
        have[qi] = qidx < nq;
        const int qc = have[qi] ? qidx : nq - 1;
        const int s1 = qc / dm.L, l = qc % dm.L;
        row[qi] = (((size_t)pb.b * dm.V + s1) * dm.H + pb.h) * dm.L + l;
        crow[qi] = (((size_t)pb.b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
        const size_t roff = (row[qi] * D + lane_elem) * S::kBytes;
        float of[DC];
        load_chunk<S, DC>((const char *)q_ + roff, qf[qi]);
        load_chunk<S, DC>((const char *)dout_ + roff, dof[qi]);
        load_chunk<S, DC>((const char *)out_ + roff, of);
        float dl = 0.f;
#pragma unroll
        for (int d = 0; d < DC; ++d) { dl = fmaf(dof[qi][d], of[d], dl); dqa[qi][d] = 0.f; }
        delta[qi] = group_sum<G>(dl);
        lse[qi] = lse_[row[qi]];
        if (have[qi] && lane == 0) delta_[row[qi]] = delta[qi];
    }

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = (((size_t)pb.b * dm.V + s2) * dm.H + pb.h) * (size_t)dm.L * D * S::kBytes;
        __syncthreads();
        stage_plane(sK, (const char *)k_ + plane, plane_bytes);
        stage_plane(sV, (const char *)v_ + plane, plane_bytes);
        __syncthreads();
#pragma unroll
        for (int qi = 0; qi < QW; ++qi) {
            if (!have[qi]) continue;
            const float2 *cq = coords + crow[qi] + (size_t)s2 * dm.P;
            for (int c0 = 0; c0 < dm.P; c0 += kWave) {
                const float2 xy = cq[min(c0 + lane, dm.P - 1)];
                stage_plane_descriptors<S, D>(xy, c0 + lane < dm.P, lane, dm.Wimg, dm.Himg, s_w, s_e);
                const int cnt = min(kWave, dm.P - c0);
                for (int j0 = 0; j0 < cnt; j0 += NS) {
                    const int j = j0 + slot;
                    const float4 w = s_w[j];
                    const int4 e = s_e[j];
                    float kk[DC], vv[DC];
                    blend_taps_lds<S, DC>(sK, e, w, lane_byte, kk);
                    blend_taps_lds<S, DC>(sV, e, w, lane_byte, vv);
                    float dot = 0.f, dp = 0.f;
#pragma unroll
                    for (int d = 0; d < DC; ++d) {
                        dot = fmaf(qf[qi][d], kk[d], dot);
                        dp = fmaf(dof[qi][d], vv[d], dp);
                    }
                    dot = group_sum<G>(dot);
                    dp = group_sum<G>(dp);
                    const float p = (j < cnt) ? __builtin_amdgcn_exp2f(dot * qscale - lse[qi]) : 0.f;
                    const float ds = p * (dp - delta[qi]);
#pragma unroll
                    for (int d = 0; d < DC; ++d) dqa[qi][d] = fmaf(ds, kk[d], dqa[qi][d]);
                }
            }
        }
    }

#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
        if (!have[qi]) continue;
#pragma unroll
        for (int off = G; off < kWave; off <<= 1) {
#pragma unroll
            for (int d = 0; d < DC; ++d) dqa[qi][d] += __shfl_xor(dqa[qi][d], off, kWave);
        }
        if (slot == 0) {
#pragma unroll
            for (int d = 0; d < DC; ++d) dqa[qi][d] *= dm.sm_scale;
            store_chunk<S, DC>((char *)dq_ + (row[qi] * D + lane_elem) * S::kBytes, dqa[qi]);
        }
    }
}

}  // namespace dsdpa
