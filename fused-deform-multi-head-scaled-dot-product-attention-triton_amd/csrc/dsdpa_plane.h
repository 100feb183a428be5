// "Plane" kernels: query-stationary forward and dq with the current key view's
// K and V planes staged in LDS, for shapes where one (b, s2, h) plane pair
// fits next to the per-wave tap descriptors.
//
// A workgroup of 16 waves owns 16*QW consecutive query rows of one (b, h) (rows
// are counted over (s1, l), so a workgroup may straddle two query views) and
// walks the V key views: stage K_s2 and V_s2 (coalesced 16-byte loads, kept in
// the storage type), barrier, every wave runs its QW rows against the staged
// planes, barrier, next view. The online-softmax state (forward) or the dq
// accumulator (backward) of each row stays in registers across the views.
//
// LDS image of a view: pixel p of the plane owns the 2*ROW bytes at (p + 1) * 2*ROW
// (ROW = D * element size), with one zeroed pad pixel before pixel 0 and one after
// pixel L-1. Slot q = p + 1 holds its K row in the first half when q is even and in
// the second half when q is odd, the V row in the other half:
//     K(q) = q*2*ROW + (q & 1)*ROW        V(q) = K(q) ^ ROW
//     K(q+1) = V(q) + 2*ROW               V(q+1) = K(q) + 2*ROW
// A sample's four taps are then two base addresses -- K of (row0, x0) and of
// (row1, x0), x0 in [-1, W-1] NOT clamped -- one XOR each, and compile-time
// offsets. A tap that falls outside the image carries weight 0 and reads either a
// pad or a neighbouring real pixel, never anything non-finite the caller did not
// put there. The gathers are ds_read_b128 of D-contiguous runs, G lanes per
// sample as in the gather kernels.
//
// Why the alternation: the LDS has 64 four-byte banks (256 bytes per clock) and
// serves a ds_read_b128 32 lanes at a time. A 128-byte row covers half the banks,
// so four rows gathered by 32 lanes take 2 clocks when two of them lie in each
// half and up to 4 when they share one (measured: 170 vs 103 bytes/clock/CU). With
// K always in the first half every K gather would be the 4-clock case. With the
// alternation the half is the parity of q, and the descriptors of a row are laid
// out so that consecutive samples alternate parity (paired_position below).
#pragma once
#include "dsdpa_common.h"

namespace dsdpa {

constexpr int kPlaneWaves = 16;

// LDS addresses as plain 32-bit numbers: the tap addresses are sums and XORs of byte offsets, and a
// pointer made from the finished number costs no instruction (adding offsets to a generic pointer to
// the dynamic LDS block costs an add per pointer). The XOR needs the block aligned to 2*ROW.
using lds_bytes = __attribute__((address_space(3))) const unsigned char *;
__device__ __forceinline__ uint32_t lds_offset(const void *p) { return (uint32_t)(size_t)(lds_bytes)p; }
__device__ __forceinline__ const unsigned char *lds_at(uint32_t off) { return (const unsigned char *)(lds_bytes)(size_t)off; }
constexpr int kPlaneLdsAlign = 2048;   // 2*ROW for the widest row (D = 256, fp32)
constexpr int kPlaneDescBytes = kPlaneWaves * kWave * (16 + 8);   // float4 weights + int2 base offsets

template <typename S, int D>
__host__ __device__ constexpr int plane_lds_bytes(int L) { return (L + 2) * 2 * D * S::kBytes; }

// global [L][D] plane -> LDS rows 1..L of the interleaved image (which = 0: K half, 1: V half)
template <typename S, int D>
__device__ __forceinline__ void stage_plane(unsigned char *lds, const char *src, int L, int which)
{
    constexpr int kRow = D * S::kBytes;
    constexpr int kChunksPerRow = kRow / 16;
    const uint4 *s4 = reinterpret_cast<const uint4 *>(src);
    const int n16 = L * kChunksPerRow;
    for (int i = threadIdx.x; i < n16; i += kPlaneWaves * kWave) {
        const int q = i / kChunksPerRow + 1, c = i % kChunksPerRow;
        *reinterpret_cast<uint4 *>(lds + (size_t)q * 2 * kRow + ((q & 1) ^ which) * kRow + c * 16) = s4[i];
    }
}

template <typename S, int D>
__device__ __forceinline__ void zero_plane_pads(unsigned char *lds, int L)
{
    constexpr int kRow = D * S::kBytes;
    constexpr int kChunks = 2 * kRow / 16;
    for (int i = threadIdx.x; i < 2 * kChunks; i += kPlaneWaves * kWave) {
        const int pad = i / kChunks, c = i % kChunks;
        *reinterpret_cast<uint4 *>(lds + (size_t)(pad ? L + 1 : 0) * 2 * kRow + c * 16) = make_uint4(0, 0, 0, 0);
    }
}

// Where lane `lane` parks its sample inside its block of descriptors (block = the lanes in `block`,
// positions counted from 0): the valid samples first, alternating parity class 0, 1, 0, 1, ... for as
// long as both classes last, then the rest of the larger class; the invalid lanes (beyond P) behind
// them. Any four consecutive positions then gather two rows from each half of the bank line.
__device__ __forceinline__ int paired_position(bool valid, int cls, int lane, unsigned long long block)
{
    const unsigned long long m0 = __ballot(valid && cls == 0) & block;
    const unsigned long long m1 = __ballot(valid && cls != 0) & block;
    const unsigned long long mi = __ballot(!valid) & block;
    const unsigned long long below = (1ull << lane) - 1ull;
    const int n0 = __popcll(m0), n1 = __popcll(m1), np = min(n0, n1);
    const int r = __popcll((cls ? m1 : m0) & below);
    const int pos_valid = r < np ? 2 * r + (cls ? 1 : 0) : np + r;
    return valid ? pos_valid : n0 + n1 + __popcll(mi & below);
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

// Descriptor table. The descriptors depend on the coordinates only, not on the head, and computing one
// costs about as many instructions as consuming two samples; so one small kernel computes them once per
// call -- one thread per coordinate pair, same order (b, s1, l, s2, p) as the coordinates -- and the
// plane kernels of all H heads read them back: 16 bytes of weights and the two K slot codes
// 2*q + (q & 1) (byte offset / ROW, so the table does not depend on the head width or storage type)
// packed into one 32-bit word. Within every run of up to 64 samples of one (b, s1, l, s2) the entries
// are stored in paired_position order.
constexpr int kDescThreads = 256;

static __global__ __launch_bounds__(kDescThreads) void plane_descriptor_kernel(
    const float *__restrict__ coords_, Dims dm, float4 *__restrict__ desc_w, uint32_t *__restrict__ desc_e)
{
    const int lane = threadIdx.x & 63;
    const long long wave = ((long long)blockIdx.x * kDescThreads + threadIdx.x) >> 6;
    const long long nblk = (long long)dm.B * dm.V * dm.L * dm.V;        // (b, s1, l, s2) runs of P samples
    long long blk;
    int n;                                                              // sample index inside the run
    unsigned long long group;                                           // lanes that share a run
    if (dm.P <= 32) {                                                   // two runs per wave
        blk = wave * 2 + (lane >> 5);
        n = lane & 31;
        group = lane < 32 ? 0xffffffffull : 0xffffffff00000000ull;
    } else {                                                            // one 64-sample piece of a run per wave
        const int pieces = (dm.P + 63) / 64;
        blk = wave / pieces;
        n = (int)(wave % pieces) * 64 + lane;
        group = ~0ull;
    }
    const bool valid = blk < nblk && n < dm.P;
    const long long src = valid ? blk * dm.P + n : 0;
    const float2 xy = reinterpret_cast<const float2 *>(coords_)[src];
    const Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
    const int x0u = min(max(tp.x0, -1), dm.Wimg - 1);
    const int cy0 = min(max(tp.y0, 0), dm.Himg - 1), cy1 = min(max(tp.y0 + 1, 0), dm.Himg - 1);
    const int qt = cy0 * dm.Wimg + x0u + 1, qb = cy1 * dm.Wimg + x0u + 1;
    const int pos = paired_position(valid, qt & 1, lane, group) + (dm.P <= 32 ? 0 : (n & ~63));
    if (valid) {
        const long long dst = blk * dm.P + pos;
        desc_w[dst] = make_float4(tp.w[0], tp.w[1], tp.w[2], tp.w[3]);
        desc_e[dst] = (uint32_t)(2 * qt + (qt & 1)) | ((uint32_t)(2 * qb + (qb & 1)) << 16);
    }
}

// Descriptors for two rows of a wave and one key view in one 64-lane pass (the PAIR instantiations,
// launched when P <= 32 and QW is even): lanes 0-31 take the even row, 32-63 the odd one, parked at
// descriptor slots 0.. and 32..   d_even / d_odd: index of the rows' first table entry for this view.
template <typename S, int D>
__device__ __forceinline__ void stage_pair_descriptors(const float4 *__restrict__ desc_w,
                                                       const uint32_t *__restrict__ desc_e, size_t d_even,
                                                       size_t d_odd, int P, int lane, float4 *s_w, int2 *s_e)
{
    constexpr int kRow = D * S::kBytes;
    const int n = lane & 31;
    const bool valid = n < P;
    const size_t i = ((lane < 32) ? d_even : d_odd) + (valid ? n : 0);
    float4 w = desc_w[i];
    const uint32_t c = desc_e[i];
    if (!valid) w = make_float4(0.f, 0.f, 0.f, 0.f);
    wave_lds_sync();
    s_w[lane] = w;
    s_e[lane] = make_int2((int)(c & 0xffffu) * kRow, (int)(c >> 16) * kRow);
    wave_lds_sync();
}

// One row, samples c0 .. c0+63.
template <typename S, int D>
__device__ __forceinline__ void stage_row_descriptors(const float4 *__restrict__ desc_w,
                                                      const uint32_t *__restrict__ desc_e, size_t d_row, int P,
                                                      int c0, int lane, float4 *s_w, int2 *s_e)
{
    constexpr int kRow = D * S::kBytes;
    const int n = c0 + lane;
    const bool valid = n < P;
    const size_t i = d_row + (valid ? n : 0);
    float4 w = desc_w[i];
    const uint32_t c = desc_e[i];
    if (!valid) w = make_float4(0.f, 0.f, 0.f, 0.f);
    wave_lds_sync();
    s_w[lane] = w;
    s_e[lane] = make_int2((int)(c & 0xffffu) * kRow, (int)(c >> 16) * kRow);
    wave_lds_sync();
}

// ------------------------------------------------------------------ forward
// One chunk (cnt <= 64 samples, descriptors at s_w/s_e[dbase ...]) of one row.
// (Requesting the taps of slot-iteration it+1 before the arithmetic of iteration it -- a hand-made
// software pipeline -- was measured: no gain for the forward, register spills for dq. The four waves
// per SIMD already overlap the LDS pipe and the VALU.)
// CNT > 0 fixes the sample count at compile time (branch-free, fully unrolled chunk).
template <typename S, int D, int DC, int CNT>
__device__ __forceinline__ void fwd_plane_chunk(uint32_t lbase, const float4 *s_w, const int2 *s_e,
                                                int dbase, int cnt_rt, int slot,
                                                const float (&qf)[DC], const uint32_t *qp, float qscale,
                                                float &m, float &lsum, float (&acc)[DC])
{
    constexpr bool kPacked = S::kBytes == 2;
    constexpr int G = D / DC, NS = kWave / G;
    constexpr int ITS = CNT > 0 ? (CNT + NS - 1) / NS : G;
    const int cnt = CNT > 0 ? CNT : cnt_rt;
    constexpr int kRow = D * S::kBytes;
    float sv[ITS];
    float mc = kNegBig;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        sv[it] = kNegBig;
        if (it * NS < cnt) {
            const int j = it * NS + slot;
            const float4 w = s_w[dbase + j];
            const int2 e = s_e[dbase + j];
            const uint32_t at = e.x + lbase, ab = e.y + lbase;     // lbase: LDS address of the image + this lane's byte
            const unsigned char *top = lds_at(at), *bot = lds_at(ab);                                          // K, left taps
            const unsigned char *topr = lds_at((at ^ kRow) + 2 * kRow), *botr = lds_at((ab ^ kRow) + 2 * kRow);   // K, right taps
            float dot = 0.f;
            if constexpr (kPacked) {
                uint32_t qq[DC / 2];
#pragma unroll
                for (int i = 0; i < DC / 2; ++i) qq[i] = qp[i];
                dot = qscale * tap_dot16<S, DC>(top, topr, bot, botr, w, qq);
            } else {
                float t0[DC], t1[DC], t2[DC], t3[DC];
                load_chunk<S, DC>(top, t0);
                load_chunk<S, DC>(topr, t1);
                load_chunk<S, DC>(bot, t2);
                load_chunk<S, DC>(botr, t3);
#pragma unroll
                for (int d = 0; d < DC; ++d) {
                    const float kk = fmaf(w.x, t0[d], fmaf(w.y, t1[d], fmaf(w.z, t2[d], w.w * t3[d])));
                    dot = fmaf(qf[d], kk, dot);
                }
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
            const int j = it * NS + slot;
            const float p = (j < cnt) ? __builtin_amdgcn_exp2f(sv[it] - m_new) : 0.f;
            lsum += p;
            const float4 w = s_w[dbase + j];
            const int2 e = s_e[dbase + j];
            const uint32_t at = e.x + lbase, ab = e.y + lbase;
            float t0[DC], t1[DC], t2[DC], t3[DC];
            load_chunk<S, DC>(lds_at(at ^ kRow), t0);                  // V, left taps
            load_chunk<S, DC>(lds_at(at + 2 * kRow), t1);              // V, right taps
            load_chunk<S, DC>(lds_at(ab ^ kRow), t2);
            load_chunk<S, DC>(lds_at(ab + 2 * kRow), t3);
            const float c0 = p * w.x, c1 = p * w.y, c2 = p * w.z, c3 = p * w.w;
#pragma unroll
            for (int d = 0; d < DC; ++d)
                acc[d] = fmaf(c0, t0[d], fmaf(c1, t1[d], fmaf(c2, t2[d], fmaf(c3, t3[d], acc[d]))));
        }
    }
}

// PAIR: two rows per descriptor pass (P <= 32); PCNT > 0: P is exactly PCNT, known at compile time.
template <typename S, int D, int DC, int QW, bool PAIR, int PCNT>
__global__ __launch_bounds__(kPlaneWaves *kWave) void fwd_plane_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float4 *__restrict__ desc_w, const uint32_t *__restrict__ desc_e, void *__restrict__ out_,
    float *__restrict__ lse_, Dims dm)
{
    constexpr int G = D / DC;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(kPlaneLdsAlign))) unsigned char smem[];
    const int img_bytes = plane_lds_bytes<S, D>(dm.L);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    float4 *s_w = reinterpret_cast<float4 *>(smem + img_bytes) + wave * kWave;
    int2 *s_e = reinterpret_cast<int2 *>(smem + img_bytes + kPlaneWaves * kWave * 16) + wave * kWave;

    const PlaneBlock pb = decode_plane_block(dm, kPlaneWaves * QW);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const uint32_t lbase = lds_offset(smem) + lane_byte;

    zero_plane_pads<S, D>(smem, dm.L);

    // fp32 storage: q widened and pre-scaled (qf); 16-bit storage: q as packed pairs (qp), scale on the logit
    constexpr bool kPacked = S::kBytes == 2;
    float qf[QW][DC], acc[QW][DC], m[QW], lsum[QW];
    uint32_t qp[QW][kPacked ? DC / 2 : 1];
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
        if constexpr (kPacked) {
            load_packed<S, DC>((const char *)q_ + (row[qi] * D + lane_elem) * S::kBytes, qp[qi]);
        } else {
            load_chunk<S, DC>((const char *)q_ + (row[qi] * D + lane_elem) * S::kBytes, qf[qi]);
#pragma unroll
            for (int d = 0; d < DC; ++d) qf[qi][d] *= qscale;
        }
        m[qi] = kNegBig;
        lsum[qi] = 0.f;
#pragma unroll
        for (int d = 0; d < DC; ++d) acc[qi][d] = 0.f;
    }

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = (((size_t)pb.b * dm.V + s2) * dm.H + pb.h) * (size_t)dm.L * D * S::kBytes;
        __syncthreads();                                       // the previous view's readers are done
        stage_plane<S, D>(smem, (const char *)k_ + plane, dm.L, 0);
        stage_plane<S, D>(smem, (const char *)v_ + plane, dm.L, 1);
        __syncthreads();
        if constexpr (PAIR) {
#pragma unroll
            for (int qr = 0; qr + 1 < QW; qr += 2) {
                if (!have[qr]) continue;                       // wave-uniform; rows are consecutive
                stage_pair_descriptors<S, D>(desc_w, desc_e, crow[qr] + (size_t)s2 * dm.P,
                                             crow[qr + 1] + (size_t)s2 * dm.P, dm.P, lane, s_w, s_e);
                fwd_plane_chunk<S, D, DC, PCNT>(lbase, s_w, s_e, 0, dm.P, slot, qf[qr], qp[qr], qscale,
                                                m[qr], lsum[qr], acc[qr]);
                if (have[qr + 1])
                    fwd_plane_chunk<S, D, DC, PCNT>(lbase, s_w, s_e, 32, dm.P, slot, qf[qr + 1], qp[qr + 1],
                                                    qscale, m[qr + 1], lsum[qr + 1], acc[qr + 1]);
            }
        } else {
#pragma unroll
            for (int qi = 0; qi < QW; ++qi) {
                if (!have[qi]) continue;
                const size_t cq = crow[qi] + (size_t)s2 * dm.P;
                for (int c0 = 0; c0 < dm.P; c0 += kWave) {
                    stage_row_descriptors<S, D>(desc_w, desc_e, cq, dm.P, c0, lane, s_w, s_e);
                    fwd_plane_chunk<S, D, DC, 0>(lbase, s_w, s_e, 0, min(kWave, dm.P - c0), slot, qf[qi],
                                                 qp[qi], qscale, m[qi], lsum[qi], acc[qi]);
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
template <typename S, int D, int DC, int CNT>
__device__ __forceinline__ void dq_plane_chunk(uint32_t lbase, const float4 *s_w, const int2 *s_e,
                                               int dbase, int cnt_rt, int slot, float qscale,
                                               const float (&qf)[DC], const float (&dof)[DC], const uint32_t *dop,
                                               float lse, float delta, float (&dqa)[DC])
{
    constexpr int G = D / DC, NS = kWave / G;
    constexpr int kRow = D * S::kBytes;
    constexpr bool kPacked = S::kBytes == 2;
    const int cnt = CNT > 0 ? CNT : cnt_rt;
    for (int j0 = 0; j0 < cnt; j0 += NS) {
        const int j = j0 + slot;
        const float4 w = s_w[dbase + j];
        const int2 e = s_e[dbase + j];
        const uint32_t at = e.x + lbase, ab = e.y + lbase;
        const unsigned char *top = lds_at(at), *bot = lds_at(ab);                      // K left taps; V right taps at +2*ROW
        const unsigned char *topx = lds_at(at ^ kRow), *botx = lds_at(ab ^ kRow);      // V left taps; K right taps at +2*ROW
        float kk[DC];
        float dot = 0.f, dp = 0.f;
        {
            float t0[DC], t1[DC], t2[DC], t3[DC];
            load_chunk<S, DC>(top, t0);
            load_chunk<S, DC>(topx + 2 * kRow, t1);
            load_chunk<S, DC>(bot, t2);
            load_chunk<S, DC>(botx + 2 * kRow, t3);
#pragma unroll
            for (int d = 0; d < DC; ++d) {
                kk[d] = fmaf(w.x, t0[d], fmaf(w.y, t1[d], fmaf(w.z, t2[d], w.w * t3[d])));
                dot = fmaf(qf[d], kk[d], dot);
            }
        }
        __builtin_amdgcn_sched_barrier(0);     // keep the V taps out of the K taps' live range (register budget)
        if constexpr (kPacked) {
            uint32_t dd[DC / 2];
#pragma unroll
            for (int i = 0; i < DC / 2; ++i) dd[i] = dop[i];
            dp = tap_dot16<S, DC>(topx, top + 2 * kRow, botx, bot + 2 * kRow, w, dd);
        } else {
            float u0[DC], u1[DC], u2[DC], u3[DC];
            load_chunk<S, DC>(topx, u0);
            load_chunk<S, DC>(top + 2 * kRow, u1);
            load_chunk<S, DC>(botx, u2);
            load_chunk<S, DC>(bot + 2 * kRow, u3);
#pragma unroll
            for (int d = 0; d < DC; ++d) {
                const float vv = fmaf(w.x, u0[d], fmaf(w.y, u1[d], fmaf(w.z, u2[d], w.w * u3[d])));
                dp = fmaf(dof[d], vv, dp);
            }
        }
        dot = group_sum<G>(dot);
        dp = group_sum<G>(dp);
        const float p = (j < cnt) ? __builtin_amdgcn_exp2f(dot * qscale - lse) : 0.f;
        const float ds = p * (dp - delta);
#pragma unroll
        for (int d = 0; d < DC; ++d) dqa[d] = fmaf(ds, kk[d], dqa[d]);
    }
}

template <typename S, int D, int DC, int QW, bool PAIR, int PCNT>
__global__ __launch_bounds__(kPlaneWaves *kWave) void bwd_dq_plane_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float4 *__restrict__ desc_w, const uint32_t *__restrict__ desc_e, const void *__restrict__ out_,
    const float *__restrict__ lse_, const void *__restrict__ dout_, void *__restrict__ dq_,
    float *__restrict__ delta_, Dims dm)
{
    constexpr int G = D / DC;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(kPlaneLdsAlign))) unsigned char smem[];
    const int img_bytes = plane_lds_bytes<S, D>(dm.L);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    float4 *s_w = reinterpret_cast<float4 *>(smem + img_bytes) + wave * kWave;
    int2 *s_e = reinterpret_cast<int2 *>(smem + img_bytes + kPlaneWaves * kWave * 16) + wave * kWave;

    const PlaneBlock pb = decode_plane_block(dm, kPlaneWaves * QW);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const uint32_t lbase = lds_offset(smem) + lane_byte;

    zero_plane_pads<S, D>(smem, dm.L);

    constexpr bool kPacked = S::kBytes == 2;
    float qf[QW][DC], dof[QW][DC], dqa[QW][DC], lse[QW], delta[QW];
    uint32_t dop[QW][kPacked ? DC / 2 : 1];      // 16-bit storage: dout as packed pairs for the dp dot products
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
        if constexpr (kPacked) load_packed<S, DC>((const char *)dout_ + roff, dop[qi]);
        load_chunk<S, DC>((const char *)out_ + roff, of);
        float dl = 0.f;
#pragma unroll
        for (int d = 0; d < DC; ++d) { dl = fmaf(dof[qi][d], of[d], dl); dqa[qi][d] = 0.f; }
        delta[qi] = group_sum<G>(dl);          // the reference's _bwd_preprocess, fused
        lse[qi] = lse_[row[qi]];
        if (have[qi] && lane == 0) delta_[row[qi]] = delta[qi];
    }

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = (((size_t)pb.b * dm.V + s2) * dm.H + pb.h) * (size_t)dm.L * D * S::kBytes;
        __syncthreads();
        stage_plane<S, D>(smem, (const char *)k_ + plane, dm.L, 0);
        stage_plane<S, D>(smem, (const char *)v_ + plane, dm.L, 1);
        __syncthreads();
        if constexpr (PAIR) {
#pragma unroll
            for (int qp = 0; qp + 1 < QW; qp += 2) {
                if (!have[qp]) continue;
                stage_pair_descriptors<S, D>(desc_w, desc_e, crow[qp] + (size_t)s2 * dm.P,
                                             crow[qp + 1] + (size_t)s2 * dm.P, dm.P, lane, s_w, s_e);
                dq_plane_chunk<S, D, DC, PCNT>(lbase, s_w, s_e, 0, dm.P, slot, qscale, qf[qp], dof[qp],
                                               dop[qp], lse[qp], delta[qp], dqa[qp]);
                if (have[qp + 1])
                    dq_plane_chunk<S, D, DC, PCNT>(lbase, s_w, s_e, 32, dm.P, slot, qscale, qf[qp + 1],
                                                   dof[qp + 1], dop[qp + 1], lse[qp + 1], delta[qp + 1], dqa[qp + 1]);
            }
        } else {
#pragma unroll
            for (int qi = 0; qi < QW; ++qi) {
                if (!have[qi]) continue;
                const size_t cq = crow[qi] + (size_t)s2 * dm.P;
                for (int c0 = 0; c0 < dm.P; c0 += kWave) {
                    stage_row_descriptors<S, D>(desc_w, desc_e, cq, dm.P, c0, lane, s_w, s_e);
                    dq_plane_chunk<S, D, DC, 0>(lbase, s_w, s_e, 0, min(kWave, dm.P - c0), slot, qscale,
                                                qf[qi], dof[qi], dop[qi], lse[qi], delta[qi], dqa[qi]);
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

// ====================================================================== one query row per slot
// The same staged planes and tap table, with the rows dealt differently: slot s of a wave (its G
// lanes) owns query row s of the wave's NS = 64/G rows for the whole kernel, and in every trip the NS
// slots consume one sample each -- of NS different rows. A lane then carries the state of ONE row (q,
// accumulator, running max and sum: ~10 registers instead of ~40 for four rows), there is nothing to
// merge across slots at the end, every trip is full whatever P is (the kernels above leave slots idle
// when P is not a multiple of NS), and a workgroup covers 16*NS rows, so each staged plane serves
// twice as many rows.
//
// Per key view and pass, lane (slot, g) fetches the table entry of sample c0+g of its own row: G samples
// per row and pass, parked sample-major (entry of trip t and slot s at t*NS + s, so the NS slots of a
// trip read one contiguous stretch). Odd slots swap the two samples of every pair of trips: with the
// table's alternating bank-half order, neighbouring slots then gather from opposite halves in every trip.
template <typename S, int D>
__device__ __forceinline__ void stage_slot_descriptors(const float4 *__restrict__ desc_w,
                                                       const uint32_t *__restrict__ desc_e, size_t d_row, int P,
                                                       int c0, int g, int slot, int G_, int NS_, float4 *s_w,
                                                       int2 *s_e)
{
    constexpr int kRow = D * S::kBytes;
    const int n = c0 + g;
    const bool valid = n < P;
    const size_t i = d_row + (valid ? n : 0);
    float4 w = desc_w[i];
    const uint32_t c = desc_e[i];
    if (!valid) w = make_float4(0.f, 0.f, 0.f, 0.f);
    const int cnt = min(G_, P - c0);                       // samples of this pass (same for every row)
    const int trip = (cnt & 1) == 0 ? g ^ (slot & 1) : g;    // pair swap only when no pair straddles the end
    wave_lds_sync();
    s_w[trip * NS_ + slot] = w;
    s_e[trip * NS_ + slot] = make_int2((int)(c & 0xffffu) * kRow, (int)(c >> 16) * kRow);
    wave_lds_sync();
}

template <typename S, int D, int DC>
__global__ __launch_bounds__(kPlaneWaves *kWave) void fwd_slot_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float4 *__restrict__ desc_w, const uint32_t *__restrict__ desc_e, void *__restrict__ out_,
    float *__restrict__ lse_, Dims dm)
{
    constexpr int G = D / DC, NS = kWave / G;
    constexpr int kRow = D * S::kBytes;
    constexpr bool kPacked = S::kBytes == 2;
    static_assert(G >= 2 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(kPlaneLdsAlign))) unsigned char smem[];
    const int img_bytes = plane_lds_bytes<S, D>(dm.L);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    float4 *s_w = reinterpret_cast<float4 *>(smem + img_bytes) + wave * kWave;
    int2 *s_e = reinterpret_cast<int2 *>(smem + img_bytes + kPlaneWaves * kWave * 16) + wave * kWave;

    const PlaneBlock pb = decode_plane_block(dm, kPlaneWaves * NS);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const uint32_t lbase = lds_offset(smem) + lane_byte;

    zero_plane_pads<S, D>(smem, dm.L);

    const int qidx = pb.qbase + wave * NS + slot;
    const bool have = qidx < nq;
    const unsigned qc = (unsigned)(have ? qidx : nq - 1);
    const unsigned s1 = dm.divL.div(qc), l = qc - s1 * (unsigned)dm.L;
    const size_t row = (((size_t)pb.b * dm.V + s1) * dm.H + pb.h) * dm.L + l;
    const size_t crow = (((size_t)pb.b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
    float qf[DC], acc[DC];
    uint32_t qp[kPacked ? DC / 2 : 1];
    if constexpr (kPacked) {
        load_packed<S, DC>((const char *)q_ + (row * D + lane_elem) * S::kBytes, qp);
    } else {
        load_chunk<S, DC>((const char *)q_ + (row * D + lane_elem) * S::kBytes, qf);
#pragma unroll
        for (int d = 0; d < DC; ++d) qf[d] *= qscale;
    }
    float m = kNegBig, lsum = 0.f;
#pragma unroll
    for (int d = 0; d < DC; ++d) acc[d] = 0.f;

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = (((size_t)pb.b * dm.V + s2) * dm.H + pb.h) * (size_t)dm.L * D * S::kBytes;
        __syncthreads();                                       // the previous view's readers are done
        stage_plane<S, D>(smem, (const char *)k_ + plane, dm.L, 0);
        stage_plane<S, D>(smem, (const char *)v_ + plane, dm.L, 1);
        __syncthreads();
        for (int c0 = 0; c0 < dm.P; c0 += G) {
            stage_slot_descriptors<S, D>(desc_w, desc_e, crow + (size_t)s2 * dm.P, dm.P, c0, g, slot, G, NS, s_w,
                                         s_e);
            const int cnt = min(G, dm.P - c0);
            float sv[G];
            float mc = kNegBig;
#pragma unroll
            for (int t = 0; t < G; ++t) {
                sv[t] = kNegBig;
                if (t < cnt) {
                    const float4 w = s_w[t * NS + slot];
                    const int2 e = s_e[t * NS + slot];
                    const uint32_t at = e.x + lbase, ab = e.y + lbase;
                    const unsigned char *top = lds_at(at), *bot = lds_at(ab);
                    const unsigned char *topr = lds_at((at ^ kRow) + 2 * kRow), *botr = lds_at((ab ^ kRow) + 2 * kRow);
                    float dot = 0.f;
                    if constexpr (kPacked) {
                        dot = qscale * tap_dot16<S, DC>(top, topr, bot, botr, w, qp);
                    } else {
                        float t0[DC], t1[DC], t2[DC], t3[DC];
                        load_chunk<S, DC>(top, t0);
                        load_chunk<S, DC>(topr, t1);
                        load_chunk<S, DC>(bot, t2);
                        load_chunk<S, DC>(botr, t3);
#pragma unroll
                        for (int d = 0; d < DC; ++d) {
                            const float kk = fmaf(w.x, t0[d], fmaf(w.y, t1[d], fmaf(w.z, t2[d], w.w * t3[d])));
                            dot = fmaf(qf[d], kk, dot);
                        }
                    }
                    sv[t] = group_sum<G>(dot);
                    mc = fmaxf(mc, sv[t]);
                }
            }
            const float m_new = fmaxf(m, mc);
            const float alpha = __builtin_amdgcn_exp2f(m - m_new);
            m = m_new;
            lsum *= alpha;
#pragma unroll
            for (int d = 0; d < DC; ++d) acc[d] *= alpha;
#pragma unroll
            for (int t = 0; t < G; ++t) {
                if (t < cnt) {
                    const float p = __builtin_amdgcn_exp2f(sv[t] - m_new);
                    lsum += p;
                    const float4 w = s_w[t * NS + slot];
                    const int2 e = s_e[t * NS + slot];
                    const uint32_t at = e.x + lbase, ab = e.y + lbase;
                    float t0[DC], t1[DC], t2[DC], t3[DC];
                    load_chunk<S, DC>(lds_at(at ^ kRow), t0);                  // V, left taps
                    load_chunk<S, DC>(lds_at(at + 2 * kRow), t1);              // V, right taps
                    load_chunk<S, DC>(lds_at(ab ^ kRow), t2);
                    load_chunk<S, DC>(lds_at(ab + 2 * kRow), t3);
                    const float c0w = p * w.x, c1w = p * w.y, c2w = p * w.z, c3w = p * w.w;
#pragma unroll
                    for (int d = 0; d < DC; ++d)
                        acc[d] = fmaf(c0w, t0[d], fmaf(c1w, t1[d], fmaf(c2w, t2[d], fmaf(c3w, t3[d], acc[d]))));
                }
            }
        }
    }

    if (have) {
        const float inv = 1.0f / lsum;
#pragma unroll
        for (int d = 0; d < DC; ++d) acc[d] *= inv;
        store_chunk<S, DC>((char *)out_ + (row * D + lane_elem) * S::kBytes, acc);
        if (g == 0) lse_[row] = m + __log2f(lsum);
    }
}

template <typename S, int D, int DC>
__global__ __launch_bounds__(kPlaneWaves *kWave) void bwd_dq_slot_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float4 *__restrict__ desc_w, const uint32_t *__restrict__ desc_e, const void *__restrict__ out_,
    const float *__restrict__ lse_, const void *__restrict__ dout_, void *__restrict__ dq_,
    float *__restrict__ delta_, Dims dm)
{
    constexpr int G = D / DC, NS = kWave / G;
    constexpr int kRow = D * S::kBytes;
    constexpr bool kPacked = S::kBytes == 2;
    static_assert(G >= 2 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(kPlaneLdsAlign))) unsigned char smem[];
    const int img_bytes = plane_lds_bytes<S, D>(dm.L);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    float4 *s_w = reinterpret_cast<float4 *>(smem + img_bytes) + wave * kWave;
    int2 *s_e = reinterpret_cast<int2 *>(smem + img_bytes + kPlaneWaves * kWave * 16) + wave * kWave;

    const PlaneBlock pb = decode_plane_block(dm, kPlaneWaves * NS);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const uint32_t lbase = lds_offset(smem) + lane_byte;

    zero_plane_pads<S, D>(smem, dm.L);

    const int qidx = pb.qbase + wave * NS + slot;
    const bool have = qidx < nq;
    const unsigned qc = (unsigned)(have ? qidx : nq - 1);
    const unsigned s1 = dm.divL.div(qc), l = qc - s1 * (unsigned)dm.L;
    const size_t row = (((size_t)pb.b * dm.V + s1) * dm.H + pb.h) * dm.L + l;
    const size_t crow = (((size_t)pb.b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
    const size_t roff = (row * D + lane_elem) * S::kBytes;
    float qf[DC], dof[DC], dqa[DC];
    uint32_t dop[kPacked ? DC / 2 : 1];
    float delta;
    {
        float of[DC];
        load_chunk<S, DC>((const char *)q_ + roff, qf);
        load_chunk<S, DC>((const char *)dout_ + roff, dof);
        if constexpr (kPacked) load_packed<S, DC>((const char *)dout_ + roff, dop);
        load_chunk<S, DC>((const char *)out_ + roff, of);
        float dl = 0.f;
#pragma unroll
        for (int d = 0; d < DC; ++d) { dl = fmaf(dof[d], of[d], dl); dqa[d] = 0.f; }
        delta = group_sum<G>(dl);              // the reference's _bwd_preprocess, fused
    }
    const float lse = lse_[row];
    if (have && g == 0) delta_[row] = delta;

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = (((size_t)pb.b * dm.V + s2) * dm.H + pb.h) * (size_t)dm.L * D * S::kBytes;
        __syncthreads();
        stage_plane<S, D>(smem, (const char *)k_ + plane, dm.L, 0);
        stage_plane<S, D>(smem, (const char *)v_ + plane, dm.L, 1);
        __syncthreads();
        for (int c0 = 0; c0 < dm.P; c0 += G) {
            stage_slot_descriptors<S, D>(desc_w, desc_e, crow + (size_t)s2 * dm.P, dm.P, c0, g, slot, G, NS, s_w,
                                         s_e);
            const int cnt = min(G, dm.P - c0);
            for (int t = 0; t < cnt; ++t) {
                const float4 w = s_w[t * NS + slot];
                const int2 e = s_e[t * NS + slot];
                const uint32_t at = e.x + lbase, ab = e.y + lbase;
                const unsigned char *top = lds_at(at), *bot = lds_at(ab);                      // K left; V right at +2*ROW
                const unsigned char *topx = lds_at(at ^ kRow), *botx = lds_at(ab ^ kRow);      // V left; K right at +2*ROW
                float kk[DC];
                float dot = 0.f, dp = 0.f;
                {
                    float t0[DC], t1[DC], t2[DC], t3[DC];
                    load_chunk<S, DC>(top, t0);
                    load_chunk<S, DC>(topx + 2 * kRow, t1);
                    load_chunk<S, DC>(bot, t2);
                    load_chunk<S, DC>(botx + 2 * kRow, t3);
#pragma unroll
                    for (int d = 0; d < DC; ++d) {
                        kk[d] = fmaf(w.x, t0[d], fmaf(w.y, t1[d], fmaf(w.z, t2[d], w.w * t3[d])));
                        dot = fmaf(qf[d], kk[d], dot);
                    }
                }
                if constexpr (kPacked) {
                    dp = tap_dot16<S, DC>(topx, top + 2 * kRow, botx, bot + 2 * kRow, w, dop);
                } else {
                    float u0[DC], u1[DC], u2[DC], u3[DC];
                    load_chunk<S, DC>(topx, u0);
                    load_chunk<S, DC>(top + 2 * kRow, u1);
                    load_chunk<S, DC>(botx, u2);
                    load_chunk<S, DC>(bot + 2 * kRow, u3);
#pragma unroll
                    for (int d = 0; d < DC; ++d) {
                        const float vv = fmaf(w.x, u0[d], fmaf(w.y, u1[d], fmaf(w.z, u2[d], w.w * u3[d])));
                        dp = fmaf(dof[d], vv, dp);
                    }
                }
                dot = group_sum<G>(dot);
                dp = group_sum<G>(dp);
                const float p = __builtin_amdgcn_exp2f(dot * qscale - lse);
                const float ds = p * (dp - delta);
#pragma unroll
                for (int d = 0; d < DC; ++d) dqa[d] = fmaf(ds, kk[d], dqa[d]);
            }
        }
    }

    if (have) {
#pragma unroll
        for (int d = 0; d < DC; ++d) dqa[d] *= dm.sm_scale;
        store_chunk<S, DC>((char *)dq_ + roff, dqa);
    }
}

}  // namespace dsdpa
