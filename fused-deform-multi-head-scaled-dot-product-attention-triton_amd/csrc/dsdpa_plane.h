// "Plane" kernels: query-stationary forward and dq with the current key view's
// K and V planes staged in LDS, for shapes where one (b, s2, h) plane pair
// fits next to the per-wave tap descriptors.
//
// A workgroup of 16 waves owns 16*NS consecutive query rows of one (b, h) (NS = 64/G
// rows per wave, one per slot of G lanes; rows are counted over (s1, l), so a
// workgroup may straddle two query views) and walks the V key views: stage K_s2 and
// V_s2 (coalesced 16-byte loads, kept in the storage type), barrier, every wave runs
// its rows against the staged planes, barrier, next view. The online-softmax state
// (forward) or the dq accumulator (backward) of a row stays in the registers of its
// slot across the views.
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

constexpr int kPlaneWaves = 16;          // at most; see plane_waves for the number a launch uses

// LDS addresses as plain 32-bit numbers: the tap addresses are sums and XORs of byte offsets, and a
// pointer made from the finished number costs no instruction (adding offsets to a generic pointer to
// the dynamic LDS block costs an add per pointer). The XOR needs the block aligned to 2*ROW.
using lds_bytes = __attribute__((address_space(3))) const unsigned char *;
__device__ __forceinline__ uint32_t lds_offset(const void *p) { return (uint32_t)(size_t)(lds_bytes)p; }
__device__ __forceinline__ const unsigned char *lds_at(uint32_t off) { return (const unsigned char *)(lds_bytes)(size_t)off; }
constexpr int kPlaneLdsAlign = 2048;   // 2*ROW for the widest row (D = 256, fp32)
// per wave: NS rows x (G + 1) descriptor places (one pad place per row, see stage_slot_descriptors);
// NS*(G+1) = 64 + NS <= 96 for every lane split
constexpr int kPlaneDescPlaces = 96;
constexpr int kPlaneDescBytes = kPlaneWaves * kPlaneDescPlaces * (16 + 8);   // float4 weights + int2 base offsets
constexpr int kPlaneGradBytes = kPlaneWaves * kPlaneDescPlaces * 8;         // fx, fy per place (coordinate-gradient kernel)

template <typename S, int D>
__host__ __device__ constexpr int plane_lds_bytes(int L) { return (L + 2) * 2 * D * S::kBytes; }

// The K and V planes of one view (L rows of D elements, `px_bytes` apart in memory) -> LDS rows 1..L of the
// interleaved image: row q = pixel q - 1 holds the pixel's K row and V row side by side, K in the half q & 1.
// The rows go from memory to LDS without passing through registers (global_load_lds_dwordx4: lane i of a wave
// writes 16 bytes at the wave's LDS base + 16 i): a wave fills 1 KB of the image per instruction, every lane
// fetching the 16 bytes of K or of V that belong at its place, and all of a wave's instructions are in flight
// together -- a loop of load, wait, LDS write pays one round trip to memory per 16 bytes of a thread, six per
// view at 18x18, D = 32. Ends with this wave's wait; the caller's barrier follows.
template <typename S, int D>
__device__ __forceinline__ void stage_plane_pair(unsigned char *lds, const char *ksrc, const char *vsrc, int L,
                                                 unsigned px_bytes)
{
    constexpr unsigned kRow = D * S::kBytes;
    static_assert((kRow & (kRow - 1)) == 0 && kRow >= 16, "row bytes: a power of two");
    const unsigned total = (unsigned)L * 2u * kRow;                    // bytes of rows 1..L
    const unsigned wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63u;
    const unsigned step = (unsigned)__builtin_amdgcn_readfirstlane((int)(blockDim.x >> 6)) * 1024u;
    const unsigned lds1 = lds_offset(lds) + 2u * kRow;                 // row 1
    for (unsigned o0 = wave * 1024u; o0 < total; o0 += step) {
        const unsigned o = o0 + 16u * lane;
        if (o < total) {                                               // (the last instruction of an image may be part full)
            const unsigned p = o / (2u * kRow), within = o % (2u * kRow);
            const unsigned half = within / kRow, col = within % kRow;
            const bool from_v = ((half ^ (p + 1u)) & 1u) != 0u;
            const char *src = (from_v ? vsrc : ksrc) + (size_t)p * px_bytes + col;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                             (__attribute__((address_space(3))) void *)(uintptr_t)(lds1 + o0), 16, 0, 0);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <typename S, int D>
__device__ __forceinline__ void zero_plane_pads(unsigned char *lds, int L)
{
    constexpr int kRow = D * S::kBytes;
    constexpr int kChunks = 2 * kRow / 16;
    for (int i = threadIdx.x; i < 2 * kChunks; i += (int)blockDim.x) {
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

// Waves per workgroup and query-row blocks per workgroup of a staged launch. The planes in LDS allow one workgroup
// per CU, so a launch runs in rounds of `cus` workgroups, and a round lasts about as long as its workgroups have
// waves times samples per view (the kernels are bound by instruction issue) plus the staging of the planes (about
// two waves' worth at 32 samples per view: 64 in these units). 16 waves is the most rows per staged plane and
// block; fewer waves can mean fewer idle CUs in the last round (2 x 8 x 16 planes of 14x14 pixels and 8 views
// make 416 workgroups of 16 waves, 1.6 rounds of 256, but 512 of 13 waves, two full rounds of shorter
// workgroups), and two row blocks per workgroup halve the staging of a launch of many rounds (few samples per
// view: the reference's sweep). Picks the pair with the lowest rounds * (blocks * waves * P + 64).
inline void plane_config(long long planes, int rows_per_plane, int rows_per_wave, int P, int cus, int max_blocks,
                         int *waves, int *row_blocks)
{
    long long best_cost = -1;
    *waves = kPlaneWaves;
    *row_blocks = 1;
    for (int rb = 1; rb <= max_blocks; ++rb) {
        for (int w = kPlaneWaves; w >= 4; --w) {
            const long long rows = (long long)rb * w * rows_per_wave;
            const long long blocks = planes * ((rows_per_plane + rows - 1) / rows);
            const long long cost = ((blocks + cus - 1) / cus) * ((long long)rb * w * P + 64);
            if (best_cost < 0 || cost < best_cost) { best_cost = cost; *waves = w; *row_blocks = rb; }
        }
    }
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
// packed into one 32-bit word (13 bits each: a plane that fits in LDS has fewer than 2200 slots). Within
// every run of up to 64 samples of one (b, s1, l, s2) the entries are stored in paired_position order.
// For the coordinate gradient (desc_g not null) the word also carries which taps lie inside the image
// -- bits 13, 14: columns x0, x0+1; bits 29, 30: rows y0, y0+1 -- and desc_g holds (fx, fy, the sample's
// index n inside its run as an integer, unused): the entries are stored in a permuted order, and the
// gradient has to go back to the sample it belongs to.
constexpr int kDescThreads = 256;
constexpr uint32_t kDescCodeMask = 0x1fffu;

static __global__ __launch_bounds__(kDescThreads) void plane_descriptor_kernel(
    const float *__restrict__ coords_, Dims dm, float4 *__restrict__ desc_w, uint32_t *__restrict__ desc_e,
    float4 *__restrict__ desc_g, ZeroJob zero)
{
    zero_buffers(zero);        // the backward's accumulators and counters ride along (empty in the forward)
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
        uint32_t word = (uint32_t)(2 * qt + (qt & 1)) | ((uint32_t)(2 * qb + (qb & 1)) << 16);
        if (desc_g) {
            // same arithmetic as make_taps, so that fx, fy and the inside tests agree with the weights
            const float x = ((xy.x * 2.0f - 1.0f) + 1.0f) * ((float)(dm.Wimg - 1) * 0.5f);
            const float y = ((xy.y * 2.0f - 1.0f) + 1.0f) * ((float)(dm.Himg - 1) * 0.5f);
            const float fx = x - floorf(x), fy = y - floorf(y);
            const bool fin = (x == x) && (y == y);
            const int x0 = tp.x0, y0 = tp.y0;
            const bool vx0 = fin && x0 >= 0 && x0 < dm.Wimg, vx1 = fin && x0 + 1 >= 0 && x0 + 1 < dm.Wimg;
            const bool vy0 = fin && y0 >= 0 && y0 < dm.Himg, vy1 = fin && y0 + 1 >= 0 && y0 + 1 < dm.Himg;
            word |= (vx0 ? 1u << 13 : 0u) | (vx1 ? 1u << 14 : 0u) | (vy0 ? 1u << 29 : 0u) | (vy1 ? 1u << 30 : 0u);
            desc_g[dst] = make_float4(fin ? fx : 0.f, fin ? fy : 0.f, __int_as_float(n), 0.f);
        }
        desc_e[dst] = word;
    }
}

// ------------------------------------------------------------------ one query row per slot
// Slot s of a wave (its G lanes) owns query row s of the wave's NS = 64/G rows for the whole kernel, and in
// every trip the NS slots consume one sample each -- of NS different rows. A lane carries the state of
// ONE row (q, accumulator, running max and sum: about 10 registers), nothing is merged across slots at
// the end, and every trip is full whatever P is. (An earlier layout gave a wave 16/DC rows and spread
// the samples of one row over the slots: four rows of state per lane, idle slots when P is not a
// multiple of NS, half as many rows per staged plane; 8 % slower forward at P = 32, more at small P.)
//
// Per key view and pass, lane (slot, g) fetches the table entry of sample c0+g of its own row: G samples
// per row and pass, parked at place slot*(G+1) + trip. The pad place per row keeps both sides free of
// bank conflicts: the lanes of a slot write G consecutive places, and the NS slots of a trip read places
// (G+1)*16 bytes apart, which fall in different 16-byte bank groups. Odd slots swap the two samples of
// every pair of trips: with the table's alternating bank-half order, neighbouring slots then gather from
// opposite halves of the bank line in every trip.
// s_g (coordinate gradient only): fx, fy of the sample; the four inside bits then ride in the low bits
// of the parked top address (ROW >= 32 bytes leaves them free): bit 0, 1: columns x0, x0+1; bit 2, 3: rows.
// Returns the index inside its run of the sample this lane fetched (coordinate gradient only, else 0).
template <typename S, int D>
__device__ __forceinline__ int stage_slot_descriptors(const float4 *__restrict__ desc_w,
                                                      const uint32_t *__restrict__ desc_e, size_t d_row, int P,
                                                      int c0, int g, int slot, int G_, float4 *s_w,
                                                      int2 *s_e, const float4 *__restrict__ desc_g = nullptr,
                                                      float2 *s_g = nullptr)
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
    int ex = (int)(c & kDescCodeMask) * kRow;
    const int ey = (int)((c >> 16) & kDescCodeMask) * kRow;
    float4 gw = make_float4(0.f, 0.f, 0.f, 0.f);
    if (desc_g) {
        gw = desc_g[i];
        ex |= (int)(((c >> 13) & 3u) | (((c >> 29) & 3u) << 2));
    }
    wave_lds_sync();
    s_w[slot * (G_ + 1) + trip] = w;
    s_e[slot * (G_ + 1) + trip] = make_int2(ex, ey);
    if (desc_g) s_g[slot * (G_ + 1) + trip] = make_float2(gw.x, gw.y);
    wave_lds_sync();
    return __float_as_int(gw.z);
}

// ROWS: query-row blocks per workgroup. With two, a workgroup of W waves covers 2*W*NS rows: every staged plane is
// worked on for the first W*NS rows and then for the second, so a launch of several rounds of workgroups stages
// half as often (at 12 views x 12 samples per view the staging is a third of a workgroup's time).
template <typename S, int D, int DC, int ROWS>
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
    float4 *s_w = reinterpret_cast<float4 *>(smem + img_bytes) + wave * kPlaneDescPlaces;
    int2 *s_e =
        reinterpret_cast<int2 *>(smem + img_bytes + kPlaneWaves * kPlaneDescPlaces * 16) + wave * kPlaneDescPlaces;

    const int rows_block = (int)(blockDim.x >> 6) * NS;                       // (workgroups of up to kPlaneWaves waves)
    const PlaneBlock pb = decode_plane_block(dm, ROWS * rows_block);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const uint32_t lbase = lds_offset(smem) + lane_byte;

    zero_plane_pads<S, D>(smem, dm.L);

    // per row block: this slot's row and its state
    bool have_s[ROWS];
    size_t row_s[ROWS], crow_s[ROWS];
    float qf_s[ROWS][DC], acc_s[ROWS][DC], m_s[ROWS], lsum_s[ROWS];
    uint32_t qp_s[ROWS][kPacked ? DC / 2 : 1];
#pragma unroll
    for (int rb = 0; rb < ROWS; ++rb) {
        const int qidx = pb.qbase + rb * rows_block + wave * NS + slot;
        have_s[rb] = qidx < nq;
        const unsigned qc = (unsigned)(have_s[rb] ? qidx : nq - 1);
        const unsigned s1 = dm.divL.div(qc), l = qc - s1 * (unsigned)dm.L;
        row_s[rb] = (((size_t)pb.b * dm.V + s1) * dm.H + pb.h) * dm.L + l;
        crow_s[rb] = (((size_t)pb.b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
        if constexpr (kPacked) {
            load_packed<S, DC>((const char *)q_ + (dm.q_row(pb.b, (int)s1, pb.h, (int)l) + lane_elem) * S::kBytes, qp_s[rb]);
        } else {
            load_chunk<S, DC>((const char *)q_ + (dm.q_row(pb.b, (int)s1, pb.h, (int)l) + lane_elem) * S::kBytes, qf_s[rb]);
#pragma unroll
            for (int d = 0; d < DC; ++d) qf_s[rb][d] *= qscale;
        }
        m_s[rb] = kNegBig;
        lsum_s[rb] = 0.f;
#pragma unroll
        for (int d = 0; d < DC; ++d) acc_s[rb][d] = 0.f;
    }

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = dm.kv_plane(pb.b, s2, pb.h) * S::kBytes;
        const unsigned px_bytes = (unsigned)dm.kv_sl * S::kBytes;
        __syncthreads();                                       // the previous view's readers are done
        stage_plane_pair<S, D>(smem, (const char *)k_ + plane, (const char *)v_ + plane, dm.L, px_bytes);
        __syncthreads();
#pragma unroll
        for (int rb = 0; rb < ROWS; ++rb) {
        const size_t crow = crow_s[rb];
        const float (&qf)[DC] = qf_s[rb];
        const uint32_t (&qp)[kPacked ? DC / 2 : 1] = qp_s[rb];
        float (&acc)[DC] = acc_s[rb];
        float &m = m_s[rb], &lsum = lsum_s[rb];
        for (int c0 = 0; c0 < dm.P; c0 += G) {
            stage_slot_descriptors<S, D>(desc_w, desc_e, crow + (size_t)s2 * dm.P, dm.P, c0, g, slot, G, s_w,
                                         s_e);
            const int cnt = min(G, dm.P - c0);
            // up to 8 trips per pass the descriptors stay in registers from the K pass to the V pass (a lane
            // holds one row: there is room); with 16 they are read again
            constexpr bool kKeep = G <= 8;
            float sv[G];
            float4 wt[kKeep ? G : 1];
            uint32_t att[kKeep ? G : 1], abt[kKeep ? G : 1];
            float mc = kNegBig;
#pragma unroll
            for (int t = 0; t < G; ++t) {
                sv[t] = kNegBig;
                if (t < cnt) {
                    const float4 w = s_w[slot * (G + 1) + t];
                    const int2 e = s_e[slot * (G + 1) + t];
                    const uint32_t at = e.x + lbase, ab = e.y + lbase;
                    if constexpr (kKeep) { wt[t] = w; att[t] = at; abt[t] = ab; }
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
                    float4 w;
                    uint32_t at, ab;
                    if constexpr (kKeep) {
                        w = wt[t]; at = att[t]; ab = abt[t];
                    } else {
                        w = s_w[slot * (G + 1) + t];
                        const int2 e = s_e[slot * (G + 1) + t];
                        at = e.x + lbase; ab = e.y + lbase;
                    }
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
    }

#pragma unroll
    for (int rb = 0; rb < ROWS; ++rb) {
        if (have_s[rb]) {
            const float inv = 1.0f / lsum_s[rb];
#pragma unroll
            for (int d = 0; d < DC; ++d) acc_s[rb][d] *= inv;
            store_chunk<S, DC>((char *)out_ + (row_s[rb] * D + lane_elem) * S::kBytes, acc_s[rb]);
            if (g == 0) lse_[row_s[rb]] = m_s[rb] + __log2f(lsum_s[rb]);
        }
    }
}

// CG: also the gradient of the coordinates (see bwd_dq_gather_kernel for the formula): per-tap dot
// products instead of blend-then-dot, the four per-tap terms masked by the inside bits, combined with
// fx, fy from the table and reduced over the slot. The lane that fetched a sample's table entry keeps
// the sample's result, and after the pass every lane adds its own sample's pair to dcoords (zeroed before
// the launch) with float atomics -- one wave-wide pair of atomics per pass, not one per trip.
// ROWS: query-row blocks per workgroup, as in the forward.
template <typename S, int D, int DC, bool CG, int ROWS>
__global__ __launch_bounds__(kPlaneWaves *kWave) void bwd_dq_slot_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float4 *__restrict__ desc_w, const uint32_t *__restrict__ desc_e, const void *__restrict__ out_,
    const float *__restrict__ lse_, const void *__restrict__ dout_, void *__restrict__ dq_,
    float2 *__restrict__ stats_, const float4 *__restrict__ desc_g, float *__restrict__ dcoords_, Dims dm)
{
    constexpr int G = D / DC, NS = kWave / G;
    constexpr int kRow = D * S::kBytes;
    constexpr bool kPacked = S::kBytes == 2 && !CG;
    static_assert(G >= 2 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(kPlaneLdsAlign))) unsigned char smem[];
    const int img_bytes = plane_lds_bytes<S, D>(dm.L);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    float4 *s_w = reinterpret_cast<float4 *>(smem + img_bytes) + wave * kPlaneDescPlaces;
    int2 *s_e =
        reinterpret_cast<int2 *>(smem + img_bytes + kPlaneWaves * kPlaneDescPlaces * 16) + wave * kPlaneDescPlaces;
    float2 *s_g = reinterpret_cast<float2 *>(smem + img_bytes + kPlaneDescBytes) + wave * kPlaneDescPlaces;   // CG only

    const int rows_block = (int)(blockDim.x >> 6) * NS;                       // (workgroups of up to kPlaneWaves waves)
    const PlaneBlock pb = decode_plane_block(dm, ROWS * rows_block);
    const int nq = dm.V * dm.L;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC, lane_byte = lane_elem * S::kBytes;
    const float qscale = dm.sm_scale * kLog2e;
    const uint32_t lbase = lds_offset(smem) + lane_byte;

    zero_plane_pads<S, D>(smem, dm.L);

    // per row block: this slot's row and its state
    bool have_s[ROWS];
    size_t crow_s[ROWS], roff_s[ROWS];
    float qf_s[ROWS][DC], dof_s[ROWS][DC], dqa_s[ROWS][DC], delta_s[ROWS], lse_s[ROWS];
    uint32_t dop_s[ROWS][kPacked ? DC / 2 : 1];
#pragma unroll
    for (int rb = 0; rb < ROWS; ++rb) {
        const int qidx = pb.qbase + rb * rows_block + wave * NS + slot;
        have_s[rb] = qidx < nq;
        const unsigned qc = (unsigned)(have_s[rb] ? qidx : nq - 1);
        const unsigned s1 = dm.divL.div(qc), l = qc - s1 * (unsigned)dm.L;
        const size_t row = (((size_t)pb.b * dm.V + s1) * dm.H + pb.h) * dm.L + l;
        crow_s[rb] = (((size_t)pb.b * dm.V + s1) * dm.L + l) * (size_t)dm.N;
        const size_t roff = (row * D + lane_elem) * S::kBytes;
        roff_s[rb] = roff;
        float of[DC];
        load_chunk<S, DC>((const char *)q_ + (dm.q_row(pb.b, (int)s1, pb.h, (int)l) + lane_elem) * S::kBytes, qf_s[rb]);
        load_chunk<S, DC>((const char *)dout_ + roff, dof_s[rb]);
        if constexpr (kPacked) load_packed<S, DC>((const char *)dout_ + roff, dop_s[rb]);
        load_chunk<S, DC>((const char *)out_ + roff, of);
        float dl = 0.f;
#pragma unroll
        for (int d = 0; d < DC; ++d) { dl = fmaf(dof_s[rb][d], of[d], dl); dqa_s[rb][d] = 0.f; }
        delta_s[rb] = group_sum<G>(dl);              // the reference's _bwd_preprocess, fused
        lse_s[rb] = lse_[row];
        if (stats_ && have_s[rb] && g == 0) stats_[row] = make_float2(lse_s[rb], delta_s[rb]);     // null: a launch of its own does it
    }

    for (int s2 = 0; s2 < dm.V; ++s2) {
        const size_t plane = dm.kv_plane(pb.b, s2, pb.h) * S::kBytes;
        const unsigned px_bytes = (unsigned)dm.kv_sl * S::kBytes;
        __syncthreads();
        stage_plane_pair<S, D>(smem, (const char *)k_ + plane, (const char *)v_ + plane, dm.L, px_bytes);
        __syncthreads();
#pragma unroll
        for (int rb = 0; rb < ROWS; ++rb) {
        const bool have = have_s[rb];
        const size_t crow = crow_s[rb];
        const float (&qf)[DC] = qf_s[rb];
        const float (&dof)[DC] = dof_s[rb];
        const uint32_t (&dop)[kPacked ? DC / 2 : 1] = dop_s[rb];
        float (&dqa)[DC] = dqa_s[rb];
        const float delta = delta_s[rb], lse = lse_s[rb];
        for (int c0 = 0; c0 < dm.P; c0 += G) {
            const int my_n = stage_slot_descriptors<S, D>(desc_w, desc_e, crow + (size_t)s2 * dm.P, dm.P, c0, g,
                                                          slot, G, s_w, s_e, CG ? desc_g : nullptr, s_g);
            const int cnt = min(G, dm.P - c0);
            const int my_trip = (cnt & 1) == 0 ? g ^ (slot & 1) : g;     // where this lane's sample was parked
            float my_gx = 0.f, my_gy = 0.f;
            for (int t = 0; t < cnt; ++t) {
                const float4 w = s_w[slot * (G + 1) + t];
                const int2 e = s_e[slot * (G + 1) + t];
                if constexpr (CG) {
                    const uint32_t inside = (uint32_t)e.x & 15u;
                    const uint32_t at = (uint32_t)e.x - inside + lbase, ab = e.y + lbase;
                    const unsigned char *kp[4] = { lds_at(at), lds_at((at ^ kRow) + 2 * kRow), lds_at(ab),
                                                   lds_at((ab ^ kRow) + 2 * kRow) };
                    const unsigned char *vp[4] = { lds_at(at ^ kRow), lds_at(at + 2 * kRow), lds_at(ab ^ kRow),
                                                   lds_at(ab + 2 * kRow) };
                    const float wt[4] = { w.x, w.y, w.z, w.w };
                    float kk[DC], dk_t[4], dv_t[4];
                    float dot = 0.f, dp = 0.f;
#pragma unroll
                    for (int d = 0; d < DC; ++d) kk[d] = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float tk[DC], tv[DC];
                        load_chunk<S, DC>(kp[i], tk);
                        load_chunk<S, DC>(vp[i], tv);
                        dk_t[i] = 0.f;
                        dv_t[i] = 0.f;
#pragma unroll
                        for (int d = 0; d < DC; ++d) {
                            dk_t[i] = fmaf(qf[d], tk[d], dk_t[i]);
                            dv_t[i] = fmaf(dof[d], tv[d], dv_t[i]);
                            kk[d] = fmaf(wt[i], tk[d], kk[d]);
                        }
                        dot = fmaf(wt[i], dk_t[i], dot);
                        dp = fmaf(wt[i], dv_t[i], dp);
                    }
                    dot = group_sum<G>(dot);
                    dp = group_sum<G>(dp);
                    const float p = __builtin_amdgcn_exp2f(dot * qscale - lse);
                    const float ds = p * (dp - delta);
#pragma unroll
                    for (int d = 0; d < DC; ++d) dqa[d] = fmaf(ds, kk[d], dqa[d]);
                    // per-tap terms, zero for taps outside the image; taps 00, 01, 10, 11 = (row, column)
                    const float a = ds * dm.sm_scale;
                    const bool c0in = inside & 1u, c1in = inside & 2u, r0in = inside & 4u, r1in = inside & 8u;
                    const float g0 = (c0in && r0in) ? fmaf(a, dk_t[0], p * dv_t[0]) : 0.f;
                    const float g1 = (c1in && r0in) ? fmaf(a, dk_t[1], p * dv_t[1]) : 0.f;
                    const float g2 = (c0in && r1in) ? fmaf(a, dk_t[2], p * dv_t[2]) : 0.f;
                    const float g3 = (c1in && r1in) ? fmaf(a, dk_t[3], p * dv_t[3]) : 0.f;
                    const float2 gf = s_g[slot * (G + 1) + t];              // fx, fy
                    const float dx0 = g1 - g0, dy0 = g2 - g0;
                    float gx = fmaf(gf.y, (g3 - g2) - dx0, dx0) * (float)(dm.Wimg - 1);
                    float gy = fmaf(gf.x, (g3 - g1) - dy0, dy0) * (float)(dm.Himg - 1);
                    gx = group_sum<G>(gx);
                    gy = group_sum<G>(gy);
                    if (t == my_trip) { my_gx = gx; my_gy = gy; }
                    continue;
                }
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
            if (CG && have && c0 + g < dm.P) {
                float *dst = dcoords_ + 2 * (crow + (size_t)s2 * dm.P + (size_t)my_n);
                atomicAdd(dst, my_gx);
                atomicAdd(dst + 1, my_gy);
            }
        }
        }
    }

#pragma unroll
    for (int rb = 0; rb < ROWS; ++rb) {
        if (have_s[rb]) {
#pragma unroll
            for (int d = 0; d < DC; ++d) dqa_s[rb][d] *= dm.sm_scale;
            store_chunk<S, DC>((char *)dq_ + roff_s[rb], dqa_s[rb]);
        }
    }
}

}  // namespace dsdpa
