// "Dense box" forward for clustered coordinates, 16-bit storage: the large matrix instructions of gfx950.
//
// Deformable sampling puts the samples of a query around a reference point, and neighbouring queries have
// neighbouring reference points: the taps of a TILE of 16 consecutive queries in one key view then fall into one
// small box of the image (64x64 image, centres spread over a fifth of it, 64 samples of sigma two pixels per
// query and view: 23 x 23 pixels in the median, 27 x 26 at most). Inside such a box the operator is two small
// dense products with a gather and a scatter between them, per (tile, key view, chunk of up to 64 samples per
// query):
//
//   S[16 x npix]  = scale * Q[16 x D] . K_box[npix x D]^T                (v_mfma_f32_16x16x32, contraction over D)
//   per sample:     logit = sum_t w_t * S[query][tap_t],  p = 2^(logit - m),  P[query][tap_t] += p * w_t
//   O[16 x D]    += P[16 x npix] . V_box[npix x D]                       (same instruction, contraction over pixels)
//
// A pixel row of K costs one matrix instruction per 32 elements for ALL 16 queries of the tile, where the
// per-query kernels pay a dot product per query and touched pixel.
//
// One workgroup of four waves owns a tile. S and P share one block of LDS (S as [pixel][query], P as
// [query][pixel]; P is built after the last S value was read); the softmax is online per chunk as in the other
// forward kernels. The rows of K and V go through LDS: the matrix instruction wants lane (n, g) to hold
// eight values of the contraction index for column n, so a load that fed it directly would have neighbouring
// lanes read from rows 256 bytes apart -- one L1 access per lane (measured: 64 per load instruction, the L1 busy
// 80 % of the time for 5 % of matrix-unit use). Here a wave fetches rows with neighbouring lanes on neighbouring
// bytes, parks them in a part of LDS of its own (no workgroup barrier inside the two products: LDS serves a
// wave's accesses in order), and reads them back in the instruction's layout:
//   * K (contraction over D, contiguous in a row): a 16-byte LDS read per lane and 32 elements; the waves take
//     the blocks of 16 pixels in turn;
//   * V (contraction over pixels, the rows' direction): ds_read_b64_tr_b16, the transposing LDS read of gfx950 --
//     within 16 lanes, lane i receives element (i & 3) of the 8-byte pieces that lanes (i >> 2) + 4 j, j = 0..3,
//     point at: with lane s pointing at elements [4 (s & 3), +4) of pixel s >> 2, lane i ends up with element i of
//     four pixels, which is the B operand's layout; every wave takes a quarter of the D columns for all 32 pixels
//     of a step (and fetches only that quarter of the rows), so no partial sums cross waves.
// The byte offsets of the box's pixels are tabled once per chunk, so that a fetch costs a table read and an add.
//
// P is accumulated in LDS as unsigned fixed point (24 fractional bits: every p*w is at most 1 and a pixel takes
// at most 64 of them per chunk; integer LDS atomics run at 11 lane-adds a clock and CU here, float ones at a
// third of one), then rounded to the storage type, once per chunk and in place, for the matrix instruction.
//
// A tile takes this path only if every one of its chunks has a box of at most DenseCfg::kPix pixels: the first chunk
// with a larger one ends the work on the tile (nothing of it has been written by then), which is marked in `todo`
// and left to fwd_gather_kernel; that kernel skips the tiles done here. Pixels of a box that no tap
// touches take part in the second product with coefficient 0; a tile whose sums come out non-finite (an infinity
// or NaN of V at such a pixel would do that) is left to the gather kernel too.
#pragma once
#include "dsdpa_common.h"

namespace dsdpa {

// Geometry of the kernel for head dimension D and tiles of TQ queries (16 or 32: one or two row blocks of the
// matrix instruction; four waves per row block). With two row blocks every staged row of K and V feeds two
// matrix instructions instead of one -- LDS bandwidth, 128 bytes a clock and CU against the 256 that four SIMDs'
// matrix units could take with one row block, is what bounds the products -- at twice the S / P block, which
// leaves room for one workgroup of eight waves per CU: measured slower than two of four, so the launcher
// instantiates 16.
template <int D, int TQ> struct DenseCfg {
    static_assert((D == 64 || D == 128) && (TQ == 16 || TQ == 32), "head dimension 64 or 128, one or two row blocks");
    static constexpr int kWaves = TQ / 4;                        // 4 or 8
    static constexpr int kThreads = kWaves * kWave;
    static constexpr int kSubs = kThreads / TQ;                  // 16 groups of four samples per query and chunk
    static constexpr int MT = TQ / 16;                           // row blocks
    static constexpr int NTW = D / 16 / kWaves;                  // column blocks of the second product per wave
    static_assert(NTW >= 1, "every wave has a column block");
    // pixels of a box, at most (a multiple of 32), and P's row pitch in 32-bit words: 4 mod 64, so that the 16 rows'
    // 16-byte reads spread over all banks; S [pixels][TQ] floats and P [TQ][pitch] words share the block
    static constexpr int kPix = TQ == 16 ? 704 : 768;
    static constexpr int kPitch = kPix + 4;
    static constexpr int kSpBytes = TQ * kPitch * 4;
    static_assert(kPitch % 64 == 4 && kPix * TQ * 4 <= kSpBytes, "S and P share the block");
    // staging, per wave: 16 pixel rows of K (row pitch D*2 + 16 bytes: 4 words mod 64, the 16 rows of a 16-byte read
    // land in different banks), or two buffers of 32 pixel rows of the wave's share of V's columns (NTW * 16
    // elements; row pitch 8 words mod 64 in 8-bank units -- or the 32 bytes themselves: the 8 rows that 32 lanes of a
    // transposing read touch land in different windows)
    static constexpr int kPitchK = D * 2 + 16;
    static constexpr int kPitchV = NTW * 32 + (NTW > 1 ? 32 : 0);
    static constexpr int kWaveStage = (16 * kPitchK > 2 * 32 * kPitchV) ? 16 * kPitchK : 2 * 32 * kPitchV;
    static constexpr int kStageBytes = kWaves * kWaveStage;
    static constexpr int kXmBytes = kSubs * TQ * 4;              // per-query exchange: [sample groups][queries]
    static constexpr int kXqBytes = TQ * 4 + 64;                 // per-query values for the lanes that hold rows of O; the waves' box parts
    static constexpr int kLdsBytes = kSpBytes + kStageBytes + kXmBytes + kXqBytes + 64 + kPix * 4;
};

typedef __bf16 dsdpa_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 dsdpa_f16x8 __attribute__((ext_vector_type(8)));
typedef float dsdpa_f32x2 __attribute__((ext_vector_type(2)));
typedef short dsdpa_i16x4 __attribute__((ext_vector_type(4)));
typedef unsigned dsdpa_u32x4 __attribute__((ext_vector_type(4)));      // (a 16-byte piece of a row in flight: plain vectors stay in registers)

template <typename S>
__device__ __forceinline__ floatx4 mfma_16x16x32(const uint4 &a, const uint4 &b, floatx4 c)
{
    if constexpr (S::kBf16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dsdpa_bf16x8, a), __builtin_bit_cast(dsdpa_bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(dsdpa_f16x8, a), __builtin_bit_cast(dsdpa_f16x8, b), c, 0, 0, 0);
}

// The transposing 8-byte LDS read (see the head of this file); `p` points into LDS, 8-byte aligned.
__device__ __forceinline__ uint2 lds_read_tr16(const unsigned char *p)
{
    typedef dsdpa_i16x4 __attribute__((address_space(3))) *lds_ptr;
    const dsdpa_i16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
    return __builtin_bit_cast(uint2, r);
}

// Orders this wave's earlier LDS accesses before its later ones for the COMPILER only. The LDS serves the
// instructions of one wave in the order they were issued, so a read that follows a write of the same wave in
// program order sees it without waiting for the write to be acknowledged; what must not happen is the compiler
// moving one across the other. (wave_lds_sync also waits for everything outstanding: a round trip per use.)
__device__ __forceinline__ void wave_lds_order()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Bounding box of the clamped tap pixels of a chunk, packed: lo = xmin | ymin << 16, hi = (0xffff - xmax) |
// (0xffff - ymax) << 16 (so that both are minima), 0xffffffff: no sample of the chunk has a tap inside the image.
struct DenseBox { int x0, y0, w, npix; };          // npix: w * h rounded up to 32; 0: the chunk does not fit

__device__ __forceinline__ DenseBox dense_box_from(uint32_t lo, uint32_t hi, int max_pix)
{
    int xlo = 0, ylo = 0, xhi = 0, yhi = 0;
    if (lo != 0xffffffffu) {                   // else: any one pixel will do
        xlo = (int)(lo & 0xffffu);
        ylo = (int)(lo >> 16);
        xhi = 0xffff - (int)(hi & 0xffffu);
        yhi = 0xffff - (int)(hi >> 16);
    }
    DenseBox b;
    b.x0 = xlo;
    b.y0 = ylo;
    b.w = xhi - xlo + 1;
    const int n = b.w * (yhi - ylo + 1);
    b.npix = n <= max_pix ? (n + 31) & ~31 : 0;
    return b;
}

// Four 24-bit fixed-point sums as four storage-type values for the matrix instruction (bf16: as they are, rounded
// to nearest even; fp16, which ends at 65504: times 2^-15).
template <typename S>
__device__ __forceinline__ uint2 dense_pack_p(const uint4 &a)
{
    const unsigned u[4] = { a.x, a.y, a.z, a.w };
    uint32_t w[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        if constexpr (S::kBf16) {
            dsdpa_f32x2 f = { (float)u[2 * j], (float)u[2 * j + 1] };
            w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, dsdpa_bf16x2));
        } else {
            union { uint32_t u; _Float16 h[2]; } cv;
            cv.h[0] = (_Float16)((float)u[2 * j] * 0x1p-15f);
            cv.h[1] = (_Float16)((float)u[2 * j + 1] * 0x1p-15f);
            w[j] = cv.u;
        }
    }
    return make_uint2(w[0], w[1]);
}

template <typename S, int D, int TQ>
__global__ __launch_bounds__((DenseCfg<D, TQ>::kThreads), 2) void fwd_dense_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, void *__restrict__ out_, float *__restrict__ lse_,
    unsigned char *__restrict__ todo_, Dims dm, int ntl)
{
    static_assert(S::kBytes == 2, "16-bit storage");
    using C = DenseCfg<D, TQ>;
    constexpr int KS = D / 32;                 // steps of the first product (and 16-byte loads per lane for 16 rows of K)
    constexpr int MT = C::MT, NTW = C::NTW, kWaves = C::kWaves, kThreads = C::kThreads, kSubs = C::kSubs;
    constexpr int CH = D / 8;                  // 16-byte pieces of a row of K
    constexpr int VCH = 2 * NTW;               // ... of a wave's share of a row of V
    constexpr int VLD = (32 * VCH + kWave - 1) / kWave;      // loads per lane for 32 rows of that share
    constexpr int kPitchK = C::kPitchK, kPitchV = C::kPitchV, kPitch = C::kPitch;
    constexpr int kRingK = 3, kRingV = 6;      // blocks of K, steps of V whose rows are in flight
    constexpr int kP16 = kPitch * 4;           // bytes between the rows of P, as 32-bit sums and as 16-bit values alike
    constexpr float kFix = 16777216.0f;        // 2^24
    constexpr float kUnfix = S::kBf16 ? 0x1p-24f : 0x1p-9f;      // what dense_pack_p leaves of it
    extern __shared__ __attribute__((aligned(16))) unsigned char dense_lds[];
    float *S_T = reinterpret_cast<float *>(dense_lds);                       // [pixel][TQ queries]
    unsigned *Pm = reinterpret_cast<unsigned *>(dense_lds);                  // [TQ queries][kPitch]
    float *xm = reinterpret_cast<float *>(dense_lds + C::kSpBytes + C::kStageBytes);   // [sample groups][TQ queries]
    float *xq = xm + kSubs * TQ;                                             // TQ per-query values for the lanes that hold rows of O
    uint32_t *boxw = reinterpret_cast<uint32_t *>(xq + TQ);                  // [waves][lo, hi]: the waves' parts of the chunk's box
    unsigned *offs = boxw + 32;                                              // byte offset of every pixel of the chunk's box

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned char *wstage = dense_lds + C::kSpBytes + wave * C::kWaveStage;  // this wave's staging
    const int tile = xcd_logical_block(blockIdx.x, gridDim.x);
    // tiles in the order (b, h, s1, tile of TQ pixels)
    int t = tile / ntl;
    const int l0 = (tile - t * ntl) * TQ;
    const int s1 = t % dm.V;
    t /= dm.V;
    const int h = t % dm.H, b = t / dm.H;
    const int nq = min(TQ, dm.L - l0);
    // (the flags for the gather kernel are kept per 16 queries, whatever TQ: (L + 15) / 16 of them per (b, h, s1))
    const size_t flag0 = (size_t)(tile / ntl) * (size_t)((dm.L + 15) >> 4) + (size_t)(l0 >> 4);
    // samples: thread (qi, sub) takes the samples [4 sub, 4 sub + 4) of a chunk for query qi
    const int qi = tid % TQ, sub = tid / TQ;
    const bool qlive = qi < nq;
    const int lq = l0 + min(qi, nq - 1);
    const float2 *crd_row = reinterpret_cast<const float2 *>(coords_) + (((size_t)b * dm.V + s1) * dm.L + lq) * (size_t)dm.N;
    // products: lane (n, g) of a wave: column n, k-group g
    const int n16 = lane & 15, g = lane >> 4;

    const int view_chunks = (dm.P + kWave - 1) / kWave;
    const int nchunks = dm.V * view_chunks;

    // Q as the A operand, per row block: row = query 16 mt + n16, eight consecutive elements per step at 8 g
    uint4 qf[MT][KS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const char *qrow = (const char *)q_ + dm.q_row(b, s1, h, l0 + min(mt * 16 + n16, nq - 1)) * 2;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[mt][ks] = *reinterpret_cast<const uint4 *>(qrow + ks * 64 + g * 16);
    }
    const float qscale = dm.sm_scale * kLog2e;
    const char *kplane0 = (const char *)k_ + dm.kv_plane(b, 0, h) * 2;
    const char *vplane0 = (const char *)v_ + dm.kv_plane(b, 0, h) * 2;
    const unsigned row_bytes = (unsigned)dm.kv_sl * 2u;

    floatx4 oacc[MT][NTW];                         // rows: queries 16 mt + 4 g .. + 3; column: element (wave * NTW + nt) * 16 + n16
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) oacc[mt][nt] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m_run = kNegBig, l_run = 0.f;            // of query qi; l_run: this thread's samples only

    // the coordinates of a chunk are requested a chunk ahead (they come from HBM or the memory-side cache, once per head)
    float2 xy_next[4];
    auto fetch_coords = [&](int ci) {
        const int s2 = ci / view_chunks, p0 = (ci - s2 * view_chunks) * kWave;
        const int cnt = min(kWave, dm.P - p0);
        const float2 *crd = crd_row + s2 * dm.P + p0;
#pragma unroll
        for (int i = 0; i < 4; ++i) xy_next[i] = crd[min(4 * sub + i, cnt - 1)];
    };
    fetch_coords(0);
    for (int ci = 0; ci < nchunks; ++ci) {
        const int s2 = ci / view_chunks, p0 = (ci - s2 * view_chunks) * kWave;
        const int cnt = min(kWave, dm.P - p0);
        // this thread's four samples of query qi: taps once, kept for the logits and the scatter further down
        const float2 xy_cur[4] = { xy_next[0], xy_next[1], xy_next[2], xy_next[3] };
        if (ci + 1 < nchunks) fetch_coords(ci + 1);
        float wgt[4][4];
        unsigned cpix[4];                       // clamped pixel of tap 00: column | row << 16
        unsigned cstep[4];                      // bit 0: tap 01 lies one column on, bit 1: tap 10 one row on
        uint32_t blo = 0xffffffffu, bhi = 0xffffffffu;
        {
            typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int p = 4 * sub + i;
                const bool live = qlive && p < cnt;
                const float2 xy = xy_cur[i];
                const Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
#pragma unroll
                for (int tpi = 0; tpi < 4; ++tpi) wgt[i][tpi] = live ? tp.w[tpi] : 0.f;
                const bool counted = (wgt[i][0] != 0.f) | (wgt[i][1] != 0.f) | (wgt[i][2] != 0.f) | (wgt[i][3] != 0.f);
                const int cx0 = min(max(tp.x0, 0), dm.Wimg - 1), cx1 = min(max(tp.x0 + 1, 0), dm.Wimg - 1);
                const int cy0 = min(max(tp.y0, 0), dm.Himg - 1), cy1 = min(max(tp.y0 + 1, 0), dm.Himg - 1);
                cpix[i] = (uint32_t)cx0 | ((uint32_t)cy0 << 16);
                cstep[i] = (cx1 > cx0 ? 1u : 0u) | (cy1 > cy0 ? 2u : 0u);
                const uint32_t l = counted ? cpix[i] : 0xffffffffu;
                const uint32_t u = counted ? (uint32_t)(0xffff - cx1) | ((uint32_t)(0xffff - cy1) << 16) : 0xffffffffu;
                blo = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, blo), __builtin_bit_cast(u16x2, l)));
                bhi = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, bhi), __builtin_bit_cast(u16x2, u)));
            }
            blo = wave_min_u16x2(blo);
            bhi = wave_min_u16x2(bhi);
            if (lane == 0) {
                boxw[wave * 2] = blo;
                boxw[wave * 2 + 1] = bhi;
            }
            __syncthreads();
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                const uint32_t l = boxw[w * 2], u = boxw[w * 2 + 1];
                blo = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, blo), __builtin_bit_cast(u16x2, l)));
                bhi = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, bhi), __builtin_bit_cast(u16x2, u)));
            }
        }
        const DenseBox bxv = dense_box_from(__builtin_amdgcn_readfirstlane(blo), __builtin_amdgcn_readfirstlane(bhi), C::kPix);
        if (bxv.npix == 0) {
            // this chunk's box is too large: nothing of the tile has been written yet; the gather kernel takes it
            if (tid < TQ / 16 && l0 + 16 * tid < dm.L) todo_[flag0 + tid] = 1;
            return;
        }
        const int bx0 = bxv.x0, by0 = bxv.y0, bw = bxv.w, npix = bxv.npix;
        const float rbw = 1.0f / (float)bw;
        const unsigned view_off = (unsigned)s2 * (unsigned)dm.kv_sv * 2u;
        // byte offset, in a (batch, head)'s K or V, of every box pixel (row-major over the box; the padding behind
        // the last pixel repeats pixels of the box)
        for (int pidx = tid; pidx < npix; pidx += kThreads) {
            const int ry = (int)(((float)pidx + 0.5f) * rbw);                 // pidx / bw, exact for these small numbers
            const int rx = pidx - ry * bw;
            const int y = min(by0 + ry, dm.Himg - 1), x = min(bx0 + rx, dm.Wimg - 1);
            offs[pidx] = view_off + (unsigned)(y * dm.Wimg + x) * row_bytes;
        }
        __syncthreads();

        // ---- S = scale * Q . K^T: the waves take the blocks of 16 pixels in turn. A block's rows come in with
        // neighbouring lanes on neighbouring bytes (lane -> piece lane % CH of row lane / CH, + 64 / CH rows per
        // further load), are parked in the wave's staging and read back as the B operand, once for all row blocks.
        {
            const int nblk = npix >> 4;
            const int krow = lane / CH;
            const unsigned kpiece = (unsigned)(lane % CH) * 16u;
            // the rows of the next kRingK blocks of this wave are in flight (a block's 16-byte loads return after
            // about as long as three blocks take)
            dsdpa_u32x4 kr[kRingK][KS];
#define DSDPA_DENSE_FETCH_K(slot_, nb_)                                                                        \
            _Pragma("unroll") for (int r = 0; r < KS; ++r)                                                     \
                kr[slot_][r] = *reinterpret_cast<const dsdpa_u32x4 *>(kplane0 + offs[min((nb_), nblk - 1) * 16 + r * (kWave / CH) + krow] + kpiece);
#pragma unroll
            for (int u = 0; u < kRingK; ++u) { DSDPA_DENSE_FETCH_K(u, wave + kWaves * u) }
            for (int nb0 = wave; nb0 < nblk; nb0 += kWaves * kRingK) {
#pragma unroll
                for (int u = 0; u < kRingK; ++u) {
                    const int nb = nb0 + kWaves * u;
                    if (nb < nblk) {
                        wave_lds_order();                  // (behind the reads of the previous block)
#pragma unroll
                        for (int r = 0; r < KS; ++r)
                            *reinterpret_cast<dsdpa_u32x4 *>(wstage + (r * (kWave / CH) + krow) * kPitchK + kpiece) = kr[u][r];
                        wave_lds_order();
                        DSDPA_DENSE_FETCH_K(u, nb + kWaves * kRingK)          // (behind the last one: unused)
                        floatx4 acc[MT];
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
                        const unsigned char *kfrag = wstage + n16 * kPitchK + g * 16;
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            const uint4 bf = *reinterpret_cast<const uint4 *>(kfrag + ks * 64);
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt) acc[mt] = mfma_16x16x32<S>(qf[mt][ks], bf, acc[mt]);
                        }
                        // rows 16 mt + 4 g .. + 3 (queries) of column n16 (pixel nb * 16 + n16)
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            *reinterpret_cast<float4 *>(S_T + (nb * 16 + n16) * TQ + mt * 16 + 4 * g) =
                                make_float4(acc[mt][0] * qscale, acc[mt][1] * qscale, acc[mt][2] * qscale, acc[mt][3] * qscale);
                    }
                }
            }
#undef DSDPA_DENSE_FETCH_K
        }
        __syncthreads();

        // the first steps' rows of V are requested here already, under the work on the samples: their addresses are
        // known (offs), and the registers are there (two waves per SIMD)
        const int nkb = npix >> 5;
        // row of a load's 64 / VCH that this lane fetches and parks. Four lanes per row: the 16 lanes that one
        // cycle of a 16-byte LDS write serves take every other row (rows of 96 bytes: 0, 2, 4, 6 start in four
        // different quarters of the banks, 0, 1, 2, 3 do not)
        const int vrow_l = VCH == 4 ? 8 * (lane >> 5) + ((lane >> 4) & 1) + 2 * ((lane & 15) >> 2) : lane / VCH;
        const unsigned vpiece = (unsigned)(wave * NTW * 32 + (lane % VCH) * 16);   // byte in the row of V
        const unsigned vpark = (unsigned)(lane % VCH) * 16u;
        // the next kRingV steps' rows are in flight, the next step's are parked while this one is worked on
        dsdpa_u32x4 vr[kRingV][VLD];
#define DSDPA_DENSE_FETCH_V(slot_, kb_)                                                                        \
        _Pragma("unroll") for (int r = 0; r < VLD; ++r)                                                    \
            vr[slot_][r] = *reinterpret_cast<const dsdpa_u32x4 *>(vplane0 + offs[min((kb_), nkb - 1) * 32 + r * (kWave / VCH) + vrow_l] + vpiece);
#define DSDPA_DENSE_PARK_V(slot_, buf_)                                                                        \
        _Pragma("unroll") for (int r = 0; r < VLD; ++r)                                                    \
            *reinterpret_cast<dsdpa_u32x4 *>(wstage + ((buf_) * 32 + r * (kWave / VCH) + vrow_l) * kPitchV + vpark) = vr[slot_][r];
#pragma unroll
        for (int u = 0; u < kRingV; ++u) { DSDPA_DENSE_FETCH_V(u, u) }

        // ---- the samples of query qi, four per thread: logits from S, then the softmax bookkeeping of the chunk
        float logit[4];
        unsigned ent[4];                        // entry of tap 00 | (column step << 16) | (row step << 17)
        float m_chunk = kNegBig;
        const int bh = (npix + bw - 1) / bw;    // (rows the tables reach, the padding's included)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool live = qlive && 4 * sub + i < cnt;
            // (a sample that counts lies inside the box; the others carry weight 0 and are only kept inside the tables)
            const int ex = min(max((int)(cpix[i] & 0xffffu) - bx0, 0), bw - 1), ey = min(max((int)(cpix[i] >> 16) - by0, 0), bh - 1);
            const int e0 = min(ey * bw + ex, npix - 1);
            const int dx = ((cstep[i] & 1u) && ex + 1 < bw) ? 1 : 0;
            const int dy = ((cstep[i] & 2u) && e0 + bw + dx < npix) ? 1 : 0;
            ent[i] = (unsigned)e0 | ((unsigned)dx << 16) | ((unsigned)dy << 17);
            const int e1 = min(e0 + dx, npix - 1), e2 = e0 + dy * bw, e3 = min(e2 + dx, npix - 1);
            const float lg = fmaf(wgt[i][0], S_T[e0 * TQ + qi], fmaf(wgt[i][1], S_T[e1 * TQ + qi],
                             fmaf(wgt[i][2], S_T[e2 * TQ + qi], wgt[i][3] * S_T[e3 * TQ + qi])));
            logit[i] = live ? lg : kNegBig;
            m_chunk = fmaxf(m_chunk, logit[i]);
        }
        xm[sub * TQ + qi] = m_chunk;
        __syncthreads();                           // (every S value has been read as well)
#pragma unroll
        for (int s = 0; s < kSubs; ++s) m_chunk = fmaxf(m_chunk, xm[s * TQ + qi]);
        const float m_new = fmaxf(m_run, m_chunk);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        l_run *= alpha;
        if (sub == 0) xq[qi] = alpha;
        // clear P where the box reaches
        for (int idx = tid; idx < TQ * (kPitch / 4); idx += kThreads) {
            const int r = idx / (kPitch / 4), c = idx - r * (kPitch / 4);
            if (4 * c < npix) *reinterpret_cast<uint4 *>(Pm + r * kPitch + 4 * c) = make_uint4(0u, 0u, 0u, 0u);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float p = __builtin_amdgcn_exp2f(logit[i] - m_new);          // (a dead sample: 2^(-huge) = 0)
            l_run += p;
            const unsigned e0 = ent[i] & 0xffffu, dx = (ent[i] >> 16) & 1u, dyw = ((ent[i] >> 17) & 1u) * (unsigned)bw;
            unsigned *prow = Pm + qi * kPitch;
            const float pf = p * kFix;
            atomicAdd(prow + e0, (unsigned)(pf * wgt[i][0] + 0.5f));
            atomicAdd(prow + min(e0 + dx, (unsigned)npix - 1u), (unsigned)(pf * wgt[i][1] + 0.5f));
            atomicAdd(prow + e0 + dyw, (unsigned)(pf * wgt[i][2] + 0.5f));
            atomicAdd(prow + min(e0 + dyw + dx, (unsigned)npix - 1u), (unsigned)(pf * wgt[i][3] + 0.5f));
        }
        // rows of O are queries 16 mt + 4 g .. + 3 in this lane
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float4 al = *reinterpret_cast<const float4 *>(xq + mt * 16 + 4 * g);
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                oacc[mt][nt][0] *= al.x; oacc[mt][nt][1] *= al.y; oacc[mt][nt][2] *= al.z; oacc[mt][nt][3] *= al.w;
            }
        }
        __syncthreads();                           // P is complete
        // P as 16-bit values for the matrix instruction, in place: every thread takes its pieces of four sums into
        // registers, and after a barrier leaves four values where the row's first half was
        {
            constexpr int kQuads = kPitch / 4;                                   // 16-byte pieces of a row
            constexpr int kMine = (TQ * kQuads + kThreads - 1) / kThreads;
            uint2 mine[kMine];
#pragma unroll
            for (int i = 0; i < kMine; ++i) {
                const int idx = tid + i * kThreads, r = idx / kQuads, c = idx - r * kQuads;
                mine[i] = make_uint2(0u, 0u);
                if (r < TQ && 4 * c < npix) mine[i] = dense_pack_p<S>(*reinterpret_cast<const uint4 *>(Pm + r * kPitch + 4 * c));
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < kMine; ++i) {
                const int idx = tid + i * kThreads, r = idx / kQuads, c = idx - r * kQuads;
                if (r < TQ && 4 * c < npix) *reinterpret_cast<uint2 *>(dense_lds + r * kP16 + c * 8) = mine[i];
            }
            __syncthreads();
        }

        // ---- O += P . V, 32 pixels a step; this wave's share of the columns, two staging buffers used in turn.
        // Contraction slot j of k-group g is pixel 4 g + j of the step for j < 4, 16 + 4 g + (j - 4) after: the A
        // operand is then two 8-byte reads of P, and the 8 rows that 32 lanes of a transposing read touch are 8
        // consecutive ones.
        {
            wave_lds_order();                      // (behind the last reads of K's staging)
            DSDPA_DENSE_PARK_V(0, 0)
            DSDPA_DENSE_FETCH_V(0, kRingV)
            const int s16 = lane & 15;
            // (slot of step kb: kb % kRingV; step kb + 1 is parked, and its slot refilled with step kb + 1 + kRingV,
            // while step kb is worked on)
            for (int kb0 = 0; kb0 < nkb; kb0 += kRingV) {
#pragma unroll
                for (int u = 0; u < kRingV; ++u) {
                    const int kb = kb0 + u;
                    if (kb < nkb) {
                        const int buf = kb & 1;
                        wave_lds_order();                  // (buffer `buf` is parked, the other one's reads are issued)
                        uint4 af[MT];
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) {
                            const unsigned char *prow = dense_lds + (mt * 16 + n16) * kP16 + (kb * 32 + 4 * g) * 2;
                            const uint2 a0 = *reinterpret_cast<const uint2 *>(prow), a1 = *reinterpret_cast<const uint2 *>(prow + 32);
                            af[mt] = make_uint4(a0.x, a0.y, a1.x, a1.y);
                        }
                        const unsigned char *vfrag = wstage + (buf * 32 + 4 * g + (s16 >> 2)) * kPitchV + 4 * (s16 & 3) * 2;
#pragma unroll
                        for (int nt = 0; nt < NTW; ++nt) {
                            const uint2 b0 = lds_read_tr16(vfrag + nt * 32), b1 = lds_read_tr16(vfrag + 16 * kPitchV + nt * 32);
                            const uint4 bf = make_uint4(b0.x, b0.y, b1.x, b1.y);
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt) oacc[mt][nt] = mfma_16x16x32<S>(af[mt], bf, oacc[mt][nt]);
                        }
                        const int un = (u + 1) % kRingV;                      // (a constant once the loop is unrolled)
                        DSDPA_DENSE_PARK_V(un, buf ^ 1)                       // (step kb + 1; behind the last one: unused)
                        DSDPA_DENSE_FETCH_V(un, kb + 1 + kRingV)
                    }
                }
            }
#undef DSDPA_DENSE_FETCH_V
#undef DSDPA_DENSE_PARK_V
        }
        __syncthreads();                           // every wave is done with this chunk's P and table of offsets
    }

    // ---- out = O / l, lse = m + log2 l
    // Pixels of a box that no tap touches took part in the second product with coefficient 0: should V hold an
    // infinity or a NaN there, the sums are NaN where the operator's result is finite. Such a tile is left to the
    // gather kernel, which reads touched pixels only.
    bool bad = false;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            const float sum = (oacc[mt][nt][0] + oacc[mt][nt][1]) + (oacc[mt][nt][2] + oacc[mt][nt][3]);
            bad = bad || !(fabsf(sum) <= 3.0e38f);
        }
    if (tid == 0) boxw[0] = 0u;
    xm[sub * TQ + qi] = l_run;
    __syncthreads();
    if (bad) boxw[0] = 1u;
    float l_tot = 0.f;
#pragma unroll
    for (int s = 0; s < kSubs; ++s) l_tot += xm[s * TQ + qi];
    if (sub == 0) {
        xq[qi] = kUnfix / l_tot;
        if (qlive) lse_[(((size_t)b * dm.V + s1) * dm.H + h) * dm.L + lq] = m_run + __log2f(l_tot);
    }
    __syncthreads();
    {
        constexpr int OP = D + 4;                 // pitch of the staging rows: the four row groups land in different banks
        float *O_s = reinterpret_cast<float *>(dense_lds);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float4 inv = *reinterpret_cast<const float4 *>(xq + mt * 16 + 4 * g);
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                const int col = (wave * NTW + nt) * 16 + n16;
                O_s[(mt * 16 + 4 * g + 0) * OP + col] = oacc[mt][nt][0] * inv.x;
                O_s[(mt * 16 + 4 * g + 1) * OP + col] = oacc[mt][nt][1] * inv.y;
                O_s[(mt * 16 + 4 * g + 2) * OP + col] = oacc[mt][nt][2] * inv.z;
                O_s[(mt * 16 + 4 * g + 3) * OP + col] = oacc[mt][nt][3] * inv.w;
            }
        }
        __syncthreads();
        const bool redo = boxw[0] != 0u;
        if (tid < TQ / 16 && l0 + 16 * tid < dm.L) todo_[flag0 + tid] = redo ? 1 : 0;
        if (redo) return;
        // TQ rows of D elements, 8 elements (16 bytes of output) a thread and pass
        for (int idx = tid; idx < TQ * (D / 8); idx += kThreads) {
            const int r = idx / (D / 8), c8 = idx - r * (D / 8);
            if (r < nq) {
                float v8[8];
                const float4 a = *reinterpret_cast<const float4 *>(O_s + r * OP + 8 * c8);
                const float4 c = *reinterpret_cast<const float4 *>(O_s + r * OP + 8 * c8 + 4);
                v8[0] = a.x; v8[1] = a.y; v8[2] = a.z; v8[3] = a.w; v8[4] = c.x; v8[5] = c.y; v8[6] = c.z; v8[7] = c.w;
                const size_t row = (((size_t)b * dm.V + s1) * dm.H + h) * dm.L + l0 + r;
                store_chunk<S, 8>((char *)out_ + (row * D + 8 * c8) * 2, v8);
            }
        }
    }
}

}  // namespace dsdpa
