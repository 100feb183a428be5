// dk/dv kernel with LDS-privatised accumulation.
//
// A workgroup owns one tile of one key/value plane (b, h, s2): th x tw "cells"
// (a cell is the 2x2 pixel block a sample's taps fall on, named by its top-left
// pixel) plus a one-pixel halo to the right and below, so that every tap of a
// sample whose cell is owned lands inside the tile. The tile's dK and dV live in
// LDS as double accumulators updated with ds_add_f64 (on gfx950 the LDS fp64
// atomic runs ~20x faster than the fp32 one), and are flushed to the global
// fp32 accumulators once, with coalesced float atomics (halo pixels are shared
// with the neighbouring tiles). The workgroup walks a range of query rows that
// sample this plane; each wave takes a query, turns its P coordinates for view
// s2 into tap descriptors, keeps (compacts) the ones whose cell the tile owns,
// and processes them G lanes per sample like the gather kernels: K/V taps come
// from global memory (L2), p and ds are recomputed from the stored
// log-sum-exp and delta.
#pragma once
#include "dsdpa_common.h"

namespace dsdpa {

constexpr int kTileWaves = 16;

struct TileGeom {
    int th, tw;        // owned cells per tile (rows, cols)
    int nty, ntx;      // tiles per plane
    int lh, lw;        // pixels held in LDS per tile (th+1, tw+1, clipped to the image)
    int qsplit;        // workgroups sharing one (plane, tile): each takes a slice of the V*L query rows
};

__device__ __forceinline__ void lds_accumulate(double *p, float x) { atomicAdd(p, (double)x); }

template <typename S, int D, int DC>
__global__ __launch_bounds__(kTileWaves *kWave) void bwd_dkdv_tile_kernel(
    const void *__restrict__ q_, const void *__restrict__ k_, const void *__restrict__ v_,
    const float *__restrict__ coords_, const float2 *__restrict__ stats_,
    const void *__restrict__ dout_, float *__restrict__ dk_acc, float *__restrict__ dv_acc,
    Dims dm, TileGeom tg)
{
    constexpr int G = D / DC;
    constexpr int NS = kWave / G;
    static_assert(G >= 1 && G <= 16 && G * DC == D, "lane split");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tile_elems = tg.lh * tg.lw * D;
    double *tileK = reinterpret_cast<double *>(smem);
    double *tileV = tileK + tile_elems;
    float4 *s_w_all = reinterpret_cast<float4 *>(tileV + tile_elems);
    uint4 *s_e_all = reinterpret_cast<uint4 *>(s_w_all + kTileWaves * kWave);
    int *s_loc_all = reinterpret_cast<int *>(s_e_all + kTileWaves * kWave);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index is uniform: keep it in an SGPR
    float4 *s_w = s_w_all + wave * kWave;
    uint4 *s_e = s_e_all + wave * kWave;
    int *s_loc = s_loc_all + wave * kWave;

    // block -> (plane, tile, query slice); plane-major so that an XCD's L2 keeps few planes
    int bid = xcd_logical_block(blockIdx.x, gridDim.x);
    const int part = bid % tg.qsplit;
    bid /= tg.qsplit;
    const int ntiles = tg.nty * tg.ntx;
    const int tile = bid % ntiles;
    const int plane = bid / ntiles;
    const int s2 = plane % dm.V;
    const int h = (plane / dm.V) % dm.H;
    const int b = plane / (dm.V * dm.H);
    const int ya = (tile / tg.ntx) * tg.th, xa = (tile % tg.ntx) * tg.tw;   // first owned cell

    for (int i = threadIdx.x; i < 2 * tile_elems; i += blockDim.x) tileK[i] = 0.0;
    __syncthreads();

    const size_t plane_base = (((size_t)b * dm.V + s2) * dm.H + h) * (size_t)dm.L * D;   // elements in dk/dv
    const char *kb = (const char *)k_ + dm.kv_plane(b, s2, h) * S::kBytes;
    const char *vb = (const char *)v_ + dm.kv_plane(b, s2, h) * S::kBytes;
    const int g = lane % G, slot = lane / G, lane_elem = g * DC;
    const float qscale = dm.sm_scale * kLog2e;
    const float2 *coords = (const float2 *)coords_;

    const int nq = dm.V * dm.L;                                  // query rows (s1, l) sampling this plane
    const int q_lo = (int)(((long long)nq * part) / tg.qsplit);
    const int q_hi = (int)(((long long)nq * (part + 1)) / tg.qsplit);

    for (int qi = q_lo + wave; qi < q_hi; qi += kTileWaves) {
        const int s1 = qi / dm.L, l = qi % dm.L;
        const size_t row = (((size_t)b * dm.V + s1) * dm.H + h) * dm.L + l;
        const size_t cbase = ((((size_t)b * dm.V + s1) * dm.L + l) * dm.V + s2) * (size_t)dm.P;
        float qf[DC], dof[DC];
        bool row_loaded = false;
        float lse = 0.f, delta = 0.f;

        for (int c0 = 0; c0 < dm.P; c0 += kWave) {
            // one sample per lane: descriptor + ownership test, then compaction
            const int n = c0 + lane;
            const bool in_range = n < dm.P;
            float2 xy = coords[cbase + (in_range ? n : dm.P - 1)];
            Taps tp = make_taps(xy.x, xy.y, dm.Wimg, dm.Himg);
            const int oy = min(max(tp.y0, 0), dm.Himg - 1), ox = min(max(tp.x0, 0), dm.Wimg - 1);
            const bool any_w = (tp.w[0] != 0.f) | (tp.w[1] != 0.f) | (tp.w[2] != 0.f) | (tp.w[3] != 0.f);
            const bool mine = in_range & any_w & (oy >= ya) & (oy < ya + tg.th) & (ox >= xa) & (ox < xa + tg.tw);
            const unsigned long long mask = __ballot(mine);
            const int cnt = __popcll(mask);
            if (cnt == 0) continue;                               // wave-uniform
            const int pos = __popcll(mask & ((1ull << lane) - 1ull));
            wave_lds_sync();
            if (mine) {
                s_w[pos] = make_float4(tp.w[0], tp.w[1], tp.w[2], tp.w[3]);
                s_e[pos] = make_uint4((unsigned)(tp.pix[0] * dm.kv_sl) * S::kBytes, (unsigned)(tp.pix[1] * dm.kv_sl) * S::kBytes,
                                      (unsigned)(tp.pix[2] * dm.kv_sl) * S::kBytes, (unsigned)(tp.pix[3] * dm.kv_sl) * S::kBytes);
                s_loc[pos] = ((tp.y0 - ya) * tg.lw + (tp.x0 - xa)) * D;   // tile-local offset of tap 00
            }
            wave_lds_sync();
            if (!row_loaded) {
                const size_t roff = (row * D + lane_elem) * S::kBytes;
                load_chunk<S, DC>((const char *)q_ + (dm.q_row(b, s1, h, l) + lane_elem) * S::kBytes, qf);
                load_chunk<S, DC>((const char *)dout_ + roff, dof);
                const float2 ld = stats_[row];
                lse = ld.x;
                delta = ld.y;
                row_loaded = true;
            }
            for (int j0 = 0; j0 < cnt; j0 += NS) {
                const int j = j0 + slot;
                const bool live = j < cnt;
                const int jj = live ? j : cnt - 1;
                float4 w = s_w[jj];
                const uint4 e = lane_offsets(s_e[jj], (unsigned)lane_elem * S::kBytes);
                const int loc = s_loc[jj];
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
                const float p = live ? __builtin_amdgcn_exp2f(dot * qscale - lse) : 0.f;
                const float dss = p * (dp - delta) * dm.sm_scale;
                const float wt[4] = { w.x, w.y, w.z, w.w };
                const int lt[4] = { loc, loc + D, loc + tg.lw * D, loc + (tg.lw + 1) * D };
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    if (live && wt[t] != 0.f) {
                        const float ck = wt[t] * dss, cv = wt[t] * p;
                        double *pk = tileK + lt[t] + lane_elem;
                        double *pv = tileV + lt[t] + lane_elem;
#pragma unroll
                        for (int d = 0; d < DC; ++d) {
                            lds_accumulate(pk + d, ck * qf[d]);
                            lds_accumulate(pv + d, cv * dof[d]);
                        }
                    }
                }
            }
        }
    }
    __syncthreads();
    // flush: tile pixel (ly, lx) -> image pixel (ya+ly, xa+lx); halo pixels may belong to no image row/col
    float *dkb = dk_acc + plane_base, *dvb = dv_acc + plane_base;
    for (int i = threadIdx.x; i < tile_elems; i += blockDim.x) {
        const int d = i % D, px = i / D;
        const int ly = px / tg.lw, lx = px % tg.lw;
        const int y = ya + ly, x = xa + lx;
        if (y < dm.Himg && x < dm.Wimg) {
            const size_t gi = ((size_t)y * dm.Wimg + x) * D + d;
            const float a = (float)tileK[i], c = (float)tileV[i];
            if (a != 0.f) atomicAdd(dkb + gi, a);
            if (c != 0.f) atomicAdd(dvb + gi, c);
        }
    }
}

}  // namespace dsdpa
