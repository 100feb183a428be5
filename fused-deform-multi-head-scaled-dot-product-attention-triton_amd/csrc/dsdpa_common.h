// Device-side building blocks shared by every kernel of the deformable
// multi-view SDPA library: storage-type conversion, bilinear tap computation,
// wave-level (64-lane) reductions, XCD-aware work mapping.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace dsdpa {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -1.0e30f;   // finite stand-in for -inf in running maxima
constexpr int kWave = 64;
constexpr int kXcds = 8;              // MI355X: 8 XCDs, workgroups dealt round-robin

// Division of a 31-bit unsigned by a run-time constant d: q = (n * mul) >> (31 + shift), exact for every
// n < 2^31 (round-up method: shift = ceil(log2 d), mul = ceil(2^(31+shift) / d) <= 2^32 - 1, or 2^31 for d = 1).
struct FastDiv {
    unsigned mul, shift;
    __host__ static FastDiv make(unsigned d)
    {
        FastDiv f;
        unsigned s = 0;
        while ((1ull << s) < d) ++s;
        f.shift = s;
        f.mul = (unsigned)(((1ull << (31 + s)) + d - 1) / d);
        return f;
    }
    __device__ __forceinline__ unsigned div(unsigned n) const
    {
        return (unsigned)(((unsigned long long)n * mul) >> (31 + shift));
    }
};

struct Dims {
    int B, V, H, Himg, Wimg, L, P, N;   // N = V*P samples per query row
    int rows;                           // B*V*H*L query rows
    float sm_scale;
    FastDiv divP, divL;                 // for decoding sample ids (s1*L + l)*P + p
    // Element strides of the inputs q and k/v (k and v share one set) over (batch, view, head, pixel); the head
    // dimension itself is contiguous. Everything else (out, lse, dout, the gradients) is contiguous
    // [B][V][H][L][D]. Offsets inside one (batch, head) -- view*sv + pixel*sl -- fit 32 bits.
    long long q_sb, q_sh, kv_sb, kv_sh;
    int q_sv, q_sl, kv_sv, kv_sl;
    __device__ __forceinline__ size_t q_row(int b, int s1, int h, int l) const
    {
        return (size_t)((long long)b * q_sb + (long long)h * q_sh) + (size_t)((unsigned)s1 * (unsigned)q_sv + (unsigned)l * (unsigned)q_sl);
    }
    __device__ __forceinline__ size_t kv_plane(int b, int view, int h) const
    {
        return (size_t)((long long)b * kv_sb + (long long)h * kv_sh) + (size_t)((unsigned)view * (unsigned)kv_sv);
    }
};

// ------------------------------------------------------------------ storage types
struct F32 {
    using type = float;
    static constexpr int kBytes = 4;
    static constexpr bool kBf16 = false;
};
struct BF16 {
    using type = uint16_t;
    static constexpr int kBytes = 2;
    static constexpr bool kBf16 = true;
};
struct F16 {
    using type = _Float16;
    static constexpr int kBytes = 2;
    static constexpr bool kBf16 = false;
};

__device__ __forceinline__ float bf16_to_f32(uint16_t x) { return __uint_as_float(((uint32_t)x) << 16); }

// round-to-nearest-even; NaN stays NaN (quiet)
__device__ __forceinline__ uint16_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Load DC consecutive elements, widened to fp32. The address is 16-byte aligned, or 8-byte aligned
// for a 4-element 16-bit chunk.
template <typename S, int DC>
__device__ __forceinline__ void load_chunk(const void *p, float (&dst)[DC])
{
    if constexpr (S::kBytes == 4) {
        static_assert(DC % 4 == 0, "fp32 chunks are multiples of 4 elements");
        const float4 *src = reinterpret_cast<const float4 *>(p);
#pragma unroll
        for (int i = 0; i < DC / 4; ++i) {
            float4 t = src[i];
            dst[4 * i + 0] = t.x; dst[4 * i + 1] = t.y; dst[4 * i + 2] = t.z; dst[4 * i + 3] = t.w;
        }
    } else {
        static_assert(DC % 4 == 0, "16-bit chunks are multiples of 4 elements");
        uint32_t w[DC / 2];
        if constexpr (DC % 8 == 0) {
            const uint4 *src = reinterpret_cast<const uint4 *>(p);
#pragma unroll
            for (int i = 0; i < DC / 8; ++i) {
                uint4 t = src[i];
                w[4 * i + 0] = t.x; w[4 * i + 1] = t.y; w[4 * i + 2] = t.z; w[4 * i + 3] = t.w;
            }
        } else {
            const uint2 *src = reinterpret_cast<const uint2 *>(p);      // 8-byte aligned
#pragma unroll
            for (int i = 0; i < DC / 4; ++i) {
                uint2 t = src[i];
                w[2 * i + 0] = t.x; w[2 * i + 1] = t.y;
            }
        }
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

// ---- 16-bit storage: packed pairs straight into the dot-product instructions (no widening) ----
// DC consecutive 16-bit elements as DC/2 packed pairs.
template <typename S, int DC>
__device__ __forceinline__ void load_packed(const void *p, uint32_t (&w)[DC / 2])
{
    static_assert(S::kBytes == 2 && DC % 4 == 0, "packed pairs exist for 16-bit storage only");
    if constexpr (DC % 8 == 0) {
        const uint4 *src = reinterpret_cast<const uint4 *>(p);
#pragma unroll
        for (int i = 0; i < DC / 8; ++i) {
            uint4 t = src[i];
            w[4 * i + 0] = t.x; w[4 * i + 1] = t.y; w[4 * i + 2] = t.z; w[4 * i + 3] = t.w;
        }
    } else {
        const uint2 *src = reinterpret_cast<const uint2 *>(p);
#pragma unroll
        for (int i = 0; i < DC / 4; ++i) {
            uint2 t = src[i];
            w[2 * i + 0] = t.x; w[2 * i + 1] = t.y;
        }
    }
}

typedef __attribute__((ext_vector_type(2))) __bf16 dsdpa_bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 dsdpa_f16x2;

// sum_d a[d] * b[d] over DC elements held as packed pairs: v_dot2_f32_bf16 / v_dot2_f32_f16, products
// exact in fp32, fp32 accumulation.
template <typename S, int DC>
__device__ __forceinline__ float packed_dot(const uint32_t (&a)[DC / 2], const uint32_t (&b)[DC / 2])
{
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < DC / 2; ++i) {
        if constexpr (S::kBf16)
            acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(dsdpa_bf16x2, a[i]),
                                                  __builtin_bit_cast(dsdpa_bf16x2, b[i]), acc, false);
        else
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(dsdpa_f16x2, a[i]),
                                         __builtin_bit_cast(dsdpa_f16x2, b[i]), acc, false);
    }
    return acc;
}

// x . (w.x*tap0 + w.y*tap1 + w.z*tap2 + w.w*tap3) for this lane's DC elements, 16-bit storage: four packed
// dot products against the un-widened taps, then the bilinear weights on the four scalars (the blend is
// linear, so it commutes with the dot product).
template <typename S, int DC>
__device__ __forceinline__ float tap_dot16(const void *p0, const void *p1, const void *p2, const void *p3,
                                           const float4 &w, const uint32_t (&x)[DC / 2])
{
    uint32_t t0[DC / 2], t1[DC / 2], t2[DC / 2], t3[DC / 2];
    load_packed<S, DC>(p0, t0);
    load_packed<S, DC>(p1, t1);
    load_packed<S, DC>(p2, t2);
    load_packed<S, DC>(p3, t3);
    const float d0 = packed_dot<S, DC>(x, t0), d1 = packed_dot<S, DC>(x, t1);
    const float d2 = packed_dot<S, DC>(x, t2), d3 = packed_dot<S, DC>(x, t3);
    return fmaf(w.x, d0, fmaf(w.y, d1, fmaf(w.z, d2, w.w * d3)));
}

// Store DC consecutive fp32 values, narrowed (RNE) to the storage type.
template <typename S, int DC>
__device__ __forceinline__ void store_chunk(void *p, const float (&src)[DC])
{
    if constexpr (S::kBytes == 4) {
        float4 *dst = reinterpret_cast<float4 *>(p);
#pragma unroll
        for (int i = 0; i < DC / 4; ++i)
            dst[i] = make_float4(src[4 * i], src[4 * i + 1], src[4 * i + 2], src[4 * i + 3]);
    } else {
        uint4 *dst = reinterpret_cast<uint4 *>(p);
#pragma unroll
        for (int i = 0; i < DC / 8; ++i) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float a = src[8 * i + 2 * j], b = src[8 * i + 2 * j + 1];
                if constexpr (S::kBf16) {
                    w[j] = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
                } else {
                    union { uint32_t u; _Float16 h[2]; } cv;
                    cv.h[0] = (_Float16)a;
                    cv.h[1] = (_Float16)b;
                    w[j] = cv.u;
                }
            }
            dst[i] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

// ------------------------------------------------------------------ bilinear taps
// The four taps of one normalised coordinate. x_pix = x*(W-1), y_pix = y*(Himg-1)
// (align_corners=True), written as the two-step un-normalisation the library
// routine uses so that both sides see the same fp32 roundings. Zero padding is
// per tap: a tap outside the image gets weight 0 (its pixel index is clamped
// into the image so that the gather stays in bounds), the other taps keep
// theirs. NaN/inf coordinates drop all four taps.
struct Taps {
    float w[4];     // 00 (row0,col0), 01 (row0,col1), 10, 11
    int pix[4];     // row*W + col, always inside [0, L)
    int x0, y0;     // floor of the pixel coordinate, limited to [-2, size+1] (not clamped into the image)
};

__device__ __forceinline__ Taps make_taps(float cx, float cy, int Wimg, int Himg)
{
    float gx = cx * 2.0f - 1.0f;
    float gy = cy * 2.0f - 1.0f;
    float x = (gx + 1.0f) * ((float)(Wimg - 1) * 0.5f);
    float y = (gy + 1.0f) * ((float)(Himg - 1) * 0.5f);
    float x0f = floorf(x), y0f = floorf(y);
    float fx = x - x0f, fy = y - y0f;
    x0f = fminf(fmaxf(x0f, -2.0f), (float)Wimg + 1.0f);   // NaN -> -2 (outside)
    y0f = fminf(fmaxf(y0f, -2.0f), (float)Himg + 1.0f);
    int x0 = (int)x0f, y0 = (int)y0f;
    int x1 = x0 + 1, y1 = y0 + 1;
    bool vx0 = (x0 >= 0) & (x0 < Wimg), vx1 = (x1 >= 0) & (x1 < Wimg);
    bool vy0 = (y0 >= 0) & (y0 < Himg), vy1 = (y1 >= 0) & (y1 < Himg);
    int cx0 = min(max(x0, 0), Wimg - 1), cx1 = min(max(x1, 0), Wimg - 1);
    int cy0 = min(max(y0, 0), Himg - 1), cy1 = min(max(y1, 0), Himg - 1);
    float wx0 = 1.0f - fx, wy0 = 1.0f - fy;
    Taps t;
    t.w[0] = (vx0 & vy0) ? wx0 * wy0 : 0.0f;
    t.w[1] = (vx1 & vy0) ? fx * wy0 : 0.0f;
    t.w[2] = (vx0 & vy1) ? wx0 * fy : 0.0f;
    t.w[3] = (vx1 & vy1) ? fx * fy : 0.0f;
    t.pix[0] = cy0 * Wimg + cx0;
    t.pix[1] = cy0 * Wimg + cx1;
    t.pix[2] = cy1 * Wimg + cx0;
    t.pix[3] = cy1 * Wimg + cx1;
    t.x0 = x0;
    t.y0 = y0;
    return t;
}

// Derivatives of the four masked weights of make_taps by the NORMALISED coordinates: with the tap order
// 00, 01, 10, 11 and x_pix = x*(W-1), y_pix = y*(Himg-1),
//   d w/dx = (W-1)    * [-(1-fy), (1-fy), -fy, fy]      d w/dy = (Himg-1) * [-(1-fx), -fx, (1-fx), fx]
// each zeroed for a tap outside the image (that tap contributes nothing, so it has no gradient
// either: the rule of ATen's bilinear grid_sampler backward, which ops/torch.py:14-15 differentiates
// through). floor() makes the sample piecewise smooth; on a cell border this is the one-sided
// derivative of the cell floor() picks, as in ATen.
struct TapGrads { float gx[4], gy[4]; };

__device__ __forceinline__ TapGrads make_tap_grads(float cx, float cy, int Wimg, int Himg)
{
    float gxn = cx * 2.0f - 1.0f;
    float gyn = cy * 2.0f - 1.0f;
    float x = (gxn + 1.0f) * ((float)(Wimg - 1) * 0.5f);
    float y = (gyn + 1.0f) * ((float)(Himg - 1) * 0.5f);
    float x0f = floorf(x), y0f = floorf(y);
    float fx = x - x0f, fy = y - y0f;
    x0f = fminf(fmaxf(x0f, -2.0f), (float)Wimg + 1.0f);
    y0f = fminf(fmaxf(y0f, -2.0f), (float)Himg + 1.0f);
    int x0 = (int)x0f, y0 = (int)y0f;
    int x1 = x0 + 1, y1 = y0 + 1;
    bool vx0 = (x0 >= 0) & (x0 < Wimg), vx1 = (x1 >= 0) & (x1 < Wimg);
    bool vy0 = (y0 >= 0) & (y0 < Himg), vy1 = (y1 >= 0) & (y1 < Himg);
    bool fin = (x == x) & (y == y);                       // NaN coordinates: no taps, no gradient
    const float sx = (float)(Wimg - 1), sy = (float)(Himg - 1);
    const bool m[4] = { vx0 && vy0 && fin, vx1 && vy0 && fin, vx0 && vy1 && fin, vx1 && vy1 && fin };
    const float ax[4] = { -(1.0f - fy), 1.0f - fy, -fy, fy };
    const float ay[4] = { -(1.0f - fx), -fx, 1.0f - fx, fx };
    TapGrads t;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        t.gx[i] = m[i] ? sx * ax[i] : 0.0f;
        t.gy[i] = m[i] ? sy * ay[i] : 0.0f;
    }
    return t;
}

// ------------------------------------------------------------------ clearing buffers
// Up to four 16-byte aligned float buffers cleared by all threads of a launch (sizes in floats; unused
// slots have size 0).
struct ZeroJob { float *p[4]; size_t n[4]; };

__device__ __forceinline__ void zero_buffers(const ZeroJob &job)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const size_t n4 = job.n[k] / 4;
        float4 *p4 = reinterpret_cast<float4 *>(job.p[k]);
        for (size_t i = first; i < n4; i += stride) p4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (size_t i = 4 * n4 + first; i < job.n[k]; i += stride) job.p[k][i] = 0.f;
    }
}

// ------------------------------------------------------------------ wave-level helpers
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}

// Sum over aligned groups of G consecutive lanes (G a power of two <= 64); every
// lane of the group ends up with the group's sum.
template <int G>
__device__ __forceinline__ float group_sum(float x)
{
    if constexpr (G >= 2) x += dpp_f32<0xB1>(x);    // quad_perm [1,0,3,2]
    if constexpr (G >= 4) x += dpp_f32<0x4E>(x);    // quad_perm [2,3,0,1]
    if constexpr (G >= 8) x += dpp_f32<0x141>(x);   // row_half_mirror
    if constexpr (G >= 16) x += dpp_f32<0x140>(x);  // row_mirror
    if constexpr (G >= 32)                            // ds_swizzle, bit mode: lane ^ 16 within each half-wave
        x += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(x), 0x401F));
    if constexpr (G >= 64) x += __shfl_xor(x, 32, kWave);
    return x;
}

// ------------------------------------------------------------------ 4x4 block matrix instructions
// gfx950 has matrix instructions that treat a wave as 16 independent blocks of 4 lanes. Measured here, one of
// them takes 10-11 clocks of the SIMD where a vector multiply-add, a packed dot product or a byte permute takes
// 4.6, and cannot overlap with vector instructions of the same SIMD, but does the work of four (4x4x1) or
// sixteen (4x4x4) multiply-adds per lane: used as a wide multiply-add, not as a GEMM (every sample has its
// own operands).
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

// v_mfma_f32_4x4x1_16b_f32: for every block b of four lanes, acc(lane 4b+j)[i] += a(lane 4b+i) * x(lane 4b+j),
// i, j = 0..3: a 4x4 outer product per block. Lane 4b+i supplies row coefficient i, every lane its own x.
__device__ __forceinline__ floatx4 block_outer_fma(float a, float x, floatx4 acc)
{
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, x, acc, 0, 0, 0);
}

// 16-bit storage, at least four lanes per slot: the weighted sum of four rows on the 4x4x4 block matrix
// instruction. For every block of four lanes it computes C[i][j] += sum_k A[i][k] * B[k][j]: k runs over the
// four rows (pixels of a unit, or taps of a sample), j over the block's lanes, each with its own
// elements of those rows, and the two rows of A that are used are the high and the low part of the four
// coefficients (each a 16-bit float; together 16 bits of mantissa), so that acc[e][0] + acc[e][1] is the sum
// with coefficients good to 2^-16. Lane 4b+i supplies row i of A: `coef` is this lane's row (the high parts
// in lanes 4b, the low parts in lanes 4b+1, zero elsewhere). The rows come as packed pairs, which two byte
// permutes per pair of rows turn into "four rows' values of one element". FIRST: acc is taken as 0 (the
// instruction's inline constant; saves clearing 4 * DC registers before the first of a run of calls).
template <typename S, int DC, bool FIRST = false>
__device__ __forceinline__ void block_blend4(const uint32_t (&r)[4][DC / 2], shortx4 coef, floatx4 (&acc)[DC])
{
    if constexpr (FIRST) {
#pragma unroll
        for (int e = 0; e < DC; ++e) acc[e] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < DC / 2; ++i) {
        const uint32_t lo01 = __builtin_amdgcn_perm(r[1][i], r[0][i], 0x05040100u);
        const uint32_t lo23 = __builtin_amdgcn_perm(r[3][i], r[2][i], 0x05040100u);
        const uint32_t hi01 = __builtin_amdgcn_perm(r[1][i], r[0][i], 0x07060302u);
        const uint32_t hi23 = __builtin_amdgcn_perm(r[3][i], r[2][i], 0x07060302u);
        const uint2 be = make_uint2(lo01, lo23), bo = make_uint2(hi01, hi23);
        if constexpr (S::kBf16) {
            acc[2 * i] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(coef, __builtin_bit_cast(shortx4, be), acc[2 * i], 0, 0, 0);
            acc[2 * i + 1] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(coef, __builtin_bit_cast(shortx4, bo), acc[2 * i + 1], 0, 0, 0);
        } else {
            typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
            acc[2 * i] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, coef), __builtin_bit_cast(halfx4, be), acc[2 * i], 0, 0, 0);
            acc[2 * i + 1] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, coef), __builtin_bit_cast(halfx4, bo), acc[2 * i + 1], 0, 0, 0);
        }
    }
}

// Four fp32 coefficients as the block matrix instruction's rows: .x, .y = the high parts (storage type, by
// truncation for bf16 / rounding for fp16) as four packed 16-bit floats, .z, .w = the same of the remainders.
template <typename S>
__device__ __forceinline__ uint4 split_coefficients(float c0, float c1, float c2, float c3)
{
    if constexpr (S::kBf16) {
        const uint32_t u0 = __float_as_uint(c0), u1 = __float_as_uint(c1), u2 = __float_as_uint(c2), u3 = __float_as_uint(c3);
        const float l0 = c0 - __uint_as_float(u0 & 0xffff0000u), l1 = c1 - __uint_as_float(u1 & 0xffff0000u);
        const float l2 = c2 - __uint_as_float(u2 & 0xffff0000u), l3 = c3 - __uint_as_float(u3 & 0xffff0000u);
        return make_uint4(__builtin_amdgcn_perm(u1, u0, 0x07060302u), __builtin_amdgcn_perm(u3, u2, 0x07060302u),
                          __builtin_amdgcn_perm(__float_as_uint(l1), __float_as_uint(l0), 0x07060302u),
                          __builtin_amdgcn_perm(__float_as_uint(l3), __float_as_uint(l2), 0x07060302u));
    } else {
        union { uint32_t u; _Float16 h[2]; } a, b, c, d;
        a.h[0] = (_Float16)c0; a.h[1] = (_Float16)c1; b.h[0] = (_Float16)c2; b.h[1] = (_Float16)c3;
        c.h[0] = (_Float16)(c0 - (float)a.h[0]); c.h[1] = (_Float16)(c1 - (float)a.h[1]);
        d.h[0] = (_Float16)(c2 - (float)b.h[0]); d.h[1] = (_Float16)(c3 - (float)b.h[1]);
        return make_uint4(a.u, b.u, c.u, d.u);
    }
}

__device__ __forceinline__ uint4 lane_offsets(const uint4 &e, unsigned lane_byte)
{
    return make_uint4(e.x + lane_byte, e.y + lane_byte, e.z + lane_byte, e.w + lane_byte);
}

// The same with two coefficient operands (the high and the low parts of four rows of coefficients, see
// split_coefficients): acc[e][i] += sum_k (hi[i][k] + lo[i][k]) * r[k][e], all four rows i in use. The byte
// permutes are done once for both.
template <typename S, int DC>
__device__ __forceinline__ void block_blend4_pair(const uint32_t (&r)[4][DC / 2], shortx4 hi, shortx4 lo, floatx4 (&acc)[DC])
{
#pragma unroll
    for (int i = 0; i < DC / 2; ++i) {
        const uint32_t lo01 = __builtin_amdgcn_perm(r[1][i], r[0][i], 0x05040100u);
        const uint32_t lo23 = __builtin_amdgcn_perm(r[3][i], r[2][i], 0x05040100u);
        const uint32_t hi01 = __builtin_amdgcn_perm(r[1][i], r[0][i], 0x07060302u);
        const uint32_t hi23 = __builtin_amdgcn_perm(r[3][i], r[2][i], 0x07060302u);
        const uint2 be = make_uint2(lo01, lo23), bo = make_uint2(hi01, hi23);
        if constexpr (S::kBf16) {
            acc[2 * i] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(hi, __builtin_bit_cast(shortx4, be), acc[2 * i], 0, 0, 0);
            acc[2 * i + 1] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(hi, __builtin_bit_cast(shortx4, bo), acc[2 * i + 1], 0, 0, 0);
            acc[2 * i] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(lo, __builtin_bit_cast(shortx4, be), acc[2 * i], 0, 0, 0);
            acc[2 * i + 1] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(lo, __builtin_bit_cast(shortx4, bo), acc[2 * i + 1], 0, 0, 0);
        } else {
            typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
            acc[2 * i] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, hi), __builtin_bit_cast(halfx4, be), acc[2 * i], 0, 0, 0);
            acc[2 * i + 1] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, hi), __builtin_bit_cast(halfx4, bo), acc[2 * i + 1], 0, 0, 0);
            acc[2 * i] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, lo), __builtin_bit_cast(halfx4, be), acc[2 * i], 0, 0, 0);
            acc[2 * i + 1] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, lo), __builtin_bit_cast(halfx4, bo), acc[2 * i + 1], 0, 0, 0);
        }
    }
}

// ------------------------------------------------------------------ reductions over the whole wave
// Every lane ends up with the result. Five steps stay in the vector ALU (DPP / swizzle), the last is a shuffle.
template <typename T, typename Op>
__device__ __forceinline__ T wave_all(T x, Op op)
{
    static_assert(sizeof(T) == 4, "32-bit values");
    auto dpp = [](T v, auto ctrl) {
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value, 0xf, 0xf, false));
    };
    x = op(x, dpp(x, std::integral_constant<int, 0xB1>{}));      // quad_perm [1,0,3,2]
    x = op(x, dpp(x, std::integral_constant<int, 0x4E>{}));      // quad_perm [2,3,0,1]
    x = op(x, dpp(x, std::integral_constant<int, 0x141>{}));     // row_half_mirror
    x = op(x, dpp(x, std::integral_constant<int, 0x140>{}));     // row_mirror
    x = op(x, __builtin_bit_cast(T, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), 0x401F)));   // lane ^ 16
    x = op(x, __builtin_bit_cast(T, __shfl_xor(__builtin_bit_cast(int, x), 32, kWave)));
    return x;
}
__device__ __forceinline__ float wave_max(float x) { return wave_all(x, [](float a, float b) { return fmaxf(a, b); }); }
__device__ __forceinline__ float wave_sum(float x) { return wave_all(x, [](float a, float b) { return a + b; }); }
// two unsigned 16-bit fields per word, minimum taken field by field (one packed 16-bit minimum per step)
__device__ __forceinline__ uint32_t wave_min_u16x2(uint32_t x)
{
    typedef unsigned short dsdpa_u16x2 __attribute__((ext_vector_type(2)));
    return wave_all(x, [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(dsdpa_u16x2, a),
                                                                        __builtin_bit_cast(dsdpa_u16x2, b)));
    });
}

// Reduce-scatter steps on the lane-swap instructions of gfx950. swap_add_32(x, y): lanes 0..31 get x summed
// over the wave's two halves (x[l] + x[l + 32]), lanes 32..63 get y summed the same way
// (v_permlane32_swap: rows 2, 3 of the first operand change places with rows 0, 1 of the second; a row is
// 16 lanes). swap_add_16(x, y): lanes with bit 16 clear get x[l] + x[l ^ 16], lanes with it set get y summed
// the same way (v_permlane16_swap: odd rows of the first operand change places with even rows of the second).
__device__ __forceinline__ float swap_add_32(float x, float y)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap_add_16(float x, float y)
{
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Orders this wave's LDS writes before its later LDS reads (and the reverse):
// waits for the wave's outstanding LDS traffic and stops the compiler from
// moving LDS accesses across. No workgroup barrier is involved.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Workgroups are dealt to the 8 XCDs round-robin by their linear id, and each
// XCD has its own L2. This maps the hardware block id to a logical one so that
// every XCD walks one contiguous range of logical ids (hence of (batch, head)
// pairs, whose K/V planes then stay in that XCD's L2). A bijection on [0, nb).
__device__ __forceinline__ int xcd_logical_block(int bid, int nb)
{
    int x = bid % kXcds, i = bid / kXcds;
    int qn = nb / kXcds, rn = nb % kXcds;
    return x * qn + min(x, rn) + i;
}

}  // namespace dsdpa
