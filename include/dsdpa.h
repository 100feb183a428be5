/*
 * dsdpa.h -- C ABI of the MI355X (gfx950) fused deformable multi-view
 * scaled-dot-product attention library (libdsdpa.so).
 *
 * The reference is pure Python: its operator boundary is the autograd
 * function `_fused_deform_sdpa` (ops/triton.py:377-466), which launches the
 * Triton kernels `_fwd_kernel` (ops/triton.py:27-194), `_bwd_preprocess`
 * (ops/triton.py:197-215) and `_bwd_kernel` (ops/triton.py:219-365). It has no
 * FFI of its own; the entry points below are what a binding for that path
 * would call instead of those three launches.
 *
 * Conventions
 *   - plain pointers and sizes only; every pointer is DEVICE memory owned by
 *     the caller; nothing is allocated or freed by the library (scratch
 *     memory comes in as the `workspace` arguments);
 *   - tensors are row-major:
 *         q, k, v, out, dout, dq, dk, dv : [B][V][H][L][D],  L = Himg*Wimg, contiguous -- except that the
 *                  inputs q, k, v may be strided over (batch, view, head, pixel), see `strides` below
 *         coords : [B][V][L][V][P][2] float32, (x, y) normalised to [0, 1],
 *                  x along WIDTH (columns), y along HEIGHT (rows); shared by
 *                  all heads (ops/torch.py:10, ops/triton.py:51)
 *         lse    : [B][V][H][L] float32, base-2 log-sum-exp of
 *                  sm_scale*log2(e)*(q.k~) per query row (the reference's
 *                  `M`, ops/triton.py:187-190)
 *   - coordinates are passed NORMALISED; the un-normalisation
 *     x_pix = x*(W-1), y_pix = y*(Himg-1) (ops/triton.py:381-383) is done
 *     inside the kernels, and out-of-image taps follow the eager reference's
 *     per-tap zero padding (ops/torch.py:14-15), not ops/triton.py:129;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     the call returns without synchronising, and everything it enqueues is
 *     ordered after what `stream` held before the call and before what is
 *     enqueued on `stream` after it (the backward forks part of its work onto a
 *     second stream of the library's and joins it again, see
 *     DSDPA_FLAG_SINGLE_STREAM; a capture of `stream` records both);
 *   - `strides` (a HOST pointer, read during the call) is NULL when q, k and v are contiguous, or holds 8
 *     element strides: q's over (batch, view, head, pixel), then those shared by k and v. The head dimension
 *     itself must be contiguous and every row start a multiple of 16 bytes (DSDPA_ERR_BAD_STRIDES). The
 *     reference's forward takes the strides of q, k, v (ops/triton.py:396-405); its backward asserts that
 *     they are equal (ops/triton.py:425-426), which is not required here. A permuted projection output
 *     (B, V, L, H, D) -> (B, V, H, L, D) is read in place, without a copy;
 *   - D (head dim) must be one of 16, 32, 64, 128, 256 (ops/triton.py:386);
 *   - every entry point returns 0 on success or a DSDPA_ERR_* code, never
 *     throws, and is re-entrant; the only process-wide state is the kernel-path
 *     selector (dsdpa_set_path) and the optional kernel timer, the only
 *     per-thread state the backward's second stream (one stream and two events
 *     per host thread and device, created by the first backward call there
 *     and kept until the process ends).
 */
#ifndef DSDPA_H
#define DSDPA_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    DSDPA_OK = 0,
    DSDPA_ERR_NULL_POINTER = 1,   /* a required pointer is NULL                           */
    DSDPA_ERR_BAD_SHAPE = 2,      /* a dimension is < 1                                   */
    DSDPA_ERR_HEAD_DIM = 3,       /* D not in {16,32,64,128,256} (ops/triton.py:386)      */
    DSDPA_ERR_TOO_LARGE = 4,      /* a per-batch slab V*H*L*D exceeds 2^30 elements or
                                     rows exceed 2^31-1                                   */
    DSDPA_ERR_HIP = 5,            /* a HIP launch failed; see dsdpa_last_hip_error()      */
    DSDPA_ERR_DTYPE = 6,          /* unknown dtype code                                   */
    DSDPA_ERR_UNSUPPORTED = 7,    /* unknown flag bit, or DSDPA_FLAG_DETERMINISTIC with dcoords */
    DSDPA_ERR_SCRATCH = 8,        /* dsdpa_fwd_noalloc: the shape needs more than DSDPA_NOALLOC_SCRATCH_BYTES */
    DSDPA_ERR_BAD_STRIDES = 9     /* strides: head dimension not contiguous, or a row start not 16-byte aligned */
};

/* Storage types (accumulation is always fp32). Mirrors the reference's dtype
 * modes, ops/triton.py:367-375: fp32 = mode 0, fp16/bf16 = mode 1. */
enum { DSDPA_F32 = 0, DSDPA_BF16 = 1, DSDPA_F16 = 2 };

/*
 * Forward: replaces the `_fwd_kernel[grid](...)` launch, ops/triton.py:396-411,
 * including the coords clone/scale (:381-383) and the zero-fill of `o` (:389).
 * Writes out (storage dtype) and lse (fp32).
 *
 * `workspace` must hold dsdpa_fwd_workspace_bytes(...) bytes (256-byte aligned; may be NULL when that is
 * 0). It is scratch for the duration of the call on `stream`. Shapes whose K and V planes fit in LDS: a
 * table of the bilinear weights and tap addresses of every coordinate pair, computed once from coords and
 * shared by all H heads (the reference recomputes them per head inside `_fwd_kernel`,
 * ops/triton.py:118-140). 16-bit storage with D = 64 or 128, P >= 64 and larger planes: one byte per
 * (batch, head, query view, 16 consecutive queries), by which the kernel that works on tiles of 16 queries
 * tells the per-query kernel launched behind it which tiles are left to do.
 */
int dsdpa_fwd_f32(const float *q, const float *k, const float *v, const float *coords,
                  float *out, float *lse, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P,
                  float sm_scale, const long long *strides, void *stream);
int dsdpa_fwd_bf16(const void *q, const void *k, const void *v, const float *coords,
                   void *out, float *lse, void *workspace,
                   int B, int V, int H, int Himg, int Wimg, int D, int P,
                   float sm_scale, const long long *strides, void *stream);
int dsdpa_fwd_f16(const void *q, const void *k, const void *v, const float *coords,
                  void *out, float *lse, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P,
                  float sm_scale, const long long *strides, void *stream);

/*
 * Forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same computation and results
 * as dsdpa_fwd_{f32,bf16,f16} (`dtype` = DSDPA_F32 / DSDPA_BF16 / DSDPA_F16 selects which), but the
 * workspace is not an argument: it is a buffer of DSDPA_NOALLOC_SCRATCH_BYTES built into the library, one
 * copy per GPU, held until the process ends. The call allocates and frees nothing. A shape whose
 * dsdpa_fwd_workspace_bytes() exceeds the buffer is refused with DSDPA_ERR_SCRATCH before anything is
 * launched (shapes that need no workspace always pass; where only the tile flags of the 16-query kernel do
 * not fit, the per-query kernel does all the work instead). All calls on one GPU share that GPU's buffer: calls
 * that overlap on one GPU (two streams, two threads) race on it; calls on one stream, or otherwise ordered,
 * are fine, since every call rewrites all of the scratch it reads.
 */
#define DSDPA_NOALLOC_SCRATCH_BYTES (32u << 20)
int dsdpa_fwd_noalloc(int dtype, const void *q, const void *k, const void *v, const float *coords,
                      void *out, float *lse,
                      int B, int V, int H, int Himg, int Wimg, int D, int P,
                      float sm_scale, const long long *strides, void *stream);

/* Flags of the backward. The reference has one backward, with float atomics (ops/triton.py:345-360).
 * DSDPA_FLAG_DETERMINISTIC: bitwise reproducible dq, dk, dv: the samples of every bilinear cell are
 * added up in ascending order of their index and the per-cell sums reach dk/dv in four passes of plain
 * stores (cells of one row/column parity share no pixel) instead of float atomics. Needs a larger
 * workspace (pass the same flags to dsdpa_bwd_workspace_bytes) and cannot be combined with dcoords. */
enum { DSDPA_FLAG_DETERMINISTIC = 1, DSDPA_FLAG_COORDS_GRAD = 2, DSDPA_FLAG_SINGLE_STREAM = 4 };
/* DSDPA_FLAG_SINGLE_STREAM: enqueue every launch of the backward on `stream` itself. By default the dk/dv side
 * (clearing the accumulators, delta, the cell binning, the dk/dv kernel) runs on a second stream of the
 * library's beside the tap table and the dq kernel: neither side reads what the other writes, and the two
 * main kernels leave each other idle issue slots (C2: 7 % off the fwd+bwd step). Only on shapes whose K/V planes
 * fit in LDS, and only from 2^21 query*samples (B*V*H*L * V*P) up: below that the fork and join cost more host
 * time than the overlap saves. Same results either way. */
/* DSDPA_FLAG_COORDS_GRAD: the workspace has room for the coordinate gradient's part of the per-coordinate
 * table (16 more bytes per coordinate pair where the staged kernels run), so that a backward given dcoords
 * stays on the staged dq kernel. Pass the same flags to dsdpa_bwd_workspace_bytes and to dsdpa_bwd_*;
 * dcoords without the bit is computed by the slower gather dq kernel, the bit without dcoords does nothing. */

/*
 * Backward: replaces everything `_fused_deform_sdpa.backward` enqueues,
 * ops/triton.py:427-462: the zero-fills (:427-430), the scaled copy of K
 * (:431-432), `_bwd_preprocess` (:436-441), `_bwd_kernel` (:443-459) and the
 * fp32 -> storage casts of dk/dv (:461-462).
 *
 * dq, dk, dv are fully overwritten (no pre-zeroing by the caller needed).
 * `dcoords` may be NULL (the reference's behaviour: no gradient for coords, ops/triton.py:464). When it
 * is given (fp32, shaped like coords) it receives the gradient of the normalised coordinates summed over
 * the heads -- what the reference's eager operator gets by differentiating through grid_sample,
 * ops/torch.py:14-15 -- and is fully overwritten too (float atomics across heads: not deterministic
 * either); see DSDPA_FLAG_COORDS_GRAD.
 * `workspace` must hold dsdpa_bwd_workspace_bytes(...) bytes (256-byte aligned):
 * the per-row delta = dout.out (one float per query row, the reference's `delta`,
 * ops/triton.py:430), the per-(batch, key view) ordering of the samples by
 * bilinear cell (one u32 and the position inside the cell, 8 bytes, per coordinate pair, plus the cell
 * offsets; it depends on coords only and is shared by all heads) and, for bf16/fp16, the fp32 dk/dv
 * accumulators that are rounded to the storage type at the end (fp32: dk and dv
 * are themselves the accumulators), and the same per-coordinate table as the forward's -- or, on shapes
 * whose K/V planes do not fit in LDS, a buffer in which the dq kernel leaves the softmax weight and its
 * gradient (8 bytes per (query row, sample)) for the dk/dv kernel: the backward runs in groups of (batch,
 * head) pairs and the buffer holds one group's, at most 128 MiB whatever the shape. The workspace is therefore
 * O(N) + O(coords) + a constant: the reference's own temporaries (dk32, dv32, delta, ops/triton.py:427-432)
 * plus 12 to 32 bytes per coordinate pair, plus at most 128 MiB; nothing in it grows with (query rows) x
 * (samples) or with samples x D. Without
 * DSDPA_FLAG_DETERMINISTIC the accumulation order into dk/dv is not deterministic (float atomics,
 * as in the reference, ops/triton.py:345-360).
 */
int dsdpa_bwd_f32(const float *q, const float *k, const float *v, const float *coords,
                  const float *out, const float *lse, const float *dout,
                  float *dq, float *dk, float *dv, float *dcoords, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P,
                  float sm_scale, const long long *strides, unsigned flags, void *stream);
int dsdpa_bwd_bf16(const void *q, const void *k, const void *v, const float *coords,
                   const void *out, const float *lse, const void *dout,
                   void *dq, void *dk, void *dv, float *dcoords, void *workspace,
                   int B, int V, int H, int Himg, int Wimg, int D, int P,
                   float sm_scale, const long long *strides, unsigned flags, void *stream);
int dsdpa_bwd_f16(const void *q, const void *k, const void *v, const float *coords,
                  const void *out, const float *lse, const void *dout,
                  void *dq, void *dk, void *dv, float *dcoords, void *workspace,
                  int B, int V, int H, int Himg, int Wimg, int D, int P,
                  float sm_scale, const long long *strides, unsigned flags, void *stream);

/* Bytes of device workspace dsdpa_fwd_* needs for a storage dtype: 20 bytes per coordinate pair when the
 * K and V planes of one view fit in LDS (the staged kernels); else one byte per 16 queries of every
 * (batch, head, view) for 16-bit storage with D = 64 or 128 and P >= 64, else 0; 0 also if an argument is
 * invalid. No counterpart in the reference. */
size_t dsdpa_fwd_workspace_bytes(int dtype, int B, int V, int H, int Himg, int Wimg, int D, int P);

/* Bytes of device workspace dsdpa_bwd_* needs for a storage dtype (0 if an argument is invalid).
 * Counterpart of the reference's delta and dk32/dv32 temporaries, ops/triton.py:428-430. */
size_t dsdpa_bwd_workspace_bytes(int dtype, int B, int V, int H, int Himg, int Wimg, int D, int P,
                                 unsigned flags);

/* Human-readable text for a DSDPA_ERR_* code. */
const char *dsdpa_error_string(int code);

/* hipError_t (as int) of the most recent failed launch on the calling thread, 0 if none. */
int dsdpa_last_hip_error(void);

/* Library version: major*10000 + minor*100 + patch. */
int dsdpa_version(void);

/*
 * Kernel-path selection, for measurement and tests. `path` is one of
 * DSDPA_PATH_*; AUTO picks per shape. Returns the previous value, or -1 if
 * `path` is unknown. Process-wide; the reference's analogue is the autotune
 * table, ops/triton.py:10-25.
 */
/* Forward and backward-dq: AUTO and LDS stage each key view's K/V planes in LDS
 * when a plane pair fits (AUTO: unless there are at most 3 samples per view and 8
 * or more views, where staging costs more than it saves), GATHER always reads the
 * taps from global memory, one query at a time. AUTO alone lets the forward work on
 * tiles of 16 queries with the matrix instructions where the shape allows it
 * (16-bit storage, D = 64 or 128, P >= 64, planes too large for LDS), and lets the
 * forward and dq walk the planes through LDS 16 columns at a time (fp32 storage,
 * P = 16 or 32, images of up to 1024 pixels whose planes do not fit in LDS whole).
 * Backward dk/dv: AUTO = cell-binned register accumulation, LDS = tiles of the
 * plane accumulated in LDS with fp64 atomics, GATHER = global float atomics per
 * tap as in the reference (ops/triton.py:345-360). */
enum { DSDPA_PATH_AUTO = 0, DSDPA_PATH_GATHER = 1, DSDPA_PATH_LDS = 2 };
int dsdpa_set_path(int path);

/*
 * Kernel timer, for measurement (the reference times whole calls with
 * triton.testing.do_bench, benchmark.py:90). While enabled (process-wide),
 * every main forward / backward kernel launch carries a pair of HIP events on
 * the launch stream (attached to the kernel's own dispatch: its start and end
 * timestamps; a timed launch costs a few microseconds of GPU idle time).
 * dsdpa_timer_collect waits for the events, returns the summed kernel time and
 * the number of launches for `which` (0 = forward kernel, 1 = backward dk/dv
 * kernel, 2 = backward dq kernel, 3 = the three cell-binning launches taken
 * together, 4 = the launches that fill the per-coordinate table, one per
 * forward and one per backward call) and releases them.
 * dsdpa_timer_enable returns the previous state.
 */
int dsdpa_timer_enable(int on);
int dsdpa_timer_collect(int which, double *total_ms, int *launches);

#ifdef __cplusplus
}
#endif
#endif /* DSDPA_H */
