/*
 * CPU oracle for deformable multi-view scaled-dot-product attention.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker the HIP kernels are
 * compared against; nothing that ships may call it. Only tests/, the smoke
 * check and the CPU-baseline leg of the benchmark load the library built
 * from it.
 *
 * It restates, as explicit scalar loops, what the reference computes with
 * library calls:
 *   forward   ops/torch.py:5-28   (grid_sample bilinear / zeros padding /
 *                                  align_corners=True, then a softmax over
 *                                  all views' samples jointly, then p @ v)
 *   backward  ops/triton.py:330-360 (which gradients exist and their
 *                                  formulas), ops/triton.py:464 (dq, dk, dv
 *                                  only)
 *
 * Layouts (row-major, contiguous):
 *   q, k, v, out, dout, dq, dk, dv : [B][V][H][L][D]   float, L = Himg*Wimg
 *   coords                         : [B][V][L][V][P][2] float, (x, y) in [0,1]
 *   lse                            : [B][V][H][L]       float, base-2
 *                                    log-sum-exp of sm_scale*log2(e)*(q.k~)
 *                                    (the reference's M, ops/triton.py:188)
 *
 * Inputs are read as float; every sum is carried in double so that the
 * oracle's own rounding is far below the 1e-4 / 1e-3 parity bars.
 *
 * What pins it (tests/test_oracle_*.py): the ATen library routine
 * grid_sample + softmax on random and out-of-bounds inputs, an independent
 * float64 brute force on tiny non-square shapes, closed forms (pixel-centre
 * coords reduce to plain scaled_dot_product_attention, constant V, zero
 * scale, everything out of bounds), softmax/gradient invariants, and for the
 * backward pass autograd through the library routine plus central finite
 * differences of the oracle's own forward.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DSDPA_LOG2E 1.4426950408889634
#define DSDPA_LN2 0.6931471805599453

typedef struct {
    int pix[4];   /* row*W + col of the 4 taps, -1 when the tap is outside the image */
    float w[4];   /* bilinear weight of each tap (kept even for outside taps) */
    float fx, fy; /* fractional position inside the cell, for the coordinate gradient */
} taps_t;

/*
 * One sample's four taps.
 * ops/torch.py:14 feeds grid*2-1 to grid_sample(align_corners=True); ATen
 * un-normalises that as ((g+1)/2)*(size-1) (GridSampler.h:27-31), so
 * x_pix = x*(W-1), y_pix = y*(Himg-1). coords[...,0] is x (column, WIDTH),
 * coords[...,1] is y (row, HEIGHT); flat pixel = row*W + col
 * (ops/torch.py:8 '(h w)'). Padding is zeros PER TAP (GridSampler.h:205-207):
 * a tap outside [0,W)x[0,Himg) contributes nothing, the others keep their
 * weight. The Triton kernel's whole-sample mask (ops/triton.py:129,135-136)
 * is NOT followed.
 */
static void sample_taps(float cx, float cy, int Wimg, int Himg, taps_t *t)
{
    float gx = cx * 2.0f - 1.0f;
    float gy = cy * 2.0f - 1.0f;
    float x = (gx + 1.0f) * ((float)(Wimg - 1) * 0.5f);
    float y = (gy + 1.0f) * ((float)(Himg - 1) * 0.5f);
    float x0f = floorf(x), y0f = floorf(y);
    float fx = x - x0f, fy = y - y0f;
    /* keep the int conversion defined for wild coordinates */
    if (x0f < -4.0f) x0f = -4.0f;
    if (y0f < -4.0f) y0f = -4.0f;
    if (x0f > (float)Wimg + 4.0f) x0f = (float)Wimg + 4.0f;
    if (y0f > (float)Himg + 4.0f) y0f = (float)Himg + 4.0f;
    int x0 = (int)x0f, y0 = (int)y0f;
    int xs[2] = { x0, x0 + 1 };
    int ys[2] = { y0, y0 + 1 };
    float wx[2] = { 1.0f - fx, fx };
    float wy[2] = { 1.0f - fy, fy };
    for (int j = 0; j < 2; ++j)
        for (int i = 0; i < 2; ++i) {
            int inb = xs[i] >= 0 && xs[i] < Wimg && ys[j] >= 0 && ys[j] < Himg;
            t->pix[j * 2 + i] = inb ? ys[j] * Wimg + xs[i] : -1;
            t->w[j * 2 + i] = wx[i] * wy[j];
        }
    t->fx = fx;
    t->fy = fy;
    /* NaN coordinates: comparisons above are false -> all taps dropped */
    if (!(x == x) || !(y == y))
        for (int i = 0; i < 4; ++i) t->pix[i] = -1;
}

/* Bilinear sample of one D-vector from a [L][D] plane (ops/torch.py:14-15). */
static void sample_vec(const float *plane, const taps_t *t, int D, double *dst)
{
    for (int d = 0; d < D; ++d) dst[d] = 0.0;
    for (int i = 0; i < 4; ++i) {
        if (t->pix[i] < 0) continue;
        const float *src = plane + (size_t)t->pix[i] * D;
        double w = (double)t->w[i];
        for (int d = 0; d < D; ++d) dst[d] += w * (double)src[d];
    }
}

/*
 * Forward (ops/torch.py:5-28). For every query row (b, s1, h, l) the N = V*P
 * samples are ordered view-major, n = s2*P + p (ops/torch.py:13-17
 * concatenates the per-view results along the sample axis). The softmax runs
 * over all N samples jointly, own view included (ops/torch.py:20-25), in
 * base 2 exactly like the reference: logits are sm_scale*log2(e)*(q.k~).
 * A sample whose four taps all fall outside has k~ = v~ = 0, logit 0, and
 * still sits in the denominator.
 */
int dsdpa_oracle_fwd(const float *q, const float *k, const float *v,
                     const float *coords, float *out, float *lse,
                     int B, int V, int H, int Himg, int Wimg, int D, int P,
                     float sm_scale)
{
    const int L = Himg * Wimg;
    const int N = V * P;
    const long rows = (long)B * V * H * L;
    const double qs = (double)sm_scale * DSDPA_LOG2E;
#pragma omp parallel
    {
        double *kt = (double *)malloc(sizeof(double) * D);
        double *vt = (double *)malloc(sizeof(double) * (size_t)N * D);
        double *s = (double *)malloc(sizeof(double) * N);
#pragma omp for schedule(static)
        for (long r = 0; r < rows; ++r) {
            int l = (int)(r % L);
            int h = (int)((r / L) % H);
            int s1 = (int)((r / ((long)L * H)) % V);
            int b = (int)(r / ((long)L * H * V));
            const float *qrow = q + (size_t)r * D;
            const float *crow = coords + ((((size_t)b * V + s1) * L + l) * V) * P * 2;
            double m = -INFINITY;
            for (int n = 0; n < N; ++n) {
                int s2 = n / P;
                taps_t t;
                sample_taps(crow[2 * n], crow[2 * n + 1], Wimg, Himg, &t);
                size_t plane = (((size_t)b * V + s2) * H + h) * (size_t)L * D;
                sample_vec(k + plane, &t, D, kt);
                sample_vec(v + plane, &t, D, vt + (size_t)n * D);
                double dot = 0.0;
                for (int d = 0; d < D; ++d) dot += (double)qrow[d] * kt[d];
                s[n] = dot * qs;
                if (s[n] > m) m = s[n];
            }
            double sum = 0.0;
            for (int n = 0; n < N; ++n) { s[n] = exp2(s[n] - m); sum += s[n]; }
            float *orow = out + (size_t)r * D;
            for (int d = 0; d < D; ++d) {
                double acc = 0.0;
                for (int n = 0; n < N; ++n) acc += s[n] * vt[(size_t)n * D + d];
                orow[d] = (float)(acc / sum);
            }
            if (lse) lse[r] = (float)(m + log2(sum));
        }
        free(kt); free(vt); free(s);
    }
    return 0;
}

/*
 * Backward (ops/triton.py:330-360, 464). With p_n the softmax weights,
 * delta = dout.out (ops/triton.py:197-215), dp_n = dout.v~_n,
 * ds_n = p_n*(dp_n - delta):
 *   dq            = sm_scale * sum_n ds_n * k~_n
 *   dK[tap pixel] += w_tap * sm_scale * ds_n * q     (inside-image taps only)
 *   dV[tap pixel] += w_tap * p_n * dout
 * p_n is recomputed from the row's own logits (not from a stored lse) so the
 * backward oracle does not inherit a forward rounding. W, H and sm_scale
 * get no gradient. Parallel over (b, h): each pair owns its dK/dV planes, so
 * there are no races and the result is deterministic.
 *
 * dcoords (may be NULL; [B][V][L][V][P][2] like coords): the gradient the
 * eager operator gets for free because grid_sample is differentiable in its
 * grid (ops/torch.py:14-15; the fused reference returns None there,
 * ops/triton.py:464). With g_t = sm_scale*ds_n*(q.K_t) + p_n*(dout.V_t) for
 * the taps t = nw, ne, sw, se that lie inside the image (0 for the others)
 * ATen's bilinear backward (GridSampler.cpp, grid_sampler_2d_backward) gives
 *   dL/dx_pix = (1-fy)*(g_ne - g_nw) + fy*(g_se - g_sw)
 *   dL/dy_pix = (1-fx)*(g_sw - g_nw) + fx*(g_se - g_ne)
 * and x_pix = x*(W-1), y_pix = y*(Himg-1), summed over the H heads that
 * share the coordinates (double accumulation, atomic across threads).
 */
int dsdpa_oracle_bwd(const float *q, const float *k, const float *v,
                     const float *coords, const float *dout,
                     float *dq, float *dk, float *dv, float *dcoords,
                     int B, int V, int H, int Himg, int Wimg, int D, int P,
                     float sm_scale)
{
    const int L = Himg * Wimg;
    const int N = V * P;
    const size_t total = (size_t)B * V * H * L * D;
    const double qs = (double)sm_scale * DSDPA_LOG2E;
    double *dk64 = (double *)calloc(total, sizeof(double));
    double *dv64 = (double *)calloc(total, sizeof(double));
    const size_t ncoord = (size_t)B * V * L * V * P * 2;
    double *dc64 = dcoords ? (double *)calloc(ncoord, sizeof(double)) : NULL;
    if (!dk64 || !dv64 || (dcoords && !dc64)) { free(dk64); free(dv64); free(dc64); return 1; }
#pragma omp parallel
    {
        double *kt = (double *)malloc(sizeof(double) * (size_t)N * D);
        double *vt = (double *)malloc(sizeof(double) * (size_t)N * D);
        double *s = (double *)malloc(sizeof(double) * N);
        taps_t *tp = (taps_t *)malloc(sizeof(taps_t) * N);
        double *dqa = (double *)malloc(sizeof(double) * D);
#pragma omp for schedule(dynamic, 1)
        for (int bh = 0; bh < B * H; ++bh) {
            int b = bh / H, h = bh % H;
            for (int s1 = 0; s1 < V; ++s1)
                for (int l = 0; l < L; ++l) {
                    size_t r = (((size_t)b * V + s1) * H + h) * L + l;
                    const float *qrow = q + r * D;
                    const float *dorow = dout + r * D;
                    const float *crow = coords + ((((size_t)b * V + s1) * L + l) * V) * P * 2;
                    double m = -INFINITY;
                    for (int n = 0; n < N; ++n) {
                        int s2 = n / P;
                        sample_taps(crow[2 * n], crow[2 * n + 1], Wimg, Himg, &tp[n]);
                        size_t plane = (((size_t)b * V + s2) * H + h) * (size_t)L * D;
                        sample_vec(k + plane, &tp[n], D, kt + (size_t)n * D);
                        sample_vec(v + plane, &tp[n], D, vt + (size_t)n * D);
                        double dot = 0.0;
                        for (int d = 0; d < D; ++d) dot += (double)qrow[d] * kt[(size_t)n * D + d];
                        s[n] = dot * qs;
                        if (s[n] > m) m = s[n];
                    }
                    double sum = 0.0;
                    for (int n = 0; n < N; ++n) { s[n] = exp2(s[n] - m); sum += s[n]; }
                    /* delta = dout . out, with out rebuilt from p and v~ */
                    double delta = 0.0;
                    for (int n = 0; n < N; ++n) {
                        s[n] /= sum;
                        double dp = 0.0;
                        for (int d = 0; d < D; ++d) dp += (double)dorow[d] * vt[(size_t)n * D + d];
                        delta += s[n] * dp;
                    }
                    for (int d = 0; d < D; ++d) dqa[d] = 0.0;
                    for (int n = 0; n < N; ++n) {
                        int s2 = n / P;
                        double p = s[n];
                        double dp = 0.0;
                        for (int d = 0; d < D; ++d) dp += (double)dorow[d] * vt[(size_t)n * D + d];
                        double ds = p * (dp - delta);
                        for (int d = 0; d < D; ++d) dqa[d] += ds * kt[(size_t)n * D + d];
                        size_t plane = (((size_t)b * V + s2) * H + h) * (size_t)L * D;
                        if (dc64) {
                            double g[4] = { 0.0, 0.0, 0.0, 0.0 };
                            for (int i = 0; i < 4; ++i) {
                                if (tp[n].pix[i] < 0) continue;
                                const float *kp = k + plane + (size_t)tp[n].pix[i] * D;
                                const float *vp = v + plane + (size_t)tp[n].pix[i] * D;
                                double qk = 0.0, dov = 0.0;
                                for (int d = 0; d < D; ++d) {
                                    qk += (double)qrow[d] * (double)kp[d];
                                    dov += (double)dorow[d] * (double)vp[d];
                                }
                                g[i] = (double)sm_scale * ds * qk + p * dov;
                            }
                            double fx = (double)tp[n].fx, fy = (double)tp[n].fy;
                            double gx = (1.0 - fy) * (g[1] - g[0]) + fy * (g[3] - g[2]);
                            double gy = (1.0 - fx) * (g[2] - g[0]) + fx * (g[3] - g[1]);
                            size_t ci = (size_t)(crow - coords) + 2 * (size_t)n;
                            double ax = gx * (double)(Wimg - 1), ay = gy * (double)(Himg - 1);
#pragma omp atomic
                            dc64[ci] += ax;
#pragma omp atomic
                            dc64[ci + 1] += ay;
                        }
                        for (int i = 0; i < 4; ++i) {
                            if (tp[n].pix[i] < 0) continue;
                            double w = (double)tp[n].w[i];
                            double *dkp = dk64 + plane + (size_t)tp[n].pix[i] * D;
                            double *dvp = dv64 + plane + (size_t)tp[n].pix[i] * D;
                            double ck = w * ds * (double)sm_scale;
                            double cv = w * p;
                            for (int d = 0; d < D; ++d) {
                                dkp[d] += ck * (double)qrow[d];
                                dvp[d] += cv * (double)dorow[d];
                            }
                        }
                    }
                    for (int d = 0; d < D; ++d) dq[r * D + d] = (float)(dqa[d] * (double)sm_scale);
                }
        }
        free(kt); free(vt); free(s); free(tp); free(dqa);
    }
    for (size_t i = 0; i < total; ++i) { dk[i] = (float)dk64[i]; dv[i] = (float)dv64[i]; }
    if (dc64) for (size_t i = 0; i < ncoord; ++i) dcoords[i] = (float)dc64[i];
    free(dk64); free(dv64); free(dc64);
    return 0;
}

/* Taps of one coordinate pair, exposed so tests can pin the sampling rule on its own. */
void dsdpa_oracle_taps(float cx, float cy, int Wimg, int Himg, int *pix4, float *w4)
{
    taps_t t;
    sample_taps(cx, cy, Wimg, Himg, &t);
    for (int i = 0; i < 4; ++i) { pix4[i] = t.pix[i]; w4[i] = t.w[i]; }
}
