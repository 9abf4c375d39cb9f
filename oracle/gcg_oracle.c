/*
 * CPU oracle for the gated chunked causal convolution  y = C * conv(B * x, h).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared with (tests/, the smoke check, and the CPU-baseline leg of the
 * benchmark).  Nothing in the shipped package links, loads or calls it.
 *
 * It restates, as plain nested sums with double-precision accumulators, the
 * formulation the reference states through library calls:
 *
 *   forward   savanna/kernels/triton_src/cgcg/ref_fwd.py:82-136
 *             (gcg_fwd_ref_corrected: Bx = B*x; depthwise F.conv1d with
 *              padding hl-1, right-truncated, filter h.repeat_interleave(dg);
 *              cross-correlation, "no flip on the filter" ref_fwd.py:41;
 *              y = C * y2)
 *   backward  savanna/kernels/triton_src/cgcg/src/bwd.py:442-471
 *             (dC = dy*y2; dy2 = dy*C; conv1d_input / conv1d_weight with
 *              padding hl-1, groups d; dh = dh_grouped.reshape(g,dg,1,hl).sum(1);
 *              dB = dBx*x; dx = dBx*B)
 *
 * Layout (ref_fwd.py:82-101): x, B, C, y, y2, dy, dx, dB, dC are
 * (bs, L, g, dg) contiguous, channel fastest; h and dh are (g, 1, hl).
 * Tap hl-1 multiplies the current sample:
 *
 *   y2[b,t,c] = sum_{j=0}^{min(hl-1,t)} h[c/dg, hl-1-j] * u[b,t-j,c],  u = B*x
 *
 * Pinned by tests/test_oracle.py against F.conv1d (the library routine the
 * reference calls), closed forms (delta taps, all-ones inputs), a brute-force
 * Python loop on tiny shapes, finite differences / the adjoint identity for the
 * gradients, and the two-pass Toeplitz form
 * (gcg_two_pass_chunked_fwd / _bwd in oracle/gcg_ref.py).
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -shared -fPIC)
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX(b, t, c) ((((size_t)(b)) * (size_t)L + (size_t)(t)) * (size_t)d + (size_t)(c))

/* ---- float I/O, double accumulation --------------------------------------- */

/* Forward.  y2 and bx may be NULL.  When round_bx_bf16 is nonzero the pre-gate
 * product u is rounded to bfloat16 (round-to-nearest-even) before it enters the
 * sum, which is what a kernel that feeds bf16 matrix cores does
 * (fwd_kernels.py:703-715 in the reference does the same through tl.dot on the
 * input dtype). */
static float round_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7f800000u) == 0x7f800000u) return f; /* inf / nan unchanged */
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}

int gcg_oracle_fwd_f32(const float *x, const float *B, const float *C, const float *h,
                       float *y, float *y2, float *bx,
                       int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                       int32_t round_bx_bf16)
{
    if (bs < 0 || L < 0 || g <= 0 || dg <= 0 || hl <= 0) return -1;
    const int64_t d = (int64_t)g * dg;
    const int64_t ncol = bs * d;
#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < ncol; ++col) {
        const int64_t b = col / d, c = col % d;
        const float *hg = h + (size_t)(c / dg) * hl;
        for (int64_t t = 0; t < L; ++t) {
            double acc = 0.0;
            const int64_t jmax = (t < hl - 1) ? t : hl - 1;
            for (int64_t j = 0; j <= jmax; ++j) {
                float u = B[IDX(b, t - j, c)] * x[IDX(b, t - j, c)];
                if (round_bx_bf16) u = round_bf16(u);
                acc += (double)hg[hl - 1 - j] * (double)u;
            }
            const size_t o = IDX(b, t, c);
            if (y2) y2[o] = (float)acc;
            if (bx) {
                float u = B[o] * x[o];
                bx[o] = round_bx_bf16 ? round_bf16(u) : u;
            }
            y[o] = (float)((double)C[o] * acc);
        }
    }
    return 0;
}

/* Backward.  dh is (g, hl) float, overwritten.  All five outputs required. */
int gcg_oracle_bwd_f32(const float *dy, const float *x, const float *B, const float *C,
                       const float *h, float *dx, float *dB, float *dC, float *dh,
                       int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl)
{
    if (bs < 0 || L < 0 || g <= 0 || dg <= 0 || hl <= 0) return -1;
    const int64_t d = (int64_t)g * dg;
    const int64_t ncol = bs * d;
    double *dh_col = (double *)calloc((size_t)(ncol > 0 ? ncol : 1) * hl, sizeof(double));
    if (!dh_col) return -2;
#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < ncol; ++col) {
        const int64_t b = col / d, c = col % d;
        const float *hg = h + (size_t)(c / dg) * hl;
        double *dhc = dh_col + (size_t)col * hl;
        for (int64_t t = 0; t < L; ++t) {
            const size_t o = IDX(b, t, c);
            /* y2[t] for dC */
            double y2 = 0.0;
            const int64_t jmax = (t < hl - 1) ? t : hl - 1;
            for (int64_t j = 0; j <= jmax; ++j) {
                const size_t i = IDX(b, t - j, c);
                const double u = (double)B[i] * (double)x[i];
                y2 += (double)hg[hl - 1 - j] * u;
                /* dh[hl-1-j] += g2[t] * u[t-j]   (conv1d_weight) */
                dhc[hl - 1 - j] += (double)dy[o] * (double)C[o] * u;
            }
            dC[o] = (float)((double)dy[o] * y2);
            /* du[t] = sum_j h[hl-1-j] * g2[t+j]   (conv1d_input, anti-causal) */
            double du = 0.0;
            const int64_t kmax = (L - 1 - t < hl - 1) ? L - 1 - t : hl - 1;
            for (int64_t j = 0; j <= kmax; ++j) {
                const size_t i = IDX(b, t + j, c);
                du += (double)hg[hl - 1 - j] * (double)dy[i] * (double)C[i];
            }
            dx[o] = (float)(du * (double)B[o]);
            dB[o] = (float)(du * (double)x[o]);
        }
    }
    /* reduce over batch and the dg channels of each group, fixed order */
    for (int32_t gi = 0; gi < g; ++gi)
        for (int32_t k = 0; k < hl; ++k) {
            double s = 0.0;
            for (int64_t b = 0; b < bs; ++b)
                for (int32_t ci = 0; ci < dg; ++ci)
                    s += dh_col[((size_t)(b * d + (int64_t)gi * dg + ci)) * hl + k];
            dh[(size_t)gi * hl + k] = (float)s;
        }
    free(dh_col);
    return 0;
}

/* ---- Toeplitz factors of the two-pass form --------------------------------- */
/* T  (cs x cs): T[i,j]  = h[hl-1-(i-j)]      for 0 <= i-j < hl, else 0
 * Tc (cs x cs): Tc[i,j] = h[hl-1-(i+cs-j)]   for 0 <= i+cs-j < hl, else 0
 * for one filter h (hl taps), as built by toeplitz(h.flip(-1), cs) and
 * correction_toeplitz(h.flip(-1), cs) in savanna/kernels/triton_src/cgcg/utils.py:5-51. */
int gcg_oracle_toeplitz_f64(const double *h, int32_t hl, int32_t cs, double *T, double *Tc)
{
    if (hl <= 0 || cs <= 0) return -1;
    for (int32_t i = 0; i < cs; ++i)
        for (int32_t j = 0; j < cs; ++j) {
            const int32_t lag = i - j, lagc = i + cs - j;
            T[(size_t)i * cs + j] = (lag >= 0 && lag < hl) ? h[hl - 1 - lag] : 0.0;
            Tc[(size_t)i * cs + j] = (lagc >= 0 && lagc < hl) ? h[hl - 1 - lagc] : 0.0;
        }
    return 0;
}
