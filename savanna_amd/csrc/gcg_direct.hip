// Direct (vector-ALU) kernels: any filter length, any group width, any element type.
//
// The pre-gate product u = B*x of a (time x channel) tile plus its filter-length
// halo is staged once in LDS as fp32; each lane then owns one channel and 16
// consecutive time rows and walks the taps in blocks of 16, holding 16 taps and a
// 31-sample window in registers so that a block costs 47 LDS reads for 256 FMAs.
// This is the fallback for shapes the MFMA and register-window kernels do not take (filters
// longer than 128 taps, narrow or odd group widths, misaligned tensors).
#include "gcg_common.h"

namespace gcg {
namespace {

constexpr int TT = 64;   // time rows per tile
constexpr int CT = 64;   // channels per tile
constexpr int RB = 16;   // rows per lane
constexpr int LB = 16;   // taps per register block

template <typename T>
__device__ __forceinline__ float ld(const T *p, int64_t off) { return Elem<T>::load(p + off); }

// ---------------------------------------------------------------------------- forward
constexpr int FWD_PASS = 128;                   // taps per LDS pass
constexpr int FWD_ROWS = TT + FWD_PASS;         // 191 used

template <typename T>
__global__ __launch_bounds__(256) void direct_fwd_kernel(const T *__restrict__ x, const T *__restrict__ B,
                                                         const T *__restrict__ C, const T *__restrict__ h,
                                                         T *__restrict__ y, T *__restrict__ y2,
                                                         T *__restrict__ bx, Dims dm, int nct, int ntt)
{
    __shared__ float us[FWD_ROWS][CT];
    int64_t wg = blockIdx.x;
    const int ct = (int)(wg % nct); wg /= nct;
    const int64_t tt = wg % ntt;
    const int64_t b = wg / ntt;
    const int tid = threadIdx.x, cl = tid & 63, r0 = (tid >> 6) * RB;
    const int64_t c0 = (int64_t)ct * CT, c = c0 + cl, d = dm.d, L = dm.L;
    const bool cvalid = c < d;
    const int hl = dm.hl;
    const int64_t es = dm.es;   // element stride of x, B, C (3 when they are interleaved in one tensor)
    const int64_t pad = dm.planar ? 2 * dm.d : 0;   // planar features: the three lie side by side in rows of 3 * d
    const int64_t t0 = tt * TT;
    typedef typename Filt<T>::type FT;           // element type of the filter
    const FT *hg = (const FT *)h + (cvalid ? (c / dm.dg) : 0) * hl;

    float acc[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[r] = 0.f;

    for (int lag_lo = 0; lag_lo < hl; lag_lo += FWD_PASS) {
        const int nlag = min(FWD_PASS, hl - lag_lo);
        const int nlb = (nlag + LB - 1) / LB;
        const int nrows = TT + LB * nlb - 1;
        const int64_t base = t0 - lag_lo - (LB * nlb - 1);
        __syncthreads();
        for (int idx = tid; idx < nrows * CT; idx += 256) {
            const int row = idx >> 6, cc = idx & 63;
            const int64_t time = base + row;
            float v = 0.f;
            if (time >= 0 && time < L && c0 + cc < d) {
                const int64_t off = (b * L + time) * d + c0 + cc, ioff = off * es + (b * L + time) * pad;
                v = ld(B, ioff) * ld(x, ioff);
            }
            us[row][cc] = v;
        }
        __syncthreads();
        for (int lb = 0; lb < nlb; ++lb) {
            float hr[LB];
#pragma unroll
            for (int jj = 0; jj < LB; ++jj) {
                const int lag = lag_lo + LB * lb + jj;
                hr[jj] = (lag < hl && cvalid) ? ld(hg, hl - 1 - lag) : 0.f;
            }
            const int rbase = r0 + LB * (nlb - 1 - lb);
            float ur[RB + LB - 1];
#pragma unroll
            for (int k = 0; k < RB + LB - 1; ++k) ur[k] = us[rbase + k][cl];
#pragma unroll
            for (int r = 0; r < RB; ++r)
#pragma unroll
                for (int jj = 0; jj < LB; ++jj) acc[r] = fmaf(hr[jj], ur[r - jj + LB - 1], acc[r]);
        }
    }
    if (!cvalid) return;
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const int64_t t = t0 + r0 + r;
        if (t < L) {
            const int64_t o = (b * L + t) * d + c, io = o * es + (b * L + t) * pad;
            if (y2) Elem<T>::store(y2 + o, acc[r]);
            if (bx) Elem<T>::store(bx + o, ld(B, io) * ld(x, io));
            Elem<T>::store(y + o, ld(C, io) * acc[r]);
        }
    }
}

// --------------------------------------------------------------------------- backward
constexpr int BWD_PASS = 32;
constexpr int BWD_ROWS = TT + BWD_PASS;         // 95 used

__host__ __device__ inline int groups_per_tile(int dg)
{
    if (CT % dg == 0) return CT / dg;
    const int v = (CT - 1) / dg + 2;
    return v < CT ? v : CT;
}

template <typename T>
__global__ __launch_bounds__(256) void direct_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                         const T *__restrict__ B, const T *__restrict__ C,
                                                         const T *__restrict__ h, T *__restrict__ dx,
                                                         T *__restrict__ dB, T *__restrict__ dC,
                                                         float *__restrict__ ws, Dims dm, int nct, int ntt,
                                                         int nseg, int tiles_per_seg, int gpt)
{
    __shared__ float us[BWD_ROWS][CT];
    __shared__ float gs[BWD_ROWS][CT];
    __shared__ float lp[LB][256];
    __shared__ float lq[LB][CT];

    int64_t wg = blockIdx.x;
    const int ct = (int)(wg % nct); wg /= nct;
    const int seg = (int)(wg % nseg);
    const int64_t b = wg / nseg;
    const int tid = threadIdx.x, cl = tid & 63, r0 = (tid >> 6) * RB;
    const int64_t c0 = (int64_t)ct * CT, c = c0 + cl, d = dm.d, L = dm.L;
    const bool cvalid = c < d;
    const int hl = dm.hl, dg = dm.dg;
    const int64_t es = dm.es;   // element stride of x, B, C, dx, dB, dC
    const int64_t pad = dm.planar ? 2 * dm.d : 0;   // planar features and gradient: rows of 3 * d
    typedef typename Filt<T>::type FT;           // element type of the filter
    const FT *hg = (const FT *)h + (cvalid ? (c / dg) : 0) * hl;
    const int64_t g0 = c0 / dg;                                            // first group in this tile
    const int64_t clast = (c0 + CT < d ? c0 + CT : d) - 1;
    const int ngl = (int)(clast / dg - g0) + 1;                            // groups in this tile
    float *slot = ws + (size_t)blockIdx.x * gpt * hl;                      // this workgroup's dh partials

    for (int pair = tid; pair < LB * gpt; pair += 256) {
        const int jj = pair & 15, gl = pair >> 4;
        for (int lag = jj; lag < hl; lag += LB) slot[gl * hl + hl - 1 - lag] = 0.f;
    }

    const int64_t tt_lo = (int64_t)seg * tiles_per_seg;
    const int64_t tt_hi = (tt_lo + tiles_per_seg < ntt) ? tt_lo + tiles_per_seg : ntt;
    for (int64_t tt = tt_lo; tt < tt_hi; ++tt) {
        const int64_t t0 = tt * TT;
        float y2a[RB], dua[RB], gown[RB];
#pragma unroll
        for (int r = 0; r < RB; ++r) { y2a[r] = 0.f; dua[r] = 0.f; gown[r] = 0.f; }

        for (int lag_lo = 0; lag_lo < hl; lag_lo += BWD_PASS) {
            const int nlag = min(BWD_PASS, hl - lag_lo);
            const int nlb = (nlag + LB - 1) / LB;
            const int nrows = TT + LB * nlb - 1;
            const int64_t ubase = t0 - lag_lo - (LB * nlb - 1);
            const int64_t gbase = t0 + lag_lo;
            __syncthreads();
            for (int idx = tid; idx < nrows * CT; idx += 256) {
                const int row = idx >> 6, cc = idx & 63;
                const bool cok = c0 + cc < d;
                int64_t time = ubase + row;
                float v = 0.f;
                if (time >= 0 && time < L && cok) {
                    const int64_t off = (b * L + time) * d + c0 + cc, ioff = off * es + (b * L + time) * pad;
                    v = ld(B, ioff) * ld(x, ioff);
                }
                us[row][cc] = v;
                time = gbase + row;
                v = 0.f;
                if (time < L && cok) {
                    const int64_t off = (b * L + time) * d + c0 + cc, ioff = off * es + (b * L + time) * pad;
                    v = ld(dy, off) * ld(C, ioff);
                }
                gs[row][cc] = v;
            }
            __syncthreads();
            if (lag_lo == 0) {
#pragma unroll
                for (int r = 0; r < RB; ++r) gown[r] = gs[r0 + r][cl];
            }
            for (int lb = 0; lb < nlb; ++lb) {
                float hr[LB];
#pragma unroll
                for (int jj = 0; jj < LB; ++jj) {
                    const int lag = lag_lo + LB * lb + jj;
                    hr[jj] = (lag < hl && cvalid) ? ld(hg, hl - 1 - lag) : 0.f;
                }
                float ur[RB + LB - 1], gr[RB + LB - 1];
                const int urow = r0 + LB * (nlb - 1 - lb), grow = r0 + LB * lb;
#pragma unroll
                for (int k = 0; k < RB + LB - 1; ++k) { ur[k] = us[urow + k][cl]; gr[k] = gs[grow + k][cl]; }
                float dhp[LB];
#pragma unroll
                for (int jj = 0; jj < LB; ++jj) dhp[jj] = 0.f;
#pragma unroll
                for (int r = 0; r < RB; ++r)
#pragma unroll
                    for (int jj = 0; jj < LB; ++jj) {
                        y2a[r] = fmaf(hr[jj], ur[r - jj + LB - 1], y2a[r]);
                        dua[r] = fmaf(hr[jj], gr[r + jj], dua[r]);
                        dhp[jj] = fmaf(gown[r], ur[r - jj + LB - 1], dhp[jj]);
                    }
                // deterministic reduction of the 16 tap partials over the tile:
                // lanes -> rows-of-a-channel -> channels-of-a-group, always in the same order
#pragma unroll
                for (int jj = 0; jj < LB; ++jj) lp[jj][tid] = dhp[jj];
                __syncthreads();
                {
                    const int jj = tid >> 4, q = tid & 15;
#pragma unroll
                    for (int cc = 4 * q; cc < 4 * q + 4; ++cc)
                        lq[jj][cc] = (lp[jj][cc] + lp[jj][64 + cc]) + (lp[jj][128 + cc] + lp[jj][192 + cc]);
                }
                __syncthreads();
                for (int pair = tid; pair < LB * ngl; pair += 256) {
                    const int jj = pair & 15, gl = pair >> 4;
                    const int lag = lag_lo + LB * lb + jj;
                    if (lag < hl) {
                        int64_t lo = (g0 + gl) * dg, hi = lo + dg;
                        lo = (lo > c0 ? lo : c0) - c0;
                        hi = (hi < clast + 1 ? hi : clast + 1) - c0;
                        float s = 0.f;
                        for (int cc = (int)lo; cc < (int)hi; ++cc) s += lq[jj][cc];
                        slot[gl * hl + hl - 1 - lag] += s;
                    }
                }
            }
        }
        if (cvalid) {
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const int64_t t = t0 + r0 + r;
                if (t < L) {
                    const int64_t o = (b * L + t) * d + c, io = o * es + (b * L + t) * pad;
                    Elem<T>::store(dC + io, ld(dy, o) * y2a[r]);
                    Elem<T>::store(dx + io, dua[r] * ld(B, io));
                    Elem<T>::store(dB + io, dua[r] * ld(x, io));
                }
            }
        }
    }
}

// dh[grp,k] = sum over batch, time segments and the channel tiles that touch the group
template <typename T>
__global__ __launch_bounds__(256) void direct_dh_reduce_kernel(const float *__restrict__ ws, T *__restrict__ dh,
                                                               Dims dm, int nct, int nseg, int gpt)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)dm.g * dm.hl) return;
    const int64_t grp = i / dm.hl;
    const int k = (int)(i % dm.hl);
    const int64_t ct_lo = grp * dm.dg / CT, ct_hi = ((grp + 1) * dm.dg - 1) / CT;
    float s = 0.f;
    for (int64_t p = 0; p < dm.bs * nseg; ++p)
        for (int64_t ct = ct_lo; ct <= ct_hi; ++ct) {
            const int64_t gl = grp - ct * CT / dm.dg;
            s += ws[((size_t)(p * nct + ct) * gpt + gl) * dm.hl + k];
        }
    typedef typename Filt<T>::type FT;
    Elem<FT>::store((FT *)dh + i, s);
}

struct BwdPlan { int nct, ntt, nseg, tps, gpt; int64_t nwg; };

BwdPlan plan_bwd(const Dims &dm)
{
    BwdPlan p;
    p.nct = (int)((dm.d + CT - 1) / CT);
    p.ntt = (int)((dm.L + TT - 1) / TT);
    int64_t want = 4096 / (dm.bs * p.nct > 0 ? dm.bs * p.nct : 1);
    if (want < 1) want = 1;
    if (want > p.ntt) want = p.ntt;
    p.tps = (int)((p.ntt + want - 1) / want);
    p.nseg = (p.ntt + p.tps - 1) / p.tps;
    p.gpt = groups_per_tile(dm.dg);
    p.nwg = dm.bs * p.nseg * p.nct;
    return p;
}

template <typename T>
int fwd_t(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
          const Dims &dm, hipStream_t st)
{
    int e = 0;
    const int nct = (int)((dm.d + CT - 1) / CT), ntt = (int)((dm.L + TT - 1) / TT);
    const int64_t nwg = dm.bs * ntt * nct;
    if (nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    e = launch_plain(direct_fwd_kernel<T>, dim3((unsigned)nwg), dim3(256), st, (const T *)x, (const T *)B,
                       (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, nct, ntt);
    return e;
}

template <typename T>
int bwd_t(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
          void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    int e = 0;
    const BwdPlan p = plan_bwd(dm);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    e = launch_plain(direct_bwd_kernel<T>, dim3((unsigned)p.nwg), dim3(256), st, (const T *)dy,
                       (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)dx, (T *)dB, (T *)dC,
                       (float *)ws, dm, p.nct, p.ntt, p.nseg, p.tps, p.gpt);
    if (e) return e;
    const int64_t n = (int64_t)dm.g * dm.hl;
    e = launch_plain(direct_dh_reduce_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), st,
                       (const float *)ws, (T *)dh, dm, p.nct, p.nseg, p.gpt);
    return e;
}

} // namespace

int direct_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h, void *y,
                      void *y2, void *bx, const Dims &dm, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return fwd_t<float>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_BF16: return fwd_t<bf16_t>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_F16:  return fwd_t<f16_t>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_BF16_F32: return fwd_t<bf16w_t>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_F16_F32:  return fwd_t<f16w_t>(x, B, C, h, y, y2, bx, dm, st);
    }
    return (int)hipErrorInvalidValue;
}

size_t direct_bwd_workspace(const Dims &dm)
{
    const BwdPlan p = plan_bwd(dm);
    return (size_t)p.nwg * p.gpt * dm.hl * sizeof(float);
}

int direct_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C, const void *h,
                      void *dx, void *dB, void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return bwd_t<float>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_BF16: return bwd_t<bf16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_F16:  return bwd_t<f16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_BF16_F32: return bwd_t<bf16w_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_F16_F32:  return bwd_t<f16w_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    }
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
