// Short causal depthwise convolution without gates (the featurizer of the hyena blocks):
//   y[b, t, c] = sum_k w[c / dg, k] * x[b, t - (hl-1) + k, c],     hl <= 8,
// on (bs, L, g, dg) tensors with the channel fastest, and its backward (dx, dw).
//
// Same register-window scheme as the gated Hyena-SE kernels: a lane owns 4 adjacent channels
// (one 8- or 16-byte vector per row) and walks a run of rows with the last 8 rows in a register
// ring; tensors are addressed through windows, so no access sits behind a branch.  The filters
// here are usually one per channel (dg = 1): a lane then holds 4 filters and 4 filter-gradient
// accumulators per tap (PCF); with dg % 4 == 0 it holds one, as in the gated kernels.
#include "gcg_rowvec.h"

#include <cstdlib>

namespace gcg {
namespace {

constexpr int RING = 8;
constexpr int BATCH = 4;        // rows fetched together

struct DwPlan { int v, nvec, nseg, ts, ncvb, threads; int64_t nrows, nwg; };

// filter taps of a lane: hr[j][v] multiplies the sample j rows in the past of channel v
template <typename T, int HL, int V, bool PCF>
__device__ __forceinline__ void load_taps(const T *w, int64_t c, int dg, int hl, float (&hr)[HL][PCF ? V : 1])
{
#pragma unroll
    for (int v = 0; v < (PCF ? V : 1); ++v) {
        const T *wg = w + ((c + v) / dg) * hl;
#pragma unroll
        for (int j = 0; j < HL; ++j) hr[j][v] = (j < hl) ? Elem<T>::load(wg + hl - 1 - j) : 0.f;
    }
}

template <typename T, int HL, int V, bool PCF, bool KEEP>
__global__ __launch_bounds__(256) void dwconv_fwd_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                         T *__restrict__ y, Dims dm, DwPlan pl)
{
    typedef typename Vec<T, V>::raw raw_t;
    constexpr int ES = sizeof(T), NF = PCF ? V : 1;
    int64_t wg = blockIdx.x;
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t L = dm.L, d = dm.d, c = (int64_t)cv * V;

    float hr[HL][NF];
    load_taps<T, HL, V, PCF>(w, c, dm.dg, dm.hl, hr);

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t0 = t_start - (HL - 1) > 0 ? t_start - (HL - 1) : 0;
    const int64_t origin = (b * L + t0) * d;
    const uint32_t row = (uint32_t)(d * ES), lane = (uint32_t)(c * ES);
    const win_t wx = make_window(x + origin, (t_end - t0) * row), wy = make_window(y + origin, (t_end - t0) * row);

    float ring[RING][V];
#pragma unroll
    for (int s = 0; s < RING; ++s)
#pragma unroll
        for (int v = 0; v < V; ++v) ring[s][v] = 0.f;
    {   // halo: rows t_start-(HL-1) .. t_start-1 (zero before the sequence) go to slots (t & 7)
        raw_t halo[HL - 1 > 0 ? HL - 1 : 1];
#pragma unroll
        for (int i = 1; i < HL; ++i) halo[i - 1] = win_load<raw_t>(wx, lane + (uint32_t)(t_start - i - t0) * row);
#pragma unroll
        for (int i = 1; i < HL; ++i) unpackv<T, V>(halo[i - 1], ring[RING - i]);
    }

    // rows are fetched BATCH at a time, one batch ahead
    raw_t in[2][BATCH];
#pragma unroll
    for (int kk = 0; kk < BATCH; ++kk) in[0][kk] = win_load<raw_t>(wx, lane + (uint32_t)(t_start + kk - t0) * row);
    for (int64_t tb = t_start; tb < t_end; tb += RING) {
#pragma unroll
        for (int half = 0; half < RING / BATCH; ++half) {
            const int cur = half % 2, nxt = (half + 1) % 2;
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk)
                in[nxt][kk] = win_load<raw_t>(wx, lane + (uint32_t)(tb + (half + 1) * BATCH + kk - t0) * row);
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const int k = half * BATCH + kk;
                float acc[V];
                unpackv<T, V>(in[cur][kk], ring[k]);
#pragma unroll
                for (int v = 0; v < V; ++v) acc[v] = 0.f;
#pragma unroll
                for (int j = HL - 1; j >= 0; --j)
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        acc[v] = fmaf(hr[j][PCF ? v : 0], ring[(k - j) & (RING - 1)][v], acc[v]);
                win_store_as<KEEP>(wy, lane + (uint32_t)(tb + k - t0) * row, packv<T, V>(acc));
            }
        }
    }
}

// Backward: dx[t] = sum_j w[hl-1-j] dy[t+j] looks forward, so the walk runs HL-1 rows past the
// run reading only dy; dw[hl-1-j] = sum_t dy[t] x[t-j] is accumulated per lane over the rows of
// the run and reduced by a second kernel in a fixed order.
template <typename T, int HL, int V, bool PCF>
__global__ __launch_bounds__(256) void dwconv_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                         const T *__restrict__ w, T *__restrict__ dx,
                                                         float *__restrict__ ws, Dims dm, DwPlan pl)
{
    typedef typename Vec<T, V>::raw raw_t;
    constexpr int ES = sizeof(T), NF = PCF ? V : 1;
    // workgroups of one XCD take adjacent channel blocks of the same rows (measured +3-5 % in the
    // backward kernels, -3 % in the forward ones, which keep the plain order)
    int64_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t L = dm.L, d = dm.d, c = (int64_t)cv * V;
    const int hl = dm.hl;

    float hr[HL][NF];
    load_taps<T, HL, V, PCF>(w, c, dm.dg, hl, hr);

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t_stop = t_end + (HL - 1);
    const int64_t t0 = t_start - (HL - 1) > 0 ? t_start - (HL - 1) : 0;
    const int64_t t_far = t_stop < L ? t_stop : L;
    const int64_t origin = (b * L + t0) * d, out_origin = (b * L + t_start) * d;
    const uint32_t row = (uint32_t)(d * ES), lane = (uint32_t)(c * ES);
    const win_t wx = make_window(x + origin, (t_end - t0) * row);
    const win_t wdy = make_window(dy + origin, (t_far - t0) * row);
    const win_t wdx = make_window(dx + out_origin, (t_end - t_start) * row);

    float ur[RING][V], gr[RING][V], dwa[HL][NF];
#pragma unroll
    for (int s = 0; s < RING; ++s)
#pragma unroll
        for (int v = 0; v < V; ++v) { ur[s][v] = 0.f; gr[s][v] = 0.f; }
#pragma unroll
    for (int j = 0; j < HL; ++j)
#pragma unroll
        for (int f = 0; f < NF; ++f) dwa[j][f] = 0.f;
    {
        raw_t halo[HL - 1 > 0 ? HL - 1 : 1];
#pragma unroll
        for (int i = 1; i < HL; ++i) halo[i - 1] = win_load<raw_t>(wx, lane + (uint32_t)(t_start - i - t0) * row);
#pragma unroll
        for (int i = 1; i < HL; ++i) unpackv<T, V>(halo[i - 1], ur[RING - i]);
    }

    for (int64_t tb = t_start; tb < t_stop; tb += RING) {
#pragma unroll
        for (int half = 0; half < RING / BATCH; ++half) {
            raw_t xr[BATCH], dyr[BATCH];
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const uint32_t o = lane + (uint32_t)(tb + half * BATCH + kk - t0) * row;
                xr[kk] = win_load<raw_t>(wx, o);      // zero past the run
                dyr[kk] = win_load<raw_t>(wdy, o);
            }
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const int k = half * BATCH + kk;
                const int64_t t = tb + k;
                const bool in_run = t < t_end;        // uniform; rows past the run belong to the next run's dw
                unpackv<T, V>(xr[kk], ur[k]);
                unpackv<T, V>(dyr[kk], gr[k]);
#pragma unroll
                for (int j = 0; j < HL; ++j) {
                    float part[NF];
#pragma unroll
                    for (int f = 0; f < NF; ++f) part[f] = 0.f;
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        const float gd = in_run ? gr[k][v] : 0.f;
                        part[PCF ? v : 0] = fmaf(gd, ur[(k - j) & (RING - 1)][v], part[PCF ? v : 0]);
                    }
#pragma unroll
                    for (int f = 0; f < NF; ++f) dwa[j][f] += part[f];
                }
                // dx of row t-(HL-1); rows before the run fall outside the output window
                float du[V];
#pragma unroll
                for (int v = 0; v < V; ++v) du[v] = 0.f;
#pragma unroll
                for (int j = 0; j < HL; ++j)
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        du[v] = fmaf(hr[j][PCF ? v : 0], gr[(k - (HL - 1) + j) & (RING - 1)][v], du[v]);
                win_store(wdx, lane + (uint32_t)(t - (HL - 1) - t_start) * row, packv<T, V>(du));
            }
        }
    }
    // partials: ws[tap][row of (batch, run)][filter slot]; filter slot = channel (PCF) or lane
    const int64_t prow = b * pl.nseg + seg;
    const int64_t nslot = PCF ? d : pl.nvec;
#pragma unroll
    for (int j = 0; j < HL; ++j)
        if (j < hl) {
            float *dst = ws + ((size_t)(hl - 1 - j) * pl.nrows + prow) * nslot + (PCF ? c : cv);
#pragma unroll
            for (int f = 0; f < NF; ++f) dst[f] = dwa[j][f];
        }
}

// Channels per lane: 4.  Eight (16-byte vectors at 16 bits) measured the same within noise at the
// 7B featurizer shape (forward 160 vs 153 us, backward 265 vs 269 us) and stays a tuning override.
int lane_width(int dtype, const Dims &dm)
{
    static const char *env = tuning_env("GCG_DWCONV_V");       // tuning override: 4 or 8
    const int want = env ? atoi(env) : 4;
    if (dtype != GCG_F32 && want == 8 && dm.d % 8 == 0 && (dm.dg == 1 || dm.dg % 8 == 0)) return 8;
    return 4;
}

DwPlan plan(const Dims &dm, int V)
{
    DwPlan p;
    p.v = V;
    p.nvec = (int)(dm.d / V);
    p.ts = 128;
    while (p.ts > 8 && dm.bs * ((dm.L + p.ts - 1) / p.ts) * p.nvec < 128 * 1024) p.ts >>= 1;
    static const char *env = tuning_env("GCG_DWCONV_ROWS");     // tuning override: rows per lane, a multiple of 8
    if (env && atoi(env) >= 8 && atoi(env) % 8 == 0) p.ts = atoi(env);
    while (p.ts > 8 && (int64_t)(p.ts + 2 * RING) * dm.d * 4 > WIN_MAX_BYTES) p.ts >>= 1;
    p.nseg = (int)((dm.L + p.ts - 1) / p.ts);
    p.nrows = dm.bs * p.nseg;
    p.threads = p.nvec >= 256 ? 256 : ((p.nvec + 63) / 64) * 64;
    p.ncvb = (p.nvec + p.threads - 1) / p.threads;
    p.nwg = dm.bs * p.nseg * p.ncvb;
    return p;
}

template <typename T, int HL, int V, bool PCF>
int fwd_launch(const void *x, const void *w, void *y, const Dims &dm, hipStream_t st)
{
    int e = 0;
    const DwPlan p = plan(dm, V);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (dm.keep_out)
        e = launch_plain((dwconv_fwd_kernel<T, HL, V, PCF, true>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                           (const T *)x, (const T *)w, (T *)y, dm, p);
    else
        e = launch_plain((dwconv_fwd_kernel<T, HL, V, PCF, false>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                           (const T *)x, (const T *)w, (T *)y, dm, p);
    return e;
}

template <typename T, int HL, int V, bool PCF>
int bwd_launch(const void *dy, const void *x, const void *w, void *dx, void *dw, void *ws, const Dims &dm,
               hipStream_t st)
{
    int e = 0;
    const DwPlan p = plan(dm, V);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    e = launch_plain((dwconv_bwd_kernel<T, HL, V, PCF>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                       (const T *)dy, (const T *)x, (const T *)w, (T *)dx, (float *)ws, dm, p);
    if (e) return e;
    // partials are ws[tap][(batch, run)][slot], slot = channel (per-channel filters) or lane
    return launch_colsum_reduce<T>((const float *)ws, (T *)dw, p.nrows, PCF ? dm.d : p.nvec, PCF ? dm.dg : dm.dg / V,
                                   dm.g, dm.hl, st);
}

template <typename T, int V, bool PCF> int fwd_hl(const void *x, const void *w, void *y, const Dims &dm, hipStream_t st)
{
    if (dm.hl <= 4) return fwd_launch<T, 4, V, PCF>(x, w, y, dm, st);
    return fwd_launch<T, 8, V, PCF>(x, w, y, dm, st);
}
template <typename T, int V, bool PCF>
int bwd_hl(const void *dy, const void *x, const void *w, void *dx, void *dw, void *ws, const Dims &dm, hipStream_t st)
{
    if (dm.hl <= 4) return bwd_launch<T, 4, V, PCF>(dy, x, w, dx, dw, ws, dm, st);
    return bwd_launch<T, 8, V, PCF>(dy, x, w, dx, dw, ws, dm, st);
}

template <typename T, int V> int fwd_v(const void *x, const void *w, void *y, const Dims &dm, hipStream_t st)
{
    return dm.dg % V == 0 ? fwd_hl<T, V, false>(x, w, y, dm, st) : fwd_hl<T, V, true>(x, w, y, dm, st);
}
template <typename T, int V>
int bwd_v(const void *dy, const void *x, const void *w, void *dx, void *dw, void *ws, const Dims &dm, hipStream_t st)
{
    return dm.dg % V == 0 ? bwd_hl<T, V, false>(dy, x, w, dx, dw, ws, dm, st)
                          : bwd_hl<T, V, true>(dy, x, w, dx, dw, ws, dm, st);
}

template <typename T> int fwd_t(int dtype, const void *x, const void *w, void *y, const Dims &dm, hipStream_t st)
{
    if constexpr (sizeof(T) == 2) {
        if (lane_width(dtype, dm) == 8) return fwd_v<T, 8>(x, w, y, dm, st);
    }
    return fwd_v<T, 4>(x, w, y, dm, st);
}
template <typename T>
int bwd_t(int dtype, const void *dy, const void *x, const void *w, void *dx, void *dw, void *ws, const Dims &dm,
          hipStream_t st)
{
    if constexpr (sizeof(T) == 2) {
        if (lane_width(dtype, dm) == 8) return bwd_v<T, 8>(dy, x, w, dx, dw, ws, dm, st);
    }
    return bwd_v<T, 4>(dy, x, w, dx, dw, ws, dm, st);
}

} // namespace

// lanes own 4 adjacent channels: either they share a filter (dg % 4 == 0) or each has its own (dg == 1)
bool dwconv_supported(const Dims &dm)
{
    return dm.hl <= RING && dm.d % 4 == 0 && (dm.dg % 4 == 0 || dm.dg == 1) &&
           (int64_t)(3 * RING) * dm.d * 4 <= WIN_MAX_BYTES && (int64_t)dm.g * dm.hl <= 0x7fffffffLL;
}

int dwconv_fwd_launch(int dtype, const void *x, const void *w, void *y, const Dims &dm, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return fwd_t<float>(dtype, x, w, y, dm, st);
    case GCG_BF16: return fwd_t<bf16_t>(dtype, x, w, y, dm, st);
    case GCG_F16:  return fwd_t<f16_t>(dtype, x, w, y, dm, st);
    }
    return (int)hipErrorInvalidValue;
}

// the larger of the two lane widths' needs, so the figure does not depend on the element type
size_t dwconv_bwd_workspace(const Dims &dm)
{
    size_t n = 0;
    for (int v : {4, 8}) {
        if (dm.d % v) continue;
        const DwPlan p = plan(dm, v);
        const int64_t nslot = dm.dg % v == 0 ? p.nvec : dm.d;
        const size_t need = (size_t)dm.hl * p.nrows * nslot * sizeof(float);
        if (need > n) n = need;
    }
    return n;
}

int dwconv_bwd_launch(int dtype, const void *dy, const void *x, const void *w, void *dx, void *dw, void *ws,
                      const Dims &dm, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return bwd_t<float>(dtype, dy, x, w, dx, dw, ws, dm, st);
    case GCG_BF16: return bwd_t<bf16_t>(dtype, dy, x, w, dx, dw, ws, dm, st);
    case GCG_F16:  return bwd_t<f16_t>(dtype, dy, x, w, dx, dw, ws, dm, st);
    }
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
