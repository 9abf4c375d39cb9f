// Featurizer conv and Hyena-SE operator in one pass over the projected features.
//
//   f[b, t, c3]  = T( sum_k wf[c3, k] * raw[b, t - (kf-1) + k, c3] )          c3 = 3*c + p   (kf <= 4 taps per channel)
//   y[b, t, c]   = f[.., 3c] * sum_k h[c / dg, k] * (f[.., 3c+1] * f[.., 3c+2])[t - (hl-1) + k]        (hl <= 8)
//
// i.e. gcg_dwconv_fwd on the (bs, L, 3d) features followed by gcg_fwd_interleaved, with f rounded to
// the element type T in between exactly as when the two run separately -- but f never goes to
// memory: the forward reads raw (3N) and writes y (N), the backward reads dy (N) and raw (3N) and
// writes d raw (3N), 11 N elements instead of 26 N for the chain of four kernels.
//
// This works in the register-window scheme because a lane owns its channels for a whole run of
// rows: the featurizer's taps reach back over rows the lane has just seen, and in the backward
// the two transposed convolutions are two delays of the same walk.  A lane takes one 12-byte piece
// of the interleaved row per step -- (C, B, x) of two channels at 16 bits, of one at fp32.
#include "gcg_rowvec.h"

#include <cstdlib>

namespace gcg {
namespace {

#ifndef MIXER_WPE
#define MIXER_WPE 2               // waves per SIMD the backward is compiled for (its register budget)
#endif
constexpr int BATCH = 4;          // rows fetched together
constexpr int KF_MAX = 4;         // featurizer taps: kernels are built for 3 and 4 (shorter filters are zero-padded)

struct MixPlan { int ch, nvec, nseg, ts, ncvb, threads; int64_t nrows, nwg; };

template <typename T> struct Piece {
    static constexpr int CH = 4 / (int)sizeof(T);      // channels of the operator per lane
    static constexpr int E = 3 * CH;                   // feature channels per lane: (C, B, x) per channel
    static __device__ __forceinline__ void unpack(const u32x3 &p, float (&f)[E])
    {
#pragma unroll
        for (int i = 0; i < 3; ++i) Word<T>::unpack(p[i], &f[i * Word<T>::N]);
    }
    static __device__ __forceinline__ u32x3 pack(const float (&f)[E])
    {
        u32x3 p;
#pragma unroll
        for (int i = 0; i < 3; ++i) p[i] = Word<T>::pack(&f[i * Word<T>::N]);
        return p;
    }
    // value as stored in a tensor of element type T
    static __device__ __forceinline__ void round_to_t(float (&f)[E])
    {
        if constexpr (sizeof(T) == 2) {
            const u32x3 p = pack(f);
            unpack(p, f);
        }
    }
    // The same words, but as values the compiler cannot trace back: a second unpack of a row kept in
    // a ring is then done where it is written, instead of the first unpack's floats being kept
    // alive for as many rows as the ring is deep (which costs twice the registers at 16 bits).
    static __device__ __forceinline__ u32x3 reread(const u32x3 &p)
    {
        uint32_t a = p[0], b = p[1], c = p[2];
        asm volatile("" : "+v"(a), "+v"(b), "+v"(c));
        return u32x3{a, b, c};
    }
    static __device__ __forceinline__ uint32_t pack_unit(const float (&f)[CH]) { return Word<T>::pack(f); }
    static __device__ __forceinline__ void unpack_unit(uint32_t w, float (&f)[CH]) { Word<T>::unpack(w, f); }
};

// taps of a lane: wfr[j][e] multiplies the raw sample j rows in the past of feature channel c3 + e,
// hr[j] the pre-gate product j rows in the past
template <typename T, int HL, int KF>
__device__ __forceinline__ void load_taps(const T *wf, const T *h, int64_t c, const Dims &dm, int kf,
                                          float (&wfr)[KF][Piece<T>::E], float (&hr)[HL])
{
#pragma unroll
    for (int e = 0; e < Piece<T>::E; ++e) {
        const T *wp = wf + (3 * c + e) * kf;
#pragma unroll
        for (int j = 0; j < KF; ++j) wfr[j][e] = (j < kf) ? Elem<T>::load(wp + kf - 1 - j) : 0.f;
    }
    const T *hg = h + (c / dm.dg) * dm.hl;
#pragma unroll
    for (int j = 0; j < HL; ++j) hr[j] = (j < dm.hl) ? Elem<T>::load(hg + dm.hl - 1 - j) : 0.f;
}

// f of the row in raw-ring slot s: taps over slots s, s-1, ... (same order of operations as the
// stand-alone featurizer kernel), rounded to T
template <typename T, int KF>
__device__ __forceinline__ void featurize(const float (&wfr)[KF][Piece<T>::E], const float (&rr)[4][Piece<T>::E], int s,
                                          float (&f)[Piece<T>::E])
{
#pragma unroll
    for (int e = 0; e < Piece<T>::E; ++e) f[e] = 0.f;
#pragma unroll
    for (int j = KF - 1; j >= 0; --j)
#pragma unroll
        for (int e = 0; e < Piece<T>::E; ++e) f[e] = fmaf(wfr[j][e], rr[(s - j) & 3][e], f[e]);
    Piece<T>::round_to_t(f);
}

// the same from a ring of packed rows (16 slots)
template <typename T, int KF>
__device__ __forceinline__ void featurize_packed(const float (&wfr)[KF][Piece<T>::E], const u32x3 (&rp)[16], int s,
                                                 float (&f)[Piece<T>::E])
{
#pragma unroll
    for (int e = 0; e < Piece<T>::E; ++e) f[e] = 0.f;
#pragma unroll
    for (int j = KF - 1; j >= 0; --j) {
        float r[Piece<T>::E];
        Piece<T>::unpack(j ? Piece<T>::reread(rp[(s - j) & 15]) : rp[(s - j) & 15], r);
#pragma unroll
        for (int e = 0; e < Piece<T>::E; ++e) f[e] = fmaf(wfr[j][e], r[e], f[e]);
    }
    Piece<T>::round_to_t(f);
}

// ---------------------------------------------------------------------------- forward
template <typename T, int HL, int KF>
__global__ __launch_bounds__(256) void mixer_se_fwd_kernel(const T *__restrict__ raw, const T *__restrict__ wf,
                                                           const T *__restrict__ h, T *__restrict__ y, Dims dm,
                                                           int kf, MixPlan pl)
{
    typedef Piece<T> P;
    constexpr int ES = sizeof(T), CH = P::CH, E = P::E, NH = HL - 1 + KF - 1;
    int64_t wg = blockIdx.x;
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t L = dm.L, d = dm.d, c = (int64_t)cv * CH;

    float wfr[KF][E], hr[HL];
    load_taps<T, HL, KF>(wf, h, c, dm, kf, wfr, hr);

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t0 = t_start - NH > 0 ? t_start - NH : 0;                 // first row of the input window
    const uint32_t orow = (uint32_t)(d * ES), irow = 3 * orow;
    const win_t wr = make_window(raw + 3 * (b * L + t0) * d, (t_end - t0) * irow);
    const win_t wy = make_window(y + (b * L + t_start) * d, (t_end - t_start) * orow);
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = 3 * lane_o;
    auto load_raw = [&](int64_t t) { return win_load<u32x3>(wr, lane_i + (uint32_t)(t - t0) * irow); };

    float rr[4][E], ur[8][CH];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int e = 0; e < E; ++e) rr[s][e] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) ur[s][ch] = 0.f;

    // Halo: the HL-1 rows before the run give the operator its history, and the KF-1 rows before
    // those give the featurizer its own.  Rows before the sequence read as zero.  t_start is a
    // multiple of 8, so row t_start - i sits in ring slots (-i) & 3 and (-i) & 7.
    {
        u32x3 hp[NH];
#pragma unroll
        for (int i = 1; i <= NH; ++i) hp[i - 1] = load_raw(t_start - i);
#pragma unroll
        for (int i = NH; i >= 1; --i) {
            P::unpack(hp[i - 1], rr[(-i) & 3]);
            if (i <= HL - 1) {
                float f[E];
                featurize<T, KF>(wfr, rr, (-i) & 3, f);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) ur[(-i) & 7][ch] = f[3 * ch + 1] * f[3 * ch + 2];
            }
        }
    }

    u32x3 in[2][BATCH];
#pragma unroll
    for (int kk = 0; kk < BATCH; ++kk) in[0][kk] = load_raw(t_start + kk);
    for (int64_t tb = t_start; tb < t_end; tb += 8) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int cur = half, nxt = half ^ 1;
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) in[nxt][kk] = load_raw(tb + (half + 1) * BATCH + kk);
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const int k = half * BATCH + kk;
                float f[E], out[CH];
                P::unpack(in[cur][kk], rr[k & 3]);
                featurize<T, KF>(wfr, rr, k & 3, f);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) {
                    ur[k][ch] = f[3 * ch + 1] * f[3 * ch + 2];
                    float acc = 0.f;
#pragma unroll
                    for (int j = HL - 1; j >= 0; --j) acc = fmaf(hr[j], ur[(k - j) & 7][ch], acc);
                    out[ch] = f[3 * ch] * acc;
                }
                win_store(wy, lane_o + (uint32_t)(tb + k - t_start) * orow, P::pack_unit(out));
            }
        }
    }
}

// --------------------------------------------------------------------------- backward
// One walk with two delays.  At step t the lane loads raw[t] and dy[t], rebuilds f[t] and
// g2[t] = dy * C, and produces dC[t] (it looks back).  HL-1 steps later du of that row is complete
// (it looks forward over g2), which gives dB, dx and so d f of row t1 = t - (HL-1); KF-1 steps
// after that the transposed featurizer taps have seen d f of rows t2 .. t2 + KF-1 and d raw of row
// t2 = t1 - (KF-1) leaves.  The walk therefore runs HL-1 + KF-1 rows past the run, and computes
// d f for KF-1 rows past the run (the next run's lane computes them too; nothing is exchanged).
// Filter gradients (dh, dwf) only take the rows of the run.
template <typename T, int HL, int KF>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MIXER_WPE))) void mixer_se_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ raw,
                                                           const T *__restrict__ wf, const T *__restrict__ h,
                                                           T *__restrict__ draw, float *__restrict__ ws_h,
                                                           float *__restrict__ ws_w, Dims dm, int kf, MixPlan pl)
{
    typedef Piece<T> P;
    constexpr int ES = sizeof(T), CH = P::CH, E = P::E, D1 = HL - 1, D2 = KF - 1, NH = D1 + D2;
    int64_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t L = dm.L, d = dm.d, c = (int64_t)cv * CH;
    const int hl = dm.hl;

    float wfr[KF][E], hr[HL];
    load_taps<T, HL, KF>(wf, h, c, dm, kf, wfr, hr);

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t_df = t_end + D2;                    // d f is needed up to here (exclusive)
    const int64_t t_stop = t_end + NH;                  // exclusive bound of the walk
    const int64_t t0 = t_start - NH > 0 ? t_start - NH : 0;
    const int64_t t_far = t_stop < L ? t_stop : L;
    const uint32_t orow = (uint32_t)(d * ES), irow = 3 * orow;
    const win_t wr = make_window(raw + 3 * (b * L + t0) * d, (t_far - t0) * irow);
    const win_t wdy = make_window(dy + (b * L + t0) * d, (t_far - t0) * orow);
    const win_t wdr = make_window(draw + 3 * (b * L + t_start) * d, (t_end - t_start) * irow);
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = 3 * lane_o;

    // rings, slot = row & (size-1):  rp raw rows as loaded (the featurizer's history and, HL-1 + KF-1
    // rows back, the terms of dwf), ur u, gr g2, xs / Bs f's x and B, dCs dC, dfr d f (the last four
    // as elements of type T, which is what they are rounded to anyway)
    float ur[8][CH], gr[8][CH], dha[HL], dwa[KF][E];
    u32x3 rp[16], dfr[4];
    uint32_t xs[8], Bs[8], dCs[8];
#pragma unroll
    for (int s = 0; s < 4; ++s) dfr[s] = u32x3{0u, 0u, 0u};
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        xs[s] = 0u; Bs[s] = 0u; dCs[s] = 0u;
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) { ur[s][ch] = 0.f; gr[s][ch] = 0.f; }
    }
#pragma unroll
    for (int s = 0; s < 16; ++s) rp[s] = u32x3{0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < HL; ++j) dha[j] = 0.f;
#pragma unroll
    for (int j = 0; j < KF; ++j)
#pragma unroll
        for (int e = 0; e < E; ++e) dwa[j][e] = 0.f;

    // halo on the left (t_start is a multiple of 16): u of the HL-1 rows before the run, raw of
    // the KF-1 rows before those
    {
        u32x3 hp[NH];
#pragma unroll
        for (int i = 1; i <= NH; ++i) hp[i - 1] = win_load<u32x3>(wr, lane_i + (uint32_t)(t_start - i - t0) * irow);
#pragma unroll
        for (int i = NH; i >= 1; --i) {
            rp[(-i) & 15] = hp[i - 1];
            if (i <= D1) {
                float f[E];
                featurize_packed<T, KF>(wfr, rp, (-i) & 15, f);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) ur[(-i) & 7][ch] = f[3 * ch + 1] * f[3 * ch + 2];
            }
        }
    }

    for (int64_t tb = t_start; tb < t_stop; tb += 16) {
#pragma unroll
        for (int q = 0; q < 16 / BATCH; ++q) {
            u32x3 in[BATCH];
            uint32_t dyr[BATCH];
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const uint32_t row = (uint32_t)(tb + q * BATCH + kk - t0);
                in[kk] = win_load<u32x3>(wr, lane_i + row * irow);          // zero past t_far
                dyr[kk] = win_load<uint32_t>(wdy, lane_o + row * orow);
            }
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const int k = q * BATCH + kk;                               // row tb + k, ring slots from k
                const int64_t t = tb + k;
                // ---- stage 1: row t
                {
                    float f[E], dyf[CH], xv[CH], Bv[CH], dCv[CH];
                    rp[k & 15] = in[kk];
                    featurize_packed<T, KF>(wfr, rp, k & 15, f);
                    P::unpack_unit(dyr[kk], dyf);
                    const bool live = t < t_df;         // rows whose d f is wanted (uniform)
                    const bool in_run = t < t_end;      // rows whose filter-gradient terms are ours
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) {
                        xv[ch] = f[3 * ch + 2];
                        Bv[ch] = f[3 * ch + 1];
                        gr[k & 7][ch] = dyf[ch] * f[3 * ch];
                        ur[k & 7][ch] = live ? Bv[ch] * xv[ch] : 0.f;
                    }
                    xs[k & 7] = P::pack_unit(xv);
                    Bs[k & 7] = P::pack_unit(Bv);
                    float y2v[CH];
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) y2v[ch] = 0.f;
#pragma unroll
                    for (int j = HL - 1; j >= 0; --j) {
                        float sacc = 0.f;
#pragma unroll
                        for (int ch = 0; ch < CH; ++ch) {
                            const float u = ur[(k - j) & 7][ch];
                            y2v[ch] = fmaf(hr[j], u, y2v[ch]);
                            sacc = fmaf(in_run ? gr[k & 7][ch] : 0.f, u, sacc);
                        }
                        dha[j] += sacc;
                    }
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) dCv[ch] = dyf[ch] * y2v[ch];
                    dCs[k & 7] = P::pack_unit(dCv);
                }
                // ---- stage 2: d f of row t1 = t - D1 (rounded to T, as the interleaved backward stores it)
                {
                    const int k1 = k - D1;
                    const int64_t t1 = t - D1;
                    float du[CH], xo[CH], Bo[CH], dCo[CH], df[E];
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) du[ch] = 0.f;
#pragma unroll
                    for (int j = 0; j < HL; ++j)
#pragma unroll
                        for (int ch = 0; ch < CH; ++ch) du[ch] = fmaf(hr[j], gr[(k1 + j) & 7][ch], du[ch]);
                    P::unpack_unit(xs[k1 & 7], xo);
                    P::unpack_unit(Bs[k1 & 7], Bo);
                    P::unpack_unit(dCs[k1 & 7], dCo);
                    const bool have = t1 >= t_start && t1 < t_df;          // uniform; outside, d f counts as zero
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) {
                        df[3 * ch] = have ? dCo[ch] : 0.f;
                        df[3 * ch + 1] = have ? du[ch] * xo[ch] : 0.f;
                        df[3 * ch + 2] = have ? du[ch] * Bo[ch] : 0.f;
                    }
                    const u32x3 dfp = P::pack(df);
                    P::unpack(dfp, df);
                    // featurizer filter gradient: dwf[.., KF-1-j] += d f[t1] * raw[t1 - j], rows of the run only
                    const bool mine = t1 >= t_start && t1 < t_end;
                    float rj[E];
#pragma unroll
                    for (int j = 0; j < KF; ++j) {
                        P::unpack(P::reread(rp[(k1 - j) & 15]), rj);
#pragma unroll
                        for (int e = 0; e < E; ++e) dwa[j][e] = fmaf(mine ? df[e] : 0.f, rj[e], dwa[j][e]);
                    }
                    dfr[k1 & 3] = dfp;
                }
                // ---- stage 3: d raw of row t2 = t1 - D2; rows outside the run fall outside the window
                {
                    const int k2 = k - D1 - D2;
                    float dr[E];
#pragma unroll
                    for (int e = 0; e < E; ++e) dr[e] = 0.f;
#pragma unroll
                    for (int j = 0; j < KF; ++j) {
                        float dfj[E];
                        P::unpack(P::reread(dfr[(k2 + j) & 3]), dfj);
#pragma unroll
                        for (int e = 0; e < E; ++e) dr[e] = fmaf(wfr[j][e], dfj[e], dr[e]);
                    }
                    win_store(wdr, lane_i + (uint32_t)(t - D1 - D2 - t_start) * irow, P::pack(dr));
                }
            }
        }
    }
    // partials: ws_h[tap][(batch, run)][lane], ws_w[tap][(batch, run)][feature channel]
    const int64_t prow = b * pl.nseg + seg;
#pragma unroll
    for (int j = 0; j < HL; ++j)
        if (j < hl) ws_h[((size_t)(hl - 1 - j) * pl.nrows + prow) * pl.nvec + cv] = dha[j];
#pragma unroll
    for (int j = 0; j < KF; ++j)
        if (j < kf) {
            float *dst = ws_w + ((size_t)(kf - 1 - j) * pl.nrows + prow) * (3 * d) + 3 * c;
#pragma unroll
            for (int e = 0; e < E; ++e) dst[e] = dwa[j][e];
        }
}

MixPlan plan(const Dims &dm, int ch)
{
    MixPlan p;
    p.ch = ch;
    p.nvec = (int)(dm.d / ch);
    p.ts = 128;
    // runs of 128 rows unless that leaves fewer than two workgroups per CU; multiples of 16 (the
    // backward's longest ring) down to 16
    while (p.ts > 16 && dm.bs * ((dm.L + p.ts - 1) / p.ts) * p.nvec < 128 * 1024) p.ts >>= 1;
    static const char *env = getenv("GCG_MIXER_ROWS");      // tuning override: rows per lane, a multiple of 16
    if (env && atoi(env) >= 16 && atoi(env) % 16 == 0) p.ts = atoi(env);
    while (p.ts > 16 && (int64_t)(p.ts + 32) * 3 * dm.d * 4 > WIN_MAX_BYTES) p.ts >>= 1;
    p.nseg = (int)((dm.L + p.ts - 1) / p.ts);
    p.nrows = dm.bs * p.nseg;
    p.threads = p.nvec >= 256 ? 256 : ((p.nvec + 63) / 64) * 64;
    p.ncvb = (p.nvec + p.threads - 1) / p.threads;
    p.nwg = dm.bs * p.nseg * p.ncvb;
    return p;
}

int lane_channels(int dtype) { return dtype == GCG_F32 ? 1 : 2; }

template <typename T, int HL, int KF>
int fwd_launch(const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf, hipStream_t st)
{
    const MixPlan p = plan(dm, Piece<T>::CH);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((mixer_se_fwd_kernel<T, HL, KF>), dim3((unsigned)p.nwg), dim3(p.threads), 0, st, (const T *)raw,
                       (const T *)wf, (const T *)h, (T *)y, dm, kf, p);
    return (int)hipGetLastError();
}

template <typename T, int HL, int KF>
int bwd_launch(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh,
               void *ws, const Dims &dm, int kf, hipStream_t st)
{
    const MixPlan p = plan(dm, Piece<T>::CH);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    float *ws_h = (float *)ws;
    float *ws_w = ws_h + (size_t)dm.hl * p.nrows * p.nvec;
    hipLaunchKernelGGL((mixer_se_bwd_kernel<T, HL, KF>), dim3((unsigned)p.nwg), dim3(p.threads), 0, st, (const T *)dy,
                       (const T *)raw, (const T *)wf, (const T *)h, (T *)draw, ws_h, ws_w, dm, kf, p);
    int e = (int)hipGetLastError();
    if (e) return e;
    e = launch_colsum_reduce<T>(ws_h, (T *)dh, p.nrows, p.nvec, dm.dg / p.ch, dm.g, dm.hl, st);
    if (e) return e;
    return launch_colsum_reduce<T>(ws_w, (T *)dwf, p.nrows, 3 * dm.d, 1, (int)(3 * dm.d), kf, st);
}

template <typename T, int KF>
int fwd_k(const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf, hipStream_t st)
{
    if (dm.hl <= 4) return fwd_launch<T, 4, KF>(raw, wf, h, y, dm, kf, st);
    if (dm.hl <= 7) return fwd_launch<T, 7, KF>(raw, wf, h, y, dm, kf, st);
    return fwd_launch<T, 8, KF>(raw, wf, h, y, dm, kf, st);
}
template <typename T>
int fwd_t(const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf, hipStream_t st)
{
    return kf <= 3 ? fwd_k<T, 3>(raw, wf, h, y, dm, kf, st) : fwd_k<T, 4>(raw, wf, h, y, dm, kf, st);
}
template <typename T, int KF>
int bwd_k(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh, void *ws,
          const Dims &dm, int kf, hipStream_t st)
{
    if (dm.hl <= 4) return bwd_launch<T, 4, KF>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    if (dm.hl <= 7) return bwd_launch<T, 7, KF>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    return bwd_launch<T, 8, KF>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
}
template <typename T>
int bwd_t(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh, void *ws,
          const Dims &dm, int kf, hipStream_t st)
{
    return kf <= 3 ? bwd_k<T, 3>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st)
                   : bwd_k<T, 4>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
}

} // namespace

bool mixer_se_supported(const Dims &dm, int kf)
{
    return dm.hl <= 8 && kf >= 1 && kf <= KF_MAX && dm.dg % 2 == 0 && (int64_t)48 * 3 * dm.d * 4 <= WIN_MAX_BYTES &&
           3 * dm.d * (int64_t)KF_MAX <= 0x7fffffffLL;
}

int mixer_se_fwd_launch(int dtype, const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf,
                        hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return fwd_t<float>(raw, wf, h, y, dm, kf, st);
    case GCG_BF16: return fwd_t<bf16_t>(raw, wf, h, y, dm, kf, st);
    case GCG_F16:  return fwd_t<f16_t>(raw, wf, h, y, dm, kf, st);
    }
    return (int)hipErrorInvalidValue;
}

size_t mixer_se_bwd_workspace(int dtype, const Dims &dm, int kf)
{
    const MixPlan p = plan(dm, lane_channels(dtype));
    return ((size_t)dm.hl * p.nrows * p.nvec + (size_t)kf * p.nrows * 3 * dm.d) * sizeof(float);
}

int mixer_se_bwd_launch(int dtype, const void *dy, const void *raw, const void *wf, const void *h, void *draw,
                        void *dwf, void *dh, void *ws, const Dims &dm, int kf, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return bwd_t<float>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    case GCG_BF16: return bwd_t<bf16_t>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    case GCG_F16:  return bwd_t<f16_t>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    }
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
