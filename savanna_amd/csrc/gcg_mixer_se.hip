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
//
// Two pairs of kernels: mixer_se_fwd_kernel / mixer_se_bwd_kernel in the plain form, one FMA per
// tap (instantiated for fp32, where a word is an element and nothing has to be unpacked), and
// mixer_se_fwd16_kernel / mixer_se_bwd16_kernel for bf16 and f16, further down.
#include "gcg_rowvec.h"

#include <cstdlib>
#include <type_traits>

namespace gcg {
namespace {

#ifndef MIXER_WPE
#define MIXER_WPE 2               // waves per SIMD the backward is compiled for (its register budget)
#endif
constexpr int BATCH = 4;          // rows fetched together
#ifndef MIXER_BATCH16
#define MIXER_BATCH16 4
#endif
#ifndef MIXER_BATCH_FWD16
#define MIXER_BATCH_FWD16 4
#endif
constexpr int BATCH16 = MIXER_BATCH16;   // the same in the 16-bit backward, whose registers are scarce
constexpr int KF_MAX = 4;         // featurizer taps: kernels are built for 3 and 4 (shorter filters are zero-padded)

// x if the wave-uniform condition holds, else +0: as a bit mask, which stays one VALU operation with a
// scalar operand (written as a select, the compiler may turn a uniform condition into a branch
// around the row's work, and a branch costs the exact wait counts of the straight-line walk)
__device__ __forceinline__ uint32_t row_mask(bool uniform_cond) { return uniform_cond ? 0xffffffffu : 0u; }
__device__ __forceinline__ float masked(float x, uint32_t m) { return __uint_as_float(__float_as_uint(x) & m); }

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
    static __device__ __forceinline__ uint32_t pack_unit(const float (&f)[CH]) { return Word<T>::pack(f); }
    static __device__ __forceinline__ void unpack_unit(uint32_t w, float (&f)[CH]) { Word<T>::unpack(w, f); }
};

// Planar features (PL; the split without interleaving, block.py:881-884): a row holds the planes C | B | x one after
// the other, d elements each, instead of (C, B, x) channel by channel.  A lane's piece is then three words orow
// bytes apart and its elements come plane by plane (at 16 bits: C0 C1 | B0 B1 | x0 x1), which is all that differs:
// where an element sits in the piece, which feature channel it is, and how the piece is loaded and stored.
template <bool PL, int CH> __device__ __forceinline__ constexpr int ei(int ch, int p) { return PL ? p * CH + ch : 3 * ch + p; }
template <bool PL, int CH> __device__ __forceinline__ int64_t feat_channel(int64_t c, int e, int64_t d)
{
    return PL ? (int64_t)(e / CH) * d + c + e % CH : 3 * c + e;
}
template <bool PL> __device__ __forceinline__ u32x3 piece_load(win_t w, uint32_t off, uint32_t orow)
{
    if constexpr (PL)
        return u32x3{win_load<uint32_t>(w, off), win_load<uint32_t>(w, off + orow), win_load<uint32_t>(w, off + 2 * orow)};
    else
        return win_load<u32x3>(w, off);
}
template <bool PL> __device__ __forceinline__ void piece_store(win_t w, uint32_t off, uint32_t orow, const u32x3 &v)
{
    if constexpr (PL) {
        win_store(w, off, (uint32_t)v[0]);
        win_store(w, off + orow, (uint32_t)v[1]);
        win_store(w, off + 2 * orow, (uint32_t)v[2]);
    } else {
        win_store(w, off, v);
    }
}

// taps of a lane: wfr[j][e] multiplies the raw sample j rows in the past of feature channel c3 + e,
// hr[j] the pre-gate product j rows in the past
template <typename T, int HL, int KF, bool PL>
__device__ __forceinline__ void load_taps(const T *wf, const T *h, int64_t c, const Dims &dm, int kf,
                                          float (&wfr)[KF][Piece<T>::E], float (&hr)[HL])
{
#pragma unroll
    for (int e = 0; e < Piece<T>::E; ++e) {
        const T *wp = wf + feat_channel<PL, Piece<T>::CH>(c, e, dm.d) * kf;
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
        Piece<T>::unpack(rp[(s - j) & 15], r);
#pragma unroll
        for (int e = 0; e < Piece<T>::E; ++e) f[e] = fmaf(wfr[j][e], r[e], f[e]);
    }
    Piece<T>::round_to_t(f);
}

// ---------------------------------------------------------------------------- forward
template <typename T, int HL, int KF, bool PL = false>
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
    load_taps<T, HL, KF, PL>(wf, h, c, dm, kf, wfr, hr);

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t0 = t_start - NH > 0 ? t_start - NH : 0;                 // first row of the input window
    const uint32_t orow = (uint32_t)(d * ES), irow = 3 * orow;
    const win_t wr = make_window(raw + 3 * (b * L + t0) * d, (t_end - t0) * irow);
    const win_t wy = make_window(y + (b * L + t_start) * d, (t_end - t_start) * orow);
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = PL ? lane_o : 3 * lane_o;
    auto load_raw = [&](int64_t t) { return piece_load<PL>(wr, lane_i + (uint32_t)(t - t0) * irow, orow); };

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
                for (int ch = 0; ch < CH; ++ch) ur[(-i) & 7][ch] = f[ei<PL, CH>(ch, 1)] * f[ei<PL, CH>(ch, 2)];
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
                    ur[k][ch] = f[ei<PL, CH>(ch, 1)] * f[ei<PL, CH>(ch, 2)];
                    float acc = 0.f;
#pragma unroll
                    for (int j = HL - 1; j >= 0; --j) acc = fmaf(hr[j], ur[(k - j) & 7][ch], acc);
                    out[ch] = f[ei<PL, CH>(ch, 0)] * acc;
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
template <typename T, int HL, int KF, bool PL = false>
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
    load_taps<T, HL, KF, PL>(wf, h, c, dm, kf, wfr, hr);

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
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = PL ? lane_o : 3 * lane_o;

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
        for (int i = 1; i <= NH; ++i) hp[i - 1] = piece_load<PL>(wr, lane_i + (uint32_t)(t_start - i - t0) * irow, orow);
#pragma unroll
        for (int i = NH; i >= 1; --i) {
            rp[(-i) & 15] = hp[i - 1];
            if (i <= D1) {
                float f[E];
                featurize_packed<T, KF>(wfr, rp, (-i) & 15, f);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) ur[(-i) & 7][ch] = f[ei<PL, CH>(ch, 1)] * f[ei<PL, CH>(ch, 2)];
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
                in[kk] = piece_load<PL>(wr, lane_i + row * irow, orow);     // zero past t_far
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
                    const uint32_t live = row_mask(t < t_df);       // rows whose d f is wanted
                    const uint32_t in_run = row_mask(t < t_end);    // rows whose filter-gradient terms are ours
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) {
                        xv[ch] = f[ei<PL, CH>(ch, 2)];
                        Bv[ch] = f[ei<PL, CH>(ch, 1)];
                        gr[k & 7][ch] = dyf[ch] * f[ei<PL, CH>(ch, 0)];
                        ur[k & 7][ch] = masked(Bv[ch] * xv[ch], live);
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
                            sacc = fmaf(masked(gr[k & 7][ch], in_run), u, sacc);
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
                    const uint32_t have = row_mask(t1 >= t_start && t1 < t_df);     // outside, d f counts as zero
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) {
                        const float duv = masked(du[ch], have);
                        df[ei<PL, CH>(ch, 0)] = masked(dCo[ch], have);
                        df[ei<PL, CH>(ch, 1)] = duv * xo[ch];
                        df[ei<PL, CH>(ch, 2)] = duv * Bo[ch];
                    }
                    const u32x3 dfp = P::pack(df);
                    P::unpack(dfp, df);
                    // featurizer filter gradient: dwf[.., KF-1-j] += d f[t1] * raw[t1 - j], rows of the run only
                    const uint32_t mine = row_mask(t1 >= t_start && t1 < t_end);
                    float rj[E];
#pragma unroll
                    for (int j = 0; j < KF; ++j) {
                        P::unpack(rp[(k1 - j) & 15], rj);
#pragma unroll
                        for (int e = 0; e < E; ++e) dwa[j][e] = fmaf(masked(df[e], mine), rj[e], dwa[j][e]);
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
                        P::unpack(dfr[(k2 + j) & 3], dfj);
#pragma unroll
                        for (int e = 0; e < E; ++e) dr[e] = fmaf(wfr[j][e], dfj[e], dr[e]);
                    }
                    piece_store<PL>(wdr, lane_i + (uint32_t)(t - D1 - D2 - t_start) * irow, orow, P::pack(dr));
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
            float *dst = ws_w + ((size_t)(kf - 1 - j) * pl.nrows + prow) * (3 * d) + (PL ? c : 3 * c);
#pragma unroll
            for (int e = 0; e < E; ++e) dst[PL ? (int64_t)(e / CH) * d + e % CH : (int64_t)e] = dwa[j][e];
        }
}

// ------------------------------------------------------------- 16-bit elements: taps two at a time
// At 16 bits a lane's 12-byte piece holds six feature channels, and unpacking them to floats for
// every tap makes the walk arithmetic-bound.  v_dot2c_f32_{bf16,f16} takes two 16-bit products
// per operand word and adds them to an fp32 accumulator, so the featurizer's sums along time are
// done on words that hold one channel's samples of two consecutive rows: v_perm_b32 builds such a
// word from the words of the two rows, and the packed taps (Wa: taps 0 and 1 rows back, Wb: 2 and 3)
// stay in 12 registers.  The same words serve the three sums along time of the backward (f, d raw, dwf).
template <typename T> struct Pair;
template <> struct Pair<bf16_t> {
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
    {
        typedef __bf16 v2 __attribute__((ext_vector_type(2)));
        v2 x, y;
        __builtin_memcpy(&x, &a, 4);
        __builtin_memcpy(&y, &b, 4);
        return __builtin_amdgcn_fdot2_f32_bf16(x, y, c, false);
    }
    // Both floats converted as one vector: written as two scalar casts put into a vector, the
    // compiler keeps the two bf16 apart, one 32-bit register each, wherever the word is later
    // assembled into another by halves, and every ring of such words then costs twice its registers.
    // (Not inline assembly: the compiler must see which instructions read the result of a dot
    // product, because it has to space them from it.)
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        typedef __bf16 bv2 __attribute__((ext_vector_type(2)));
        typedef float fv2 __attribute__((ext_vector_type(2)));
        const bv2 r = __builtin_convertvector(fv2{lo, hi}, bv2);
        uint32_t u;
        __builtin_memcpy(&u, &r, 4);
        return u;
    }
};
template <> struct Pair<f16_t> {
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
    {
        typedef _Float16 v2 __attribute__((ext_vector_type(2)));
        v2 x, y;
        __builtin_memcpy(&x, &a, 4);
        __builtin_memcpy(&y, &b, 4);
        return __builtin_amdgcn_fdot2(x, y, c, false);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_f16x2(lo, hi); }
};
// a row of six floats / a pair of floats as elements of T
template <typename T> __device__ __forceinline__ u32x3 pack6(const float (&f)[6])
{
    return u32x3{Pair<T>::pack2(f[0], f[1]), Pair<T>::pack2(f[2], f[3]), Pair<T>::pack2(f[4], f[5])};
}
// p[e] = (low half: row `lo`'s sample of feature channel e, high half: row `hi`'s)
__device__ __forceinline__ void pair_rows(const u32x3 &lo, const u32x3 &hi, uint32_t (&p)[6])
{
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        p[2 * i] = __builtin_amdgcn_perm(hi[i], lo[i], 0x05040100u);
        p[2 * i + 1] = __builtin_amdgcn_perm(hi[i], lo[i], 0x07060302u);
    }
}
// word whose low half is half hx of x and whose high half is half hy of y
template <int HX, int HY> __device__ __forceinline__ uint32_t halves(uint32_t x, uint32_t y)
{
    constexpr uint32_t sel = (2u * HX) | ((2u * HX + 1u) << 8) | ((4u + 2u * HY) << 16) | ((5u + 2u * HY) << 24);
    return __builtin_amdgcn_perm(y, x, sel);
}
// packed taps of a lane: Wa[e] = (tap 0 rows back, tap 1 row back), Wb[e] = (2 back, 3 back); hr as above
// (FT: element type of the operator's filter -- T, or float for fp32 arithmetic on 16-bit tensors: the taps of the
// operator are used as fp32 values either way)
template <typename T, int HL, bool PL, typename FT>
__device__ __forceinline__ void load_taps16(const T *wf, const FT *h, int64_t c, const Dims &dm, int kf,
                                            uint32_t (&Wa)[6], uint32_t (&Wb)[6], float (&hr)[HL])
{
#pragma unroll
    for (int e = 0; e < 6; ++e) {
        const T *wp = wf + feat_channel<PL, 2>(c, e, dm.d) * kf;
        float w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = (j < kf) ? Elem<T>::load(wp + kf - 1 - j) : 0.f;
        Wa[e] = Word<T>::pack(&w[0]);
        Wb[e] = Word<T>::pack(&w[2]);
    }
    const FT *hg = h + (c / dm.dg) * dm.hl;
#pragma unroll
    for (int j = 0; j < HL; ++j) hr[j] = (j < dm.hl) ? Elem<FT>::load(hg + dm.hl - 1 - j) : 0.f;
}
// f of row t from pe_t = pair_rows(raw[t], raw[t-1]) and pe_t2 = pair_rows(raw[t-2], raw[t-3]), rounded to T
// (fp: the same row as elements of T)
template <typename T>
__device__ __forceinline__ void featurize16(const uint32_t (&Wa)[6], const uint32_t (&Wb)[6], const uint32_t (&pe_t)[6],
                                            const uint32_t (&pe_t2)[6], float (&f)[6], u32x3 &fp)
{
#pragma unroll
    for (int e = 0; e < 6; ++e) f[e] = Pair<T>::dot2(pe_t[e], Wa[e], Pair<T>::dot2(pe_t2[e], Wb[e], 0.f));
    fp = pack6<T>(f);
    Piece<T>::unpack(fp, f);
}
template <typename T>
__device__ __forceinline__ void featurize16(const uint32_t (&Wa)[6], const uint32_t (&Wb)[6], const uint32_t (&pe_t)[6],
                                            const uint32_t (&pe_t2)[6], float (&f)[6])
{
    u32x3 fp;
    featurize16<T>(Wa, Wb, pe_t, pe_t2, f, fp);
}

template <typename T, int HL, bool PL = false, typename FT = T>
__global__ __launch_bounds__(256) void mixer_se_fwd16_kernel(const T *__restrict__ raw, const T *__restrict__ wf,
                                                             const FT *__restrict__ h, T *__restrict__ y, Dims dm,
                                                             int kf, MixPlan pl)
{
    constexpr int ES = 2, CH = 2, NH = HL - 1 + 3;
    int64_t wg = blockIdx.x;
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t L = dm.L, d = dm.d, c = (int64_t)cv * CH;

    uint32_t Wa[6], Wb[6];
    float hr[HL];
    load_taps16<T, HL, PL, FT>(wf, h, c, dm, kf, Wa, Wb, hr);

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t0 = t_start - NH > 0 ? t_start - NH : 0;
    const uint32_t orow = (uint32_t)(d * ES), irow = 3 * orow;
    const win_t wr = make_window(raw + 3 * (b * L + t0) * d, (t_end - t0) * irow);
    const win_t wy = make_window(y + (b * L + t_start) * d, (t_end - t_start) * orow);
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = PL ? lane_o : 3 * lane_o;
    auto load_raw = [&](int64_t t) { return piece_load<PL>(wr, lane_i + (uint32_t)(t - t0) * irow, orow); };

    // pe[row & 3] = pair_rows(raw[row], raw[row - 1]); ur[row & 7] = u of the row
    uint32_t pe[4][6];
    float ur[8][CH];
    u32x3 prev = u32x3{0u, 0u, 0u};
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int e = 0; e < 6; ++e) pe[s][e] = 0u;
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) ur[s][ch] = 0.f;

    // halo: HL-1 rows of u before the run, and three more rows of raw before those for their f
    {
        u32x3 hp[NH];
#pragma unroll
        for (int i = 1; i <= NH; ++i) hp[i - 1] = load_raw(t_start - i);
#pragma unroll
        for (int i = NH; i >= 1; --i) {
            pair_rows(hp[i - 1], prev, pe[(-i) & 3]);
            prev = hp[i - 1];
            if (i <= HL - 1) {
                float f[6];
                featurize16<T>(Wa, Wb, pe[(-i) & 3], pe[(-i - 2) & 3], f);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) ur[(-i) & 7][ch] = f[ei<PL, CH>(ch, 1)] * f[ei<PL, CH>(ch, 2)];
            }
        }
    }

    // FB rows are in flight while FB are worked on
    constexpr int FB = PL ? 2 * MIXER_BATCH_FWD16 : MIXER_BATCH_FWD16;     // (planar rows arrive as three small loads each)
    u32x3 in[2][FB];
#pragma unroll
    for (int kk = 0; kk < FB; ++kk) in[0][kk] = load_raw(t_start + kk);
    for (int64_t tb = t_start; tb < t_end; tb += 2 * FB) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int cur = half, nxt = half ^ 1;
#pragma unroll
            for (int kk = 0; kk < FB; ++kk) in[nxt][kk] = load_raw(tb + (half + 1) * FB + kk);
#pragma unroll
            for (int kk = 0; kk < FB; ++kk) {
                const int k = half * FB + kk;
                float f[6], out[CH];
                pair_rows(in[cur][kk], prev, pe[k & 3]);
                prev = in[cur][kk];
                featurize16<T>(Wa, Wb, pe[k & 3], pe[(k - 2) & 3], f);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) {
                    ur[k & 7][ch] = f[ei<PL, CH>(ch, 1)] * f[ei<PL, CH>(ch, 2)];
                    float acc = 0.f;
#pragma unroll
                    for (int j = HL - 1; j >= 0; --j) acc = fmaf(hr[j], ur[(k - j) & 7][ch], acc);
                    out[ch] = f[ei<PL, CH>(ch, 0)] * acc;
                }
                win_store(wy, lane_o + (uint32_t)(tb + k - t_start) * orow, Pair<T>::pack2(out[0], out[1]));
            }
        }
    }
}

// The backward walk above with the featurizer's three sums done two taps (or two rows) at a time.
// d raw lags d f by three rows whatever the filter length (the fourth tap is zero for shorter filters).
template <typename T, int HL, int KF, bool PL = false, typename FT = T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MIXER_WPE)))
void mixer_se_bwd16_kernel(const T *__restrict__ dy, const T *__restrict__ raw, const T *__restrict__ wf,
                           const FT *__restrict__ h, T *__restrict__ draw, float *__restrict__ ws_h,
                           float *__restrict__ ws_w, Dims dm, int kf, MixPlan pl)
{
    typedef Piece<T> P;
    constexpr int ES = 2, CH = 2, E = 6, D1 = HL - 1, D2 = 3, NH = D1 + D2;
    int64_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t L = dm.L, d = dm.d, c = (int64_t)cv * CH;
    const int hl = dm.hl;

    uint32_t Wa[6], Wb[6];
    float hr[HL];
    load_taps16<T, HL, PL, FT>(wf, h, c, dm, kf, Wa, Wb, hr);

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t_stop = t_end + NH;
    const int64_t t0 = t_start - NH > 0 ? t_start - NH : 0;
    const int64_t t_far = t_stop < L ? t_stop : L;
    const uint32_t orow = (uint32_t)(d * ES), irow = 3 * orow;
    const win_t wr = make_window(raw + 3 * (b * L + t0) * d, (t_far - t0) * irow);
    const win_t wdy = make_window(dy + (b * L + t0) * d, (t_far - t0) * orow);
    const win_t wdr = make_window(draw + 3 * (b * L + t_start) * d, (t_end - t_start) * irow);
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = PL ? lane_o : 3 * lane_o;

    // rings, slot = row & (size-1): rp raw rows as loaded; pe = pair_rows(raw[row], raw[row-1]);
    // ur u; gr g2; xs / Bs / dCs f's x, B and dC as elements of T; pd = pair_rows(d f[row-1], d f[row])
    float ur[8][CH], gr[8][CH], dha[HL], dwa[KF][E];
    u32x3 rp[16], dfprev = u32x3{0u, 0u, 0u};
    uint32_t pe[4][6], pd[4][6], xs[8], Bs[8], dCs[8];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int e = 0; e < 6; ++e) { pe[s][e] = 0u; pd[s][e] = 0u; }
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

    // halo on the left (t_start is a multiple of 16)
    {
        u32x3 hp[NH];
#pragma unroll
        for (int i = 1; i <= NH; ++i) hp[i - 1] = piece_load<PL>(wr, lane_i + (uint32_t)(t_start - i - t0) * irow, orow);
#pragma unroll
        for (int i = NH; i >= 1; --i) {
            rp[(-i) & 15] = hp[i - 1];
            pair_rows(rp[(-i) & 15], rp[(-i - 1) & 15], pe[(-i) & 3]);
            if (i <= D1) {
                float f[E];
                featurize16<T>(Wa, Wb, pe[(-i) & 3], pe[(-i - 2) & 3], f);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) ur[(-i) & 7][ch] = f[ei<PL, CH>(ch, 1)] * f[ei<PL, CH>(ch, 2)];
            }
        }
    }

    // Rows are counted from the run's start.  No row of the walk needs a run-time mask:
    //  * before the run, d f comes out zero by itself, because the rings of x, B and dC start at zero;
    //  * a run cut short by the end of the sequence reads zeros there (dy = 0 gives g2 = du = dC = 0);
    //  * a full run ends at row ts, a multiple of 16, so the rows past it are the last iteration of the
    //    walk, and what they may contribute is known when the kernel is compiled (`past` below):
    //    nothing to dh, d f only for 3 rows, dwf only from pairs of rows inside the run.
    const int ts = pl.ts, n_stop = (int)(t_end - t_start) + NH;
    const uint32_t in0 = lane_i + (uint32_t)(t_start - t0) * irow, dy0 = lane_o + (uint32_t)(t_start - t0) * orow;
    // the next batch of rows is in flight while the current one is worked on
    u32x3 in[2][BATCH16];
    uint32_t dyr[2][BATCH16];
    uint32_t vin = in0, vdy = dy0, vout = lane_i - (uint32_t)NH * irow;      // offsets of the next row to load / store
    auto fetch = [&](int slot) {
#pragma unroll
        for (int kk = 0; kk < BATCH16; ++kk) {
            in[slot][kk] = piece_load<PL>(wr, vin, orow);     // zero past t_far
            dyr[slot][kk] = win_load<uint32_t>(wdy, vdy);
            vin += irow;
            vdy += orow;
        }
    };
    // one row of the walk: k = its place in the iteration of 16 (ring slots), past = the iteration after a full run
    auto row = [&](auto past_tag, int k, const u32x3 &inrow, uint32_t dyrow) {
        constexpr bool past = decltype(past_tag)::value;
        const int k1 = k - D1;                                 // the row whose d f completes now
        if (past && k >= NH) return;                           // nothing of these rows reaches the run
        // ---- stage 1: row t
        {
            float f[E], dyf[CH], dCv[CH];
            u32x3 fp;
            rp[k & 15] = inrow;
            pair_rows(rp[k & 15], rp[(k - 1) & 15], pe[k & 3]);
            featurize16<T>(Wa, Wb, pe[k & 3], pe[(k - 2) & 3], f, fp);
            P::unpack_unit(dyrow, dyf);
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) {
                gr[k & 7][ch] = dyf[ch] * f[ei<PL, CH>(ch, 0)];
                ur[k & 7][ch] = f[ei<PL, CH>(ch, 1)] * f[ei<PL, CH>(ch, 2)];
            }
            xs[k & 7] = PL ? (uint32_t)fp[2] : halves<0, 1>(fp[1], fp[2]);          // (x of channel 0, x of channel 1)
            Bs[k & 7] = PL ? (uint32_t)fp[1] : halves<1, 0>(fp[0], fp[2]);          // (B, B)
            float y2v[CH];
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) y2v[ch] = 0.f;
#pragma unroll
            for (int j = HL - 1; j >= 0; --j) {
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) y2v[ch] = fmaf(hr[j], ur[(k - j) & 7][ch], y2v[ch]);
                if (!past)                                   // rows past the run belong to the next run's dh
                    dha[j] = fmaf(gr[k & 7][0], ur[(k - j) & 7][0], fmaf(gr[k & 7][1], ur[(k - j) & 7][1], dha[j]));
            }
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) dCv[ch] = dyf[ch] * y2v[ch];
            dCs[k & 7] = Pair<T>::pack2(dCv[0], dCv[1]);
        }
        // ---- stage 2: d f of row t1 = t - D1, as elements of T; past the run it is wanted for 3 rows
        {
            u32x3 dfp = u32x3{0u, 0u, 0u};
            if (!past || k1 < D2) {
                float du[CH], xo[CH], Bo[CH], dBv[CH], dxv[CH];
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) du[ch] = 0.f;
#pragma unroll
                for (int j = 0; j < HL; ++j)
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) du[ch] = fmaf(hr[j], gr[(k1 + j) & 7][ch], du[ch]);
                P::unpack_unit(xs[k1 & 7], xo);
                P::unpack_unit(Bs[k1 & 7], Bo);
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) {
                    dBv[ch] = du[ch] * xo[ch];
                    dxv[ch] = du[ch] * Bo[ch];
                }
                // the row (dC, dB, dx) x 2 channels, assembled from words of two channels each
                const uint32_t pC = dCs[k1 & 7], pB = Pair<T>::pack2(dBv[0], dBv[1]), pX = Pair<T>::pack2(dxv[0], dxv[1]);
                dfp = PL ? u32x3{pC, pB, pX} : u32x3{halves<0, 0>(pC, pB), halves<0, 1>(pX, pC), halves<1, 1>(pB, pX)};
            }
            pair_rows(dfprev, dfp, pd[k1 & 3]);
            dfprev = dfp;
            // dwf[.., kf-1-j] += d f[t1-1] * raw[t1-1-j] + d f[t1] * raw[t1-j], every second row; runs start
            // and end on even rows, so a pair lies in the run when its first row does
            if ((k1 & 1) != 0 && (!past || k1 - 1 < 0)) {
#pragma unroll
                for (int j = 0; j < KF; ++j) {
                    uint32_t qr[6];
                    pair_rows(rp[(k1 - 1 - j) & 15], rp[(k1 - j) & 15], qr);
#pragma unroll
                    for (int e = 0; e < E; ++e) dwa[j][e] = Pair<T>::dot2(pd[k1 & 3][e], qr[e], dwa[j][e]);
                }
            }
        }
        // ---- stage 3: d raw of row t2 = t1 - 3 from d f of rows t2 .. t2 + 3
        {
            float dr[E];
#pragma unroll
            for (int e = 0; e < E; ++e)
                dr[e] = Pair<T>::dot2(pd[(k1 - 2) & 3][e], Wa[e], Pair<T>::dot2(pd[k1 & 3][e], Wb[e], 0.f));
            piece_store<PL>(wdr, vout, orow, pack6<T>(dr));
            vout += irow;
        }
    };
    fetch(0);
    for (int tb = 0; tb < ts && tb < n_stop; tb += 16) {
#pragma unroll
        for (int q = 0; q < 16 / BATCH16; ++q) {
            fetch((q & 1) ^ 1);
#pragma unroll
            for (int kk = 0; kk < BATCH16; ++kk) row(std::false_type{}, q * BATCH16 + kk, in[q & 1][kk], dyr[q & 1][kk]);
        }
    }
    if (n_stop > ts) {
#pragma unroll
        for (int q = 0; q < (NH + BATCH16 - 1) / BATCH16; ++q) {
            fetch((q & 1) ^ 1);
#pragma unroll
            for (int kk = 0; kk < BATCH16; ++kk) row(std::true_type{}, q * BATCH16 + kk, in[q & 1][kk], dyr[q & 1][kk]);
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
            float *dst = ws_w + ((size_t)(kf - 1 - j) * pl.nrows + prow) * (3 * d) + (PL ? c : 3 * c);
#pragma unroll
            for (int e = 0; e < E; ++e) dst[PL ? (int64_t)(e / CH) * d + e % CH : (int64_t)e] = dwa[j][e];
        }
}

MixPlan plan(const Dims &dm, int ch, bool backward)
{
    MixPlan p;
    p.ch = ch;
    p.nvec = (int)(dm.d / ch);
    // The longest runs that still leave two workgroups per CU: the halo of up to 10 rows each side
    // and the filter-gradient partials cost 9 % of the traffic at 128 rows, 4 % at 512.  The
    // backward, which holds two workgroups per CU at a time, gains nothing beyond 512 rows; the
    // forward does (measured at the 40B shape: 409 us at 512 rows, 383 at 1024).  Multiples of 16
    // (the backward's longest ring) down to 16.
    p.ts = backward ? 512 : 1024;
    while (p.ts > 16 && dm.bs * ((dm.L + p.ts - 1) / p.ts) * p.nvec < 128 * 1024) p.ts >>= 1;
    static const char *env = tuning_env("GCG_MIXER_ROWS");      // tuning override: rows per lane, a multiple of 16
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

// FT: element type of h and dh (float with 16-bit T: fp32 filter and arithmetic on 16-bit tensors)
template <typename T, int HL, int KF, typename FT>
int fwd_launch(const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf, hipStream_t st)
{
    int e = 0;
    const MixPlan p = plan(dm, Piece<T>::CH, false);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if constexpr (sizeof(T) == 2) {
        if (dm.planar)
            e = launch_plain((mixer_se_fwd16_kernel<T, HL, true, FT>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)raw, (const T *)wf, (const FT *)h, (T *)y, dm, kf, p);
        else
            e = launch_plain((mixer_se_fwd16_kernel<T, HL, false, FT>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)raw, (const T *)wf, (const FT *)h, (T *)y, dm, kf, p);
    } else {
        if (dm.planar)
            e = launch_plain((mixer_se_fwd_kernel<T, HL, KF, true>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)raw, (const T *)wf, (const T *)h, (T *)y, dm, kf, p);
        else
            e = launch_plain((mixer_se_fwd_kernel<T, HL, KF>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)raw, (const T *)wf, (const T *)h, (T *)y, dm, kf, p);
    }
    return e;
}

template <typename T, int HL, int KF, typename FT>
int bwd_launch(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh,
               void *ws, const Dims &dm, int kf, hipStream_t st)
{
    int e = 0;
    const MixPlan p = plan(dm, Piece<T>::CH, true);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    float *ws_h = (float *)ws;
    float *ws_w = ws_h + (size_t)dm.hl * p.nrows * p.nvec;
    if constexpr (sizeof(T) == 2) {
        if (dm.planar)
            e = launch_plain((mixer_se_bwd16_kernel<T, HL, KF, true, FT>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)dy, (const T *)raw, (const T *)wf, (const FT *)h, (T *)draw, ws_h, ws_w, dm, kf, p);
        else
            e = launch_plain((mixer_se_bwd16_kernel<T, HL, KF, false, FT>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)dy, (const T *)raw, (const T *)wf, (const FT *)h, (T *)draw, ws_h, ws_w, dm, kf, p);
    } else {
        if (dm.planar)
            e = launch_plain((mixer_se_bwd_kernel<T, HL, KF, true>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)dy, (const T *)raw, (const T *)wf, (const T *)h, (T *)draw, ws_h, ws_w, dm, kf, p);
        else
            e = launch_plain((mixer_se_bwd_kernel<T, HL, KF>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                             (const T *)dy, (const T *)raw, (const T *)wf, (const T *)h, (T *)draw, ws_h, ws_w, dm, kf, p);
    }
    if (e) return e;
    // both filter gradients in one launch
    const ColsumJob jh{ws_h, dh, p.nrows, p.nvec, dm.dg / p.ch, dm.g, dm.hl};
    const ColsumJob jw{ws_w, dwf, p.nrows, 3 * dm.d, 1, (int)(3 * dm.d), kf};
    return (launch_colsum_reduce2<FT, T>(jh, jw, st));
}

template <typename T, int KF, typename FT>
int fwd_k(const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf, hipStream_t st)
{
    if (dm.hl <= 4) return fwd_launch<T, 4, KF, FT>(raw, wf, h, y, dm, kf, st);
    if (dm.hl <= 7) return fwd_launch<T, 7, KF, FT>(raw, wf, h, y, dm, kf, st);
    return fwd_launch<T, 8, KF, FT>(raw, wf, h, y, dm, kf, st);
}
template <typename T, typename FT = T>
int fwd_t(const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf, hipStream_t st)
{
    return kf <= 3 ? fwd_k<T, 3, FT>(raw, wf, h, y, dm, kf, st) : fwd_k<T, 4, FT>(raw, wf, h, y, dm, kf, st);
}
template <typename T, int KF, typename FT>
int bwd_k(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh, void *ws,
          const Dims &dm, int kf, hipStream_t st)
{
    if (dm.hl <= 4) return bwd_launch<T, 4, KF, FT>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    if (dm.hl <= 7) return bwd_launch<T, 7, KF, FT>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    return bwd_launch<T, 8, KF, FT>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
}
template <typename T, typename FT = T>
int bwd_t(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh, void *ws,
          const Dims &dm, int kf, hipStream_t st)
{
    return kf <= 3 ? bwd_k<T, 3, FT>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st)
                   : bwd_k<T, 4, FT>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
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
    case GCG_BF16_F32: return fwd_t<bf16_t, float>(raw, wf, h, y, dm, kf, st);      // h in fp32
    case GCG_F16_F32:  return fwd_t<f16_t, float>(raw, wf, h, y, dm, kf, st);
    }
    return (int)hipErrorInvalidValue;
}

size_t mixer_se_bwd_workspace(int dtype, const Dims &dm, int kf)
{
    const MixPlan p = plan(dm, lane_channels(dtype), true);
    return ((size_t)dm.hl * p.nrows * p.nvec + (size_t)kf * p.nrows * 3 * dm.d) * sizeof(float);
}

int mixer_se_bwd_launch(int dtype, const void *dy, const void *raw, const void *wf, const void *h, void *draw,
                        void *dwf, void *dh, void *ws, const Dims &dm, int kf, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return bwd_t<float>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    case GCG_BF16: return bwd_t<bf16_t>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    case GCG_F16:  return bwd_t<f16_t>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    case GCG_BF16_F32: return bwd_t<bf16_t, float>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);    // h, dh in fp32
    case GCG_F16_F32:  return bwd_t<f16_t, float>(dy, raw, wf, h, draw, dwf, dh, ws, dm, kf, st);
    }
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
