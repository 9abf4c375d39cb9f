// Register sliding-window kernels for short filters (hl <= 8, Hyena-SE).
//
// At 7 taps the operator moves 8 bytes per output for 14 flops, far below the
// machine balance, so there is nothing for the matrix cores to do: each lane owns
// V adjacent channels (one vector load per row) and walks a run of time rows,
// keeping the last 8 rows of the pre-gate product (and, in the backward, of the
// gated upstream gradient and the raw x / B rows) in a register ring whose slot
// indices are compile-time after unrolling by 8.  Adjacent lanes take adjacent
// channel vectors, so every row access of a wave is one contiguous segment.
#include "gcg_rowvec.h"

#include <cstdlib>

namespace gcg {
namespace {

constexpr int RING = 8;
constexpr int BATCH = 4;   // rows fetched together
constexpr int HALO_BURST = 4;   // halo rows fetched together


// Interleaved operands (element stride 3): a lane's V channels of one row are 3V consecutive
// elements, (C, B, x) per channel, i.e. three raw vectors.  split3 / join3 convert between
// that order and per-tensor channel vectors; every index is a compile-time constant.
template <typename T, int V>
__device__ __forceinline__ void split3(const typename Vec<T, V>::raw (&p)[3], float (&xf)[V], float (&Bf)[V],
                                       float (&Cf)[V])
{
    float f[3][V];
#pragma unroll
    for (int i = 0; i < 3; ++i) unpackv<T, V>(p[i], f[i]);
#pragma unroll
    for (int v = 0; v < V; ++v) {
        Cf[v] = f[(3 * v) / V][(3 * v) % V];
        Bf[v] = f[(3 * v + 1) / V][(3 * v + 1) % V];
        xf[v] = f[(3 * v + 2) / V][(3 * v + 2) % V];
    }
}
template <typename T, int V>
__device__ __forceinline__ void join3(const float (&xf)[V], const float (&Bf)[V], const float (&Cf)[V],
                                      typename Vec<T, V>::raw (&p)[3])
{
    float f[3][V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        f[(3 * v) / V][(3 * v) % V] = Cf[v];
        f[(3 * v + 1) / V][(3 * v + 1) % V] = Bf[v];
        f[(3 * v + 2) / V][(3 * v + 2) % V] = xf[v];
    }
#pragma unroll
    for (int i = 0; i < 3; ++i) p[i] = packv<T, V>(f[i]);
}

// One input row of a lane: three raw vectors, (x, B, C) of separate tensors or the three
// thirds of the interleaved row.
template <typename T, int V, bool PK>
__device__ __forceinline__ void row_floats(const typename Vec<T, V>::raw (&p)[3], float (&xf)[V], float (&Bf)[V],
                                           float (&Cf)[V])
{
    if constexpr (PK) {
        split3<T, V>(p, xf, Bf, Cf);
    } else {
        unpackv<T, V>(p[0], xf);
        unpackv<T, V>(p[1], Bf);
        unpackv<T, V>(p[2], Cf);
    }
}

struct WinPlan { int v, nvec, nseg, ts, ncvb, threads; int64_t nthreads, nwg; };


// ---------------------------------------------------------------------------- forward
// PK: x, B, C are interleaved in one tensor that starts at C (element stride 3).
// EXTRA: also write the convolution before the post-gate (y2) and the pre-gate product (bx).
// Tensors are addressed through windows over the rows of this run, so no load or store sits
// behind a branch: rows before the sequence start read as zero, rows past the run are dropped.
template <typename T, int HL, int V, bool PK, bool EXTRA>
__global__ __launch_bounds__(256) void window_fwd_kernel(const T *__restrict__ x, const T *__restrict__ B,
                                                         const T *__restrict__ C, const T *__restrict__ h,
                                                         T *__restrict__ y, T *__restrict__ y2,
                                                         T *__restrict__ bx, Dims dm, WinPlan pl)
{
    typedef typename Vec<T, V>::raw raw_t;
    constexpr int ES = sizeof(T), IS = PK ? 3 : 1;     // element bytes, element stride of the inputs
    // (batch, run, block of channel vectors) come from the workgroup index, so row offsets
    // are wave-uniform and only the channel offset is per lane
    int64_t wg = blockIdx.x;
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t L = dm.L, d = dm.d;
    const int64_t c = (int64_t)cv * V;
    const int hl = dm.hl;
    typedef typename Filt<T>::type FT;           // element type of the filter
    const FT *hg = (const FT *)h + (c / dm.dg) * hl;

    float hr[HL];  // hr[j] multiplies the sample j rows in the past
#pragma unroll
    for (int j = 0; j < HL; ++j) hr[j] = (j < hl) ? Elem<FT>::load(hg + hl - 1 - j) : 0.f;

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t0 = t_start - (HL - 1) > 0 ? t_start - (HL - 1) : 0;       // first row of the windows
    const int64_t origin = (b * L + t0) * d, rows = t_end - t0;
    // time-major inputs: the rows of this batch entry lie bs rows apart (a window then spans the other
    // entries' rows in between, which no offset of this lane reaches)
    // planar inputs: the thirds of rows of 3 d elements (a window then spans the other thirds in between as well)
    const int64_t in_origin = dm.tmajor ? (t0 * dm.bs + b) * d : dm.planar ? 3 * origin : origin;
    const uint32_t orow = (uint32_t)(d * ES), irow = IS * orow * (uint32_t)(dm.tmajor ? dm.bs : dm.planar ? 3 : 1);   // bytes per row: outputs, inputs
    const win_t wx = make_window((PK ? C : x) + IS * in_origin, rows * irow);
    const win_t wB = make_window(B + in_origin, PK ? 0 : rows * irow), wC = make_window(C + in_origin, PK ? 0 : rows * irow);
    const win_t wy = make_window(y + origin, rows * orow);
    const win_t wy2 = make_window(EXTRA && y2 ? y2 + origin : y + origin, EXTRA && y2 ? rows * orow : 0);
    const win_t wbx = make_window(EXTRA && bx ? bx + origin : y + origin, EXTRA && bx ? rows * orow : 0);
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = IS * lane_o;
    auto load_in = [&](int64_t t, raw_t (&p)[3], bool with_c) {
        const uint32_t o = lane_i + (uint32_t)(t - t0) * irow;
        if constexpr (PK) {
            load_piece(wx, o, p);
        } else {
            p[0] = win_load<raw_t>(wx, o);
            p[1] = win_load<raw_t>(wB, o);
            p[2] = with_c ? win_load<raw_t>(wC, o) : zero_raw<T, V>();
        }
    };

    float ring[RING][V];
#pragma unroll
    for (int s = 0; s < RING; ++s)
#pragma unroll
        for (int v = 0; v < V; ++v) ring[s][v] = 0.f;
    // halo: rows t_start-(HL-1) .. t_start-1 go to slots (t & 7); t_start is a multiple of 8
    // (fetched HALO_BURST rows at a time, so the staging registers stay below the main loop's)
#pragma unroll
    for (int i0 = 1; i0 < HL; i0 += HALO_BURST) {
        raw_t halo[HALO_BURST][3];
#pragma unroll
        for (int i = i0; i < i0 + HALO_BURST && i < HL; ++i) load_in(t_start - i, halo[i - i0], false);
#pragma unroll
        for (int i = i0; i < i0 + HALO_BURST && i < HL; ++i) {
            float xf[V], Bf[V], Cf[V];
            row_floats<T, V, PK>(halo[i - i0], xf, Bf, Cf);
#pragma unroll
            for (int v = 0; v < V; ++v) ring[RING - i][v] = xf[v] * Bf[v];
        }
    }

    // Rows are fetched BATCH at a time.  At 16 bits one batch ahead: while a batch is worked on,
    // the loads of the next are in flight (past the run they fall outside the windows and cost
    // nothing).  At fp32 the second staging buffer would cost a wave per SIMD; measured slower.
    constexpr bool AHEAD = sizeof(T) == 2;
    raw_t in[AHEAD ? 2 : 1][BATCH][3];
    if constexpr (AHEAD) {
#pragma unroll
        for (int kk = 0; kk < BATCH; ++kk) load_in(t_start + kk, in[0][kk], true);
    }
    for (int64_t tb = t_start; tb < t_end; tb += RING) {
#pragma unroll
        for (int half = 0; half < RING / BATCH; ++half) {
            constexpr int NB = RING / BATCH;
            const int cur = AHEAD ? half % 2 : 0, nxt = AHEAD ? (half + 1) % 2 : 0;
            static_assert(NB % 2 == 0, "the staging buffers alternate with the batches of a ring turn");
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk)
                load_in(tb + (half + (AHEAD ? 1 : 0)) * BATCH + kk, in[nxt][kk], true);
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const int k = half * BATCH + kk;
                const int64_t t = tb + k;
                float xf[V], Bf[V], Cf[V], acc[V], out[V];
                row_floats<T, V, PK>(in[cur][kk], xf, Bf, Cf);
#pragma unroll
                for (int v = 0; v < V; ++v) { ring[k][v] = xf[v] * Bf[v]; acc[v] = 0.f; }
#pragma unroll
                for (int j = HL - 1; j >= 0; --j)
#pragma unroll
                    for (int v = 0; v < V; ++v) acc[v] = fmaf(hr[j], ring[(k - j) & (RING - 1)][v], acc[v]);
                const uint32_t o = lane_o + (uint32_t)(t - t0) * orow;
                if constexpr (EXTRA) {
                    win_store(wy2, o, packv<T, V>(acc));
                    win_store(wbx, o, packv<T, V>(ring[k]));
                }
#pragma unroll
                for (int v = 0; v < V; ++v) out[v] = Cf[v] * acc[v];
                win_store(wy, o, packv<T, V>(out));
            }
        }
    }
}

// --------------------------------------------------------------------------- backward
// Per lane: rows [t_start, t_end).  Row r is loaded at step r; dC[r] and the dh terms
// of row r are produced at once (they look back), du[r-(HL-1)] is produced at step r
// (it looks forward), so the walk runs HL-1 rows past t_end reading only dy and C.
// PK: x, B, C are interleaved in one tensor that starts at C, and dx, dB, dC in one that starts
// at dC.  A row of the output then holds dC (ready at step r) next to dx, dB (ready HL-1 steps
// later), so dC waits in a register ring like the raw x and B rows do.
// Windows: x and B end with the run, dy and C HL-1 rows later, the outputs start with the run;
// every row outside reads as zero or is dropped, so the walk has no branch around an access.
// (occupancy floor: three workgroups per CU at 16 bits, two at fp32, so that the scheduler
// does not trade waves for longer load batches)
template <typename T, int HL, int V, bool PK, bool KEEP>
__global__ __launch_bounds__(256) void window_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                         const T *__restrict__ B, const T *__restrict__ C,
                                                         const T *__restrict__ h, T *__restrict__ dx,
                                                         T *__restrict__ dB, T *__restrict__ dC,
                                                         float *__restrict__ ws, Dims dm, WinPlan pl)
{
    typedef typename Vec<T, V>::raw raw_t;
    constexpr int ES = sizeof(T), IS = PK ? 3 : 1;
    // workgroups of one XCD take adjacent channel blocks of the same rows (measured +3-5 % in the
    // backward kernels, -3 % in the forward ones, which keep the plain order)
    int64_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int cvb = (int)(wg % pl.ncvb); wg /= pl.ncvb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= pl.nvec) return;
    const int64_t gid = (b * pl.nseg + seg) * pl.nvec + cv;     // index of this lane's workspace slot
    const int64_t L = dm.L, d = dm.d;
    const int64_t c = (int64_t)cv * V;
    const int hl = dm.hl;
    typedef typename Filt<T>::type FT;           // element type of the filter
    const FT *hg = (const FT *)h + (c / dm.dg) * hl;

    float hr[HL];
#pragma unroll
    for (int j = 0; j < HL; ++j) hr[j] = (j < hl) ? Elem<FT>::load(hg + hl - 1 - j) : 0.f;

    const int64_t t_start = (int64_t)seg * pl.ts;
    const int64_t t_end = (t_start + pl.ts < L) ? t_start + pl.ts : L;
    const int64_t t_stop = t_end + (HL - 1);                     // exclusive bound of the walk
    const int64_t t0 = t_start - (HL - 1) > 0 ? t_start - (HL - 1) : 0;
    const int64_t t_far = t_stop < L ? t_stop : L;
    const int64_t origin = (b * L + t0) * d;
    // time-major x, B, C, dx, dB, dC: the rows of this batch entry lie bs rows apart
    // (planar x, B, C, dx, dB, dC: the thirds of rows of 3 d elements)
    const int64_t in_origin = dm.tmajor ? (t0 * dm.bs + b) * d : dm.planar ? 3 * origin : origin;
    const int64_t out_origin = dm.tmajor ? (t_start * dm.bs + b) * d : (b * L + t_start) * d * (dm.planar ? 3 : 1);
    const uint32_t orow = (uint32_t)(d * ES), irow = IS * orow * (uint32_t)(dm.tmajor ? dm.bs : dm.planar ? 3 : 1);
    // PK: wx is the interleaved tensor and reaches as far as dy (C is part of it)
    const win_t wx = make_window((PK ? C : x) + IS * in_origin, ((PK ? t_far : t_end) - t0) * irow);
    const win_t wB = make_window(B + in_origin, PK ? 0 : (t_end - t0) * irow);
    const win_t wC = make_window(C + in_origin, PK ? 0 : (t_far - t0) * irow);
    const win_t wdy = make_window(dy + origin, (t_far - t0) * orow);
    const win_t wdC = make_window(dC + IS * out_origin, (t_end - t_start) * irow);
    const win_t wdx = make_window(dx + out_origin, PK ? 0 : (t_end - t_start) * irow);
    const win_t wdB = make_window(dB + out_origin, PK ? 0 : (t_end - t_start) * irow);
    const uint32_t lane_o = (uint32_t)(c * ES), lane_i = IS * lane_o;

    float ur[RING][V], gr[RING][V], dha[HL];
    raw_t xs[RING], Bs[RING], dCs[PK ? RING : 1];
#pragma unroll
    for (int s = 0; s < RING; ++s) {
        xs[s] = zero_raw<T, V>(); Bs[s] = zero_raw<T, V>();
        if constexpr (PK) dCs[s] = zero_raw<T, V>();
#pragma unroll
        for (int v = 0; v < V; ++v) { ur[s][v] = 0.f; gr[s][v] = 0.f; }
    }
#pragma unroll
    for (int j = 0; j < HL; ++j) dha[j] = 0.f;
#pragma unroll
    for (int i0 = 1; i0 < HL; i0 += HALO_BURST) {
        raw_t halo[HALO_BURST][3];
#pragma unroll
        for (int i = i0; i < i0 + HALO_BURST && i < HL; ++i) {
            const uint32_t o = lane_i + (uint32_t)(t_start - i - t0) * irow;
            if constexpr (PK) {
                load_piece(wx, o, halo[i - i0]);
            } else {
                halo[i - i0][0] = win_load<raw_t>(wx, o);
                halo[i - i0][1] = win_load<raw_t>(wB, o);
                halo[i - i0][2] = zero_raw<T, V>();
            }
        }
#pragma unroll
        for (int i = i0; i < i0 + HALO_BURST && i < HL; ++i) {
            float xf[V], Bf[V], Cf[V];
            row_floats<T, V, PK>(halo[i - i0], xf, Bf, Cf);
#pragma unroll
            for (int v = 0; v < V; ++v) ur[RING - i][v] = xf[v] * Bf[v];
        }
    }

    for (int64_t tb = t_start; tb < t_stop; tb += RING) {
#pragma unroll
        for (int half = 0; half < RING / BATCH; ++half) {
            // rows are fetched BATCH at a time into staging registers; the x / B rings are only
            // overwritten slot by slot below, after the delayed du row has read them
            raw_t dyr[BATCH], in[BATCH][3];
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const int64_t t = tb + half * BATCH + kk;
                const uint32_t o = lane_i + (uint32_t)(t - t0) * irow;
                if constexpr (PK) {
                    load_piece(wx, o, in[kk]);
                } else {
                    in[kk][0] = win_load<raw_t>(wx, o);
                    in[kk][1] = win_load<raw_t>(wB, o);
                    in[kk][2] = win_load<raw_t>(wC, o);
                }
                dyr[kk] = win_load<raw_t>(wdy, lane_o + (uint32_t)(t - t0) * orow);
            }
#pragma unroll
            for (int kk = 0; kk < BATCH; ++kk) {
                const int k = half * BATCH + kk;
                const int64_t t = tb + k;
                const bool in_run = t < t_end;          // uniform; past the run only g2 is wanted
                float dyf[V], xf[V], Bf[V], Cf[V];
                unpackv<T, V>(dyr[kk], dyf);
                row_floats<T, V, PK>(in[kk], xf, Bf, Cf);
                if constexpr (PK) {
                    xs[k] = packv<T, V>(xf);
                    Bs[k] = packv<T, V>(Bf);
                } else {
                    xs[k] = in[kk][0];
                    Bs[k] = in[kk][1];
                }
#pragma unroll
                for (int v = 0; v < V; ++v) gr[k][v] = dyf[v] * Cf[v];
                {
                    float y2v[V], o[V], gd[V];
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        ur[k][v] = in_run ? xf[v] * Bf[v] : 0.f;
                        gd[v] = in_run ? gr[k][v] : 0.f;     // rows past the run belong to the next run's dh
                        y2v[v] = 0.f;
                    }
#pragma unroll
                    for (int j = HL - 1; j >= 0; --j) {
                        float sacc = 0.f;
#pragma unroll
                        for (int v = 0; v < V; ++v) {
                            const float u = ur[(k - j) & (RING - 1)][v];
                            y2v[v] = fmaf(hr[j], u, y2v[v]);
                            sacc = fmaf(gd[v], u, sacc);
                        }
                        dha[j] += sacc;
                    }
#pragma unroll
                    for (int v = 0; v < V; ++v) o[v] = dyf[v] * y2v[v];
                    if constexpr (PK) dCs[k] = packv<T, V>(o);
                    else win_store(wdC, lane_o + (uint32_t)(t - t_start) * irow, packv<T, V>(o));
                }
                // du for row t-(HL-1): sum_j hr[j] * g2[row + j]; rows before the run fall outside
                // the output windows
                {
                    const int64_t out_t = t - (HL - 1);
                    float du[V], xo[V], Bo[V], o[V];
#pragma unroll
                    for (int v = 0; v < V; ++v) du[v] = 0.f;
#pragma unroll
                    for (int j = 0; j < HL; ++j)
#pragma unroll
                        for (int v = 0; v < V; ++v)
                            du[v] = fmaf(hr[j], gr[(k - (HL - 1) + j) & (RING - 1)][v], du[v]);
                    unpackv<T, V>(xs[(k - (HL - 1)) & (RING - 1)], xo);
                    unpackv<T, V>(Bs[(k - (HL - 1)) & (RING - 1)], Bo);
                    if constexpr (PK) {
                        float oB[V], oC[V];
                        raw_t p[3];
#pragma unroll
                        for (int v = 0; v < V; ++v) { o[v] = du[v] * Bo[v]; oB[v] = du[v] * xo[v]; }
                        unpackv<T, V>(dCs[(k - (HL - 1)) & (RING - 1)], oC);
                        join3<T, V>(o, oB, oC, p);
                        const uint32_t q = lane_i + (uint32_t)(out_t - t_start) * irow;
                        if constexpr (KEEP) store_piece_as<true>(wdC, q, p);
                        else store_piece(wdC, q, p);
                    } else {
                        const uint32_t q = lane_o + (uint32_t)(out_t - t_start) * irow;
#pragma unroll
                        for (int v = 0; v < V; ++v) o[v] = du[v] * Bo[v];
                        win_store(wdx, q, packv<T, V>(o));
#pragma unroll
                        for (int v = 0; v < V; ++v) o[v] = du[v] * xo[v];
                        win_store(wdB, q, packv<T, V>(o));
                    }
                }
            }
        }
    }
    // per-lane filter-gradient partials, tap-major so the reducer reads rows
    float *slot = ws + gid;
#pragma unroll
    for (int j = 0; j < HL; ++j)
        if (j < hl) slot[(size_t)(hl - 1 - j) * pl.nthreads] = dha[j];
}

WinPlan plan(const Dims &dm, int v)
{
    WinPlan p;
    p.v = v;
    p.nvec = (int)(dm.d / v);
    p.ts = 1024;
    // the longest runs (up to 1024 rows) that still leave two workgroups per CU: measured best at the
    // 7B and 40B shapes for either operand layout (fewer halo rows and filter-gradient partials;
    // one step further and the machine is no longer covered)
    while (p.ts > 8 && dm.bs * ((dm.L + p.ts - 1) / p.ts) * p.nvec < 128 * 1024) p.ts >>= 1;
    static const char *env = tuning_env("GCG_WINDOW_ROWS");   // tuning override: rows per lane, a multiple of 8
    if (env && atoi(env) >= 8 && atoi(env) % 8 == 0) p.ts = atoi(env);
    // the rows of a run, its halo and an interleaved fp32 row width must fit one tensor window
    while (p.ts > 8 && (int64_t)(p.ts + 2 * RING) * 3 * dm.d * 4 * (dm.tmajor ? dm.bs : 1) > WIN_MAX_BYTES) p.ts >>= 1;   // (planar rows are 3 d wide too)
    p.nseg = (int)((dm.L + p.ts - 1) / p.ts);
    p.nthreads = dm.bs * p.nseg * p.nvec;       // workspace slots (one per lane with work)
    p.threads = p.nvec >= 256 ? 256 : ((p.nvec + 63) / 64) * 64;   // narrow tensors: fewer idle lanes
    p.ncvb = (p.nvec + p.threads - 1) / p.threads;
    p.nwg = dm.bs * p.nseg * p.ncvb;
    return p;
}

constexpr int BWD_V = 4;   // the backward keeps four rings per lane: 4 channels is what fits
// interleaved operands: the lane width that makes a row piece 12 contiguous bytes
template <typename T> constexpr int il_v() { return 4 / (int)sizeof(T); }

template <typename T, int HL, int V>
int fwd_v(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
          const Dims &dm, hipStream_t st)
{
    int e = 0;
    if (dm.es == 3) {
        constexpr int VI = il_v<T>();
        const WinPlan p = plan(dm, VI);
        if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
        e = launch_main((window_fwd_kernel<T, HL, VI, true, false>), dim3((unsigned)p.nwg), dim3(p.threads), st,
                           (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
        return e;
    }
    const WinPlan p = plan(dm, V);
    const int64_t nwg = p.nwg;
    if (nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (y2 || bx)
        e = launch_main((window_fwd_kernel<T, HL, V, false, true>), dim3((unsigned)nwg), dim3(p.threads), st,
                           (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    else
        e = launch_main((window_fwd_kernel<T, HL, V, false, false>), dim3((unsigned)nwg), dim3(p.threads), st,
                           (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    return e;
}

template <typename T, int HL>
int bwd_t(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
          void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    int e = 0;
    const WinPlan p = plan(dm, dm.es == 3 ? il_v<T>() : BWD_V);
    const int64_t nwg = p.nwg;
    if (nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (dm.es == 3 && dm.keep_out)
        e = launch_main((window_bwd_kernel<T, HL, il_v<T>(), true, true>), dim3((unsigned)nwg), dim3(p.threads),
                           st, (const T *)dy, (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)dx, (T *)dB,
                           (T *)dC, (float *)ws, dm, p);
    else if (dm.es == 3)
        e = launch_main((window_bwd_kernel<T, HL, il_v<T>(), true, false>), dim3((unsigned)nwg), dim3(p.threads),
                           st, (const T *)dy, (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)dx, (T *)dB,
                           (T *)dC, (float *)ws, dm, p);
    else
        e = launch_main((window_bwd_kernel<T, HL, BWD_V, false, false>), dim3((unsigned)nwg), dim3(p.threads), st,
                           (const T *)dy, (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)dx, (T *)dB,
                           (T *)dC, (float *)ws, dm, p);
    if (e) return e;
    // partials are ws[tap][(batch, run)][lane]; a filter owns dg / v adjacent lanes
    typedef typename Filt<T>::type FT;
    return launch_colsum_reduce<FT>((const float *)ws, (FT *)dh, dm.bs * p.nseg, p.nvec, dm.dg / p.v, dm.g, dm.hl, st);
}

// Four channels per lane in both directions.  Eight (16-byte vectors for the 16-bit types) was
// measured slower at the 40B shape: half as many lanes in flight outweighs the wider access.
template <typename T, int HL>
int fwd_t(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
          const Dims &dm, hipStream_t st)
{
    return fwd_v<T, HL, 4>(x, B, C, h, y, y2, bx, dm, st);
}

template <typename T>
int fwd_hl(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
           const Dims &dm, hipStream_t st)
{
    if (dm.hl <= 4) return fwd_t<T, 4>(x, B, C, h, y, y2, bx, dm, st);
    if (dm.hl <= 7) return fwd_t<T, 7>(x, B, C, h, y, y2, bx, dm, st);
    return fwd_t<T, 8>(x, B, C, h, y, y2, bx, dm, st);
}

template <typename T>
int bwd_hl(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
           void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    if (dm.hl <= 4) return bwd_t<T, 4>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dm.hl <= 7) return bwd_t<T, 7>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    return bwd_t<T, 8>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
}

} // namespace

bool window_supported(const Dims &dm)
{
    return dm.hl <= RING && dm.dg % 4 == 0 && (int64_t)dm.g * dm.hl <= 0x7fffffffLL &&
           (int64_t)(3 * RING) * 3 * dm.d * 4 * (dm.tmajor ? dm.bs : 1) <= WIN_MAX_BYTES && !(dm.tmajor && dm.es == 3) &&
           !(dm.planar && (dm.es == 3 || dm.tmajor));
}

int window_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h, void *y,
                      void *y2, void *bx, const Dims &dm, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return fwd_hl<float>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_BF16: return fwd_hl<bf16_t>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_F16:  return fwd_hl<f16_t>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_BF16_F32: return fwd_hl<bf16w_t>(x, B, C, h, y, y2, bx, dm, st);
    case GCG_F16_F32:  return fwd_hl<f16w_t>(x, B, C, h, y, y2, bx, dm, st);
    }
    return (int)hipErrorInvalidValue;
}

// one figure for the separate-tensor backward (4 channels per lane) and the interleaved one
// (2 or 1) of every element type: the largest of the three plans
size_t window_bwd_workspace(const Dims &dm)
{
    int64_t n = 0;
    for (int v : {1, 2, BWD_V}) {
        if (dm.d % v) continue;
        const WinPlan p = plan(dm, v);
        if (p.nthreads > n) n = p.nthreads;
    }
    return (size_t)n * dm.hl * sizeof(float);
}

int window_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C, const void *h,
                      void *dx, void *dB, void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    switch (dtype) {
    case GCG_F32:  return bwd_hl<float>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_BF16: return bwd_hl<bf16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_F16:  return bwd_hl<f16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_BF16_F32: return bwd_hl<bf16w_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case GCG_F16_F32:  return bwd_hl<f16w_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    }
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
