// Banded Toeplitz GEMM on the matrix cores (bf16 / f16 / fp32 I/O, fp32 accumulate, hl <= 128).
//
// Streaming form of the two-pass chunked convolution.  A workgroup of NW waves owns 16*NW
// adjacent channels of one batch row and walks a run of time steps of 32 rows.  Wave w owns
// the 16 channels [16w, 16w+16) -- one filter -- and computes, per step, the transposed
// output tile  Y2^T (16 channels x 32 times) = sum_i  U_{s-i}^T (16 x 32)  *  W_i (32 x 32)
// on the matrix cores, where U_{s-i} is the pre-gate product of step s-i and W_i the slice of
// the banded Toeplitz matrix of the filter at time offset 32*i.  The NK = 5 slices (10 operand
// tiles of 16 output times) live in registers for the whole walk, and the last NK operand
// tiles of U are carried in registers, so the "carry from the previous chunk" of the two-pass
// form never goes back to memory: q, k, v are read once and y written once.
//
// Memory side: the waves load each 32-row tile with full rows (32*NW bytes at 16 bits), form
// u = x*B in registers, park it row-major in LDS, and every wave fetches its matrix operand
// from there.  The fp32 result tile returns through LDS to the row layout, is gated with C in
// fp32 and stored with full rows.
//
// Element types.  bf16 / f16: v_mfma_f32_16x16x32; the operand (8 consecutive time samples of
// one channel per lane) comes from the transposing LDS read ds_read_b64_tr_b16.  fp32: every
// operand is split into three bf16 planes whose sum is the fp32 value, the planes sit side by
// side in the LDS tiles, and the same 32-deep product is six bf16 matrix instructions (the
// plane pairs that matter to 2^-24), accumulated in fp32: fp32 accuracy at 3/8 of the matrix
// time of the fp32 instructions.  Memory traffic stays fp32.
#include "gcg_mfma_tile.h"

namespace gcg {
namespace {

// Per-workgroup timestamps of the 100 MHz constant clock, for builds with -DGCG_TRACE only (`make trace`):
// thread 0 of every workgroup stamps slot k of its 16 at the marked points of both kernels.  The stamp is a
// store through a window that only thread 0's offset falls into, so that no branch is put between a load and its use.
#ifdef GCG_TRACE
constexpr int TRACE_WGS = 1 << 16, TRACE_SLOTS = 16;
__device__ unsigned long long g_trace[(size_t)TRACE_WGS * TRACE_SLOTS];
#define TR_INIT const win_t tr_win = make_window(g_trace + (size_t)(blockIdx.x < TRACE_WGS ? blockIdx.x : 0) * TRACE_SLOTS, TRACE_SLOTS * 8)
// -DGCG_TRACE=1: start, walk start, walk end and end only (the forward is sensitive to more); =2: every mark
#define TR(k) do { if (GCG_TRACE >= 2 || (k) == 0 || (k) == 5 || (k) == 6 || (k) == 7) { const unsigned long long t_ = wall_clock64(); \
        __builtin_amdgcn_raw_buffer_store_b64(u32x2{(uint32_t)t_, (uint32_t)(t_ >> 32)}, tr_win, \
                                              threadIdx.x == 0 ? (k) * 8 : (int)WIN_OFF, 0, 0); } } while (0)
// a stamp in slot k on the iteration for which `cond` holds (no branch: the other iterations' offsets miss the window)
#define TR_IF(cond, k) do { if (GCG_TRACE >= 2) { const unsigned long long t_ = wall_clock64(); \
        __builtin_amdgcn_raw_buffer_store_b64(u32x2{(uint32_t)t_, (uint32_t)(t_ >> 32)}, tr_win, \
                                              (threadIdx.x == 0 && (cond)) ? (k) * 8 : (int)WIN_OFF, 0, 0); } } while (0)
#else
#define TR_INIT do { } while (0)
#define TR(k) do { } while (0)
#define TR_IF(cond, k) do { } while (0)
#endif

// Cache policy of the output stores (tuning builds may override).  Measured at the 7B layer shape, against the
// nontemporal hint alone (92.4 and 172.1 us): forward with device-scope stores (sc1: written through the XCD's L2,
// no dirty lines left for the end of the kernel) 90.2 us on 16-bit tensors (89.9 - 90.1 where the output buffer is the
// same from call to call, 1 - 1.5 us less than the hint alone where it is not), with both hints 92.8; fp32 tensors
// lose with it (212 -> 260 us) and keep the hint.  Backward: both hints 171.1 or 176.1 by the box, sc1 alone 179.6; the
// hint alone stays.
#ifndef GCG_MFMA_FWD_ST
#define GCG_MFMA_FWD_ST 16
#endif
#ifndef GCG_MFMA_BWD_ST
#define GCG_MFMA_BWD_ST WIN_NT_ST
#endif
#ifndef GCG_MFMA_BWD_ST_DC
#define GCG_MFMA_BWD_ST_DC GCG_MFMA_BWD_ST
#endif
#ifndef GCG_MFMA_FWD_LD
#define GCG_MFMA_FWD_LD WIN_NT
#endif
#ifndef GCG_MFMA_FWD_LEAD_LD
#define GCG_MFMA_FWD_LEAD_LD WIN_NT
#endif
// Idle cycles in front of each output store of the backward's long runs (tuning builds may override).  Measured
// at the 7B layer shape (2 x 8192 x 4096, bf16): 0 cycles 172.3 - 173.8 us, 16: 171.0, 24: 169.5, 32: 167.3 - 170.4,
// 36 - 40: 165.5 - 169.8 (by the box), 48: 168.5 - 171.1, 64: 178; at 1 x 32768 x 8192 24 - 32 cycles gain 1 %, more
// gains nothing; runs of 16 steps lose 2 % with any.  The stores of a step leave while its workgroup's next rows are
// still on their way, and a little later is better for those.
#ifndef GCG_MFMA_BWD_ST_GAP
#define GCG_MFMA_BWD_ST_GAP 36
#endif
#ifndef GCG_MFMA_BWD_LD
#define GCG_MFMA_BWD_LD WIN_NT
#endif

// ---------------------------------------------------------------------------- forward
// EXTRA: also write the convolution before the post-gate (y2o) and the pre-gate product (bxo).
// PL: x, B, C are the thirds of the rows of one (bs, L, 3 d) tensor (Dims::planar): their rows lie 3 d elements apart.
template <typename T, int NK, int NW, bool EXTRA, bool PL = false>
__global__ __launch_bounds__(64 * NW) void mfma_fwd_kernel(const T *__restrict__ x, const T *__restrict__ B,
                                                       const T *__restrict__ C, const T *__restrict__ h,
                                                       T *__restrict__ y, T *__restrict__ y2o,
                                                       T *__restrict__ bxo, Dims dm, MfmaPlan pl)
{
    typedef MT<T> M;
    typedef typename M::op_t op_t;
    typedef typename M::hraw_t hraw_t;
    typedef Geo<T, NW> G;
    constexpr int CB = G::CB, UROW = G::UROW, YROW = G::YROW, ES = M::ES;
    // LDS: filter tables | u tile of the current step | fp32 result tile.  Before the walk the NK-1
    // lead-in tiles of u lie side by side from the u tile on (over the result tile, not yet in use).
    constexpr int NLEAD_T = NK > 1 ? NK - 1 : 0;
    constexpr int OFF_U = (NW * HTAB * (int)sizeof(hraw_t) + 15) & ~15, OFF_Y = OFF_U + STEP * UROW;
    constexpr int LDS_WALK = STEP * UROW + STEP * YROW, LDS_LEAD = NLEAD_T * STEP * UROW;
    __shared__ __attribute__((aligned(16))) unsigned char smem[OFF_U + (LDS_WALK > LDS_LEAD ? LDS_WALK : LDS_LEAD)];
    unsigned char *u_rm = smem + OFF_U, *y_st = smem + OFF_Y;
    hraw_t (*htab)[HTAB] = (hraw_t (*)[HTAB])smem;
    TR_INIT;
    TR(0);

    int cb, seg, bi;
    wg_place(pl.xcd ? xcd_contiguous_u32(blockIdx.x, gridDim.x) : blockIdx.x, pl, cb, seg, bi);
    const int64_t b = bi;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int r = tid / G::LPR, a = tid % G::LPR;   // row layout: row r of the step, channels 8a..8a+7
    const int j = l & 15, q = l >> 4;               // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;

    // Windows over rows [t0, t1) of this batch row; a lane's offset is lane_off + step_off(s).
    const int64_t t0 = (s_lo - (NK - 1)) * STEP > 0 ? (s_lo - (NK - 1)) * STEP : 0;
    const int64_t t1 = s_hi * STEP < L ? s_hi * STEP : L;
    const int64_t row_bytes = d * ES, win_bytes = (t1 - t0) * row_bytes;
    const int64_t origin = (b * L + t0) * d;
    constexpr int IM = PL ? 3 : 1;                  // row stride of x, B, C in rows of y
    const win_t wx = make_window(x + IM * origin, IM * win_bytes), wB = make_window(B + IM * origin, IM * win_bytes);
    const win_t wC = make_window(C + IM * origin, IM * win_bytes), wy = make_window(y + origin, win_bytes);
    const win_t wy2 = make_window(EXTRA && y2o ? y2o + origin : y + origin, EXTRA && y2o ? win_bytes : 0);
    const win_t wbx = make_window(EXTRA && bxo ? bxo + origin : y + origin, EXTRA && bxo ? win_bytes : 0);
    const uint32_t lane_off = (uint32_t)(r * row_bytes + (c0 + 8 * a) * ES) + (c0 + 8 * a < d ? 0u : WIN_OFF);
    const uint32_t lane_in = PL ? (uint32_t)(r * IM * row_bytes + (c0 + 8 * a) * ES) + (c0 + 8 * a < d ? 0u : WIN_OFF) : lane_off;
    auto step_off = [&](int64_t s) { return (uint32_t)((s * STEP - t0) * row_bytes); };

    op_t A[NK];            // A[(ph - i + NK) % NK]: operand of step s-i while step s runs in phase ph
#pragma unroll
    for (int i = 0; i < NK; ++i) A[i] = M::zero_op();

    unsigned char *u_wr = u_rm + r * UROW + 8 * M::LES * a;
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    const unsigned char *y_rd = y_st + r * YROW + 32 * a;

    // The filter taps of this wave's group are requested before any row: the filter table and the
    // Toeplitz operand tiles are then built while the rows are in flight (loads complete in the
    // order of issue, so taps requested after the rows would arrive after all of them).
    // htab[lag + 32] = h[hl-1-lag] for 0 <= lag < hl, else 0.
    hraw_t hv[HTAB / 64];
    load_taps<T>(dm, h, (c0 + 16 * w < d) ? fdiv((uint32_t)(cb * NW + w), pl.q_dg16) : 0, l, hv);

    // The operands of the NK-1 steps before the segment are rebuilt first (zero before the
    // start of the sequence).  Their rows are requested together, so the replay costs one
    // memory latency instead of NK-1; step s_lo-i lands in ring slot NK-i, where phase 0
    // expects it.  The rows of the first step follow them: they are needed last.
    constexpr int NLEAD = NK > 1 ? NK - 1 : 1;
    Row<T> lx[NLEAD], lB[NLEAD];
    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            const uint32_t o = lane_in + IM * step_off(s_lo - i);
            lx[i - 1] = ldw_row_policy<T, GCG_MFMA_FWD_LEAD_LD>(wx, o);
            lB[i - 1] = ldw_row_policy<T, GCG_MFMA_FWD_LEAD_LD>(wB, o);
        }
    }
    Row<T> xr, Br, Cr;
    auto fetch = [&](int64_t s, Row<T> &xo, Row<T> &Bo, Row<T> &Co) {
        const uint32_t o = lane_in + IM * step_off(s);
        xo = ldw_row_policy<T, GCG_MFMA_FWD_LD>(wx, o);
        Bo = ldw_row_policy<T, GCG_MFMA_FWD_LD>(wB, o);
        Co = ldw_row_policy<T, GCG_MFMA_FWD_LD>(wC, o);
    };
    fetch(s_lo, xr, Br, Cr);
    TR(1);

    store_taps(htab[w], l, hv);
    __syncthreads();
    TR(2);
    typename M::wop_t W0[NK], W1[NK];   // output rows 0..15 / 16..31 of the step against input step s-i
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = M::toeplitz(htab[w], 32 * i, j, q);
        W1[i] = M::toeplitz(htab[w], 32 * i + 16, j, q);
    }
    TR(3);

    if constexpr (NK > 1) {
        // all lead-in tiles go to LDS together: one pair of barriers instead of NK-1
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            float xf[8], Bf[8], uf[8];
            unpack8<T>(lx[i - 1], xf);
            unpack8<T>(lB[i - 1], Bf);
#pragma unroll
            for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
            store_operand<T>(u_wr + (i - 1) * STEP * UROW, UROW, uf);
        }
        __syncthreads();
        TR(4);
#pragma unroll
        for (int i = 1; i < NK; ++i) A[NK - i] = M::load_operand(u_rm + (i - 1) * STEP * UROW, UROW, w, j, q, false);
        __syncthreads();
    }

    TR(5);
    int64_t s = s_lo;
    while (s < s_hi) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < s_hi) {
                TR_IF(4 * (s - s_lo) == (s_hi - s_lo), 8);
                TR_IF(4 * (s - s_lo) == 2 * (s_hi - s_lo), 9);
                TR_IF(4 * (s - s_lo) == 3 * (s_hi - s_lo), 10);
                // rows of the next step; past the segment they fall outside the window
                Row<T> xn, Bn, Cn;
                fetch(s + 1, xn, Bn, Cn);

                float xf[8], Bf[8], uf[8];
                unpack8<T>(xr, xf);
                unpack8<T>(Br, Bf);
#pragma unroll
                for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
                store_operand<T>(u_wr, UROW, uf);
                const uint32_t o = lane_off + step_off(s);
                if constexpr (EXTRA) stw_row<T>(wbx, o, pack8<T>(uf));
                __syncthreads();
                A[ph] = M::load_operand(u_rm, UROW, w, j, q, false);
                {
                    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < NK; ++i) {
                        acc0 = M::mfma(A[(ph - i + NK) % NK], W0[i], acc0);
                        acc1 = M::mfma(A[(ph - i + NK) % NK], W1[i], acc1);
                    }
                    *(f32x4 *)y_wr = acc0;
                    *(f32x4 *)(y_wr + 16 * YROW) = acc1;
                }
                __syncthreads();
                {
                    const f32x4 p0 = *(const f32x4 *)y_rd;
                    const f32x4 p1 = *(const f32x4 *)(y_rd + 16);
                    float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                    float Cf[8], yf[8];
                    unpack8<T>(Cr, Cf);
#pragma unroll
                    for (int e = 0; e < 8; ++e) yf[e] = Cf[e] * y2f[e];
                    stw_row_policy<T, (ES == 2 ? GCG_MFMA_FWD_ST : WIN_NT_ST)>(wy, o, pack8<T>(yf));
                    if constexpr (EXTRA) stw_row<T>(wy2, o, pack8<T>(y2f));
                }
                xr = xn; Br = Bn; Cr = Cn;
                ++s;
            }
        }
    }
    TR(6);
}

// --------------------------------------------------------------------------- backward
// One fused kernel for dC, dx, dB and the filter-gradient partials; the activations the
// reference saves (Bx, y2) are recomputed on chip.  Iteration sigma of a workgroup produces
// the outputs of step sigma.  Looking back it needs u of steps sigma-NK+1..sigma (for y2 and
// dC = dy*y2); looking forward it needs g2 = dy*C of steps sigma..sigma+NK-1 (for
// du[t] = sum_lag h[hl-1-lag] g2[t+lag]).  So iteration sigma loads x, B of step sigma and
// dy, C of step sigma+NK-1: nothing is read twice, and only dy waits NK-1 steps in registers.
//
// The anti-causal product reuses the forward Toeplitz operands: feeding the g2 operand with
// its 32 time samples in reverse order turns W(p, i) into the operand of the transposed
// band for output half 1-p, with the 16 output columns coming out reversed.
//
// Filter gradient: dh[hl-1-lag] = sum g2[t,c] u[t-lag,c].  For the new u step the products
// against the NK g2 steps in the ring are accumulated as ND = 2*NK-1 tiles
//   P_delta[i][j] += sum_c G2[32*sigma + 16*delta + i, c] * U[32*sigma + j, c]
// (one 32-deep product contracts 16 channels x 2 row halves), lag = 16*delta + i - j.  At the
// end the diagonals of the P tiles are summed in a fixed order into per-wave partials in
// the workspace, and a second kernel adds the partials in a fixed order.
// PL: x, B, C and dx, dB, dC are thirds of the rows of (bs, L, 3 d) tensors (Dims::planar).
// GAP: idle cycles in front of the output stores (GCG_MFMA_BWD_ST_GAP), for long runs.
template <typename T, int NK, int NW, bool PL = false, bool GAP = false>
__global__ __launch_bounds__(64 * NW) void mfma_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                       const T *__restrict__ B, const T *__restrict__ C,
                                                       const T *__restrict__ h, T *__restrict__ dx,
                                                       T *__restrict__ dB, T *__restrict__ dC,
                                                       T *__restrict__ dh, float *__restrict__ ws, Dims dm,
                                                       MfmaPlan pl)
{
    typedef MT<T> M;
    typedef typename M::op_t op_t;
    typedef typename M::hraw_t hraw_t;
    typedef Geo<T, NW> G;
    constexpr int CB = G::CB, UROW = G::UROW, YROW = G::YROW, ES = M::ES;
    constexpr int ND = 2 * NK - 1;
    constexpr int RING_ROWS = STEP * NK;
    constexpr int OFF_U = 0;                                // u of the current step, row-major
    constexpr int OFF_G = OFF_U + STEP * UROW;              // g2 ring, NK steps, row-major
    constexpr int OFF_Y = OFF_G + RING_ROWS * UROW;         // y2 tile, fp32, row-major
    constexpr int OFF_D = OFF_Y + STEP * YROW;              // du tile, fp32, row-major
    constexpr int OFF_H = OFF_D + STEP * YROW;              // filter tables
    constexpr int LDS_MAIN = OFF_H + NW * HTAB * (int)sizeof(hraw_t);
    constexpr int LDS_TAIL = NW * (16 * ND + 16) * 17 * 4;  // P tiles at the end (dh_finish)
    // A 4-wave workgroup at 16 bits asks for more than half of the CU's 160 KB, so that a CU holds one
    // (two on a CU, two waves per SIMD, are a third slower than one).
    constexpr int LDS_NEED = LDS_MAIN > LDS_TAIL ? LDS_MAIN : LDS_TAIL;
    constexpr int LDS_ALONE = (NW == 4 && ES == 2) ? 82 * 1024 : 0;
    constexpr int LDS_BYTES = LDS_NEED > LDS_ALONE ? LDS_NEED : LDS_ALONE;
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_BYTES];
    unsigned char *u_rm = smem + OFF_U, *g_rm = smem + OFF_G, *y_st = smem + OFF_Y, *d_st = smem + OFF_D;
    hraw_t *htab = (hraw_t *)(smem + OFF_H);
    TR_INIT;
    TR(0);

    const uint32_t wg_id = xcd_contiguous_u32(blockIdx.x, gridDim.x);
    int cb, seg, bi;
    wg_place(wg_id, pl, cb, seg, bi);
    const int64_t b = bi;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int r = tid / G::LPR, a = tid % G::LPR;   // row layout: row r of the step, channels 8a..8a+7
    const int j = l & 15, q = l >> 4;               // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;
    const bool wave_valid = c0 + 16 * w < d;

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;

    // Windows of this batch row: x, B and the outputs over rows [t0, t1), dy and C over [t0, t2)
    // (the backward looks NK-1 steps ahead for g2).  A lane's offset is lane_off + step_off(s).
    const int64_t t0 = (s_lo - (NK - 1)) * STEP > 0 ? (s_lo - (NK - 1)) * STEP : 0;
    const int64_t t1 = s_hi * STEP < L ? s_hi * STEP : L;
    const int64_t t2 = (s_hi + NK - 1) * STEP < L ? (s_hi + NK - 1) * STEP : L;
    const int64_t row_bytes = d * ES, origin = (b * L + t0) * d;
    const int64_t near_bytes = (t1 - t0) * row_bytes, far_bytes = (t2 - t0) * row_bytes;
    constexpr int IM = PL ? 3 : 1;                  // row stride of x, B, C, dx, dB, dC in rows of dy
    const win_t wx = make_window(x + IM * origin, IM * near_bytes), wB = make_window(B + IM * origin, IM * near_bytes);
    const win_t wdy = make_window(dy + origin, far_bytes), wC = make_window(C + IM * origin, IM * far_bytes);
    const win_t wdx = make_window(dx + IM * origin, IM * near_bytes), wdB = make_window(dB + IM * origin, IM * near_bytes);
    const win_t wdC = make_window(dC + IM * origin, IM * near_bytes);
    const uint32_t lane_off = (uint32_t)(r * row_bytes + (c0 + 8 * a) * ES) + (c0 + 8 * a < d ? 0u : WIN_OFF);
    const uint32_t lane_in = PL ? (uint32_t)(r * IM * row_bytes + (c0 + 8 * a) * ES) + (c0 + 8 * a < d ? 0u : WIN_OFF) : lane_off;
    auto step_off = [&](int64_t sg) { return (uint32_t)((sg * STEP - t0) * row_bytes); };

    // While step s runs in phase ph:  Au[(ph - i + NK) % NK] is the u operand of step s-i,
    // Ag[(ph + i) % NK] the time-reversed g2 operand of step s+i, dyq[(ph + i) % NK] dy of step s+i.
    op_t Au[NK], Ag[NK];
    Row<T> dyq[NK];
    f32x4 P[ND];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        Au[i] = M::zero_op();
        Ag[i] = M::zero_op();
        dyq[i] = zero_row<T>();
    }
#pragma unroll
    for (int i = 0; i < ND; ++i) P[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // LDS addresses of this lane
    const int rm_off = r * UROW + 8 * M::LES * a;                                // row layout, 8 channels
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    unsigned char *d_wr = d_st + (15 - j) * YROW + (16 * w + 4 * q) * 4;      // columns come out reversed
    const unsigned char *y_rd = y_st + r * YROW + 32 * a;
    const unsigned char *d_rd = d_st + r * YROW + 32 * a;

    // The filter taps of this wave's group are requested before any row, so that the filter table
    // and the Toeplitz tiles are built while the rows are in flight (loads complete in order of issue).
    hraw_t hv[HTAB / 64];
    load_taps<T>(dm, h, wave_valid ? fdiv((uint32_t)(cb * NW + w), pl.q_dg16) : 0, l, hv);

    // rows of iteration sg: x, B of step sg and dy, C of step sg+NK-1 (zero outside the windows)
    auto fetch = [&](int64_t sg, Row<T> &xo, Row<T> &Bo, Row<T> &dyo, Row<T> &Co) {
        const uint32_t o = lane_in + IM * step_off(sg), o2 = lane_off + step_off(sg + NK - 1);
        xo = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wx, o);
        Bo = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wB, o);
        dyo = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wdy, o2);
        Co = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wC, PL ? lane_in + IM * step_off(sg + NK - 1) : o2);
    };

    // Lead-in: u of the NK-1 steps before the segment and g2 of its first NK-1 steps, i.e. the
    // rows iterations s_lo-NK+1 .. s_lo-1 would have brought.  They are requested together,
    // so the lead-in costs one memory latency instead of NK-1; the rows of the first iteration
    // follow them (needed last).
    constexpr int NLEAD = NK > 1 ? NK - 1 : 1;
    Row<T> wx_[NLEAD], wB_[NLEAD], wdy_[NLEAD], wC_[NLEAD];
    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) fetch(s_lo - i, wx_[i - 1], wB_[i - 1], wdy_[i - 1], wC_[i - 1]);
    }
    Row<T> xr, Br, dyr, Cr;
    fetch(s_lo, xr, Br, dyr, Cr);
    TR(1);

    store_taps(htab + w * HTAB, l, hv);
    __syncthreads();
    TR(2);
    typename M::wop_t W0[NK], W1[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = M::toeplitz(htab + w * HTAB, 32 * i, j, q);
        W1[i] = M::toeplitz(htab + w * HTAB, 32 * i + 16, j, q);
    }
    TR(3);

    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            // iteration s_lo-i carries u of step s_lo-i and g2 / dy of step s_lo+NK-1-i
            float f0[8], f1[8], pf[8];
            unpack8<T>(wx_[i - 1], f0);
            unpack8<T>(wB_[i - 1], f1);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = f0[e] * f1[e];
            store_operand<T>(u_rm + rm_off, UROW, pf);
            unpack8<T>(wdy_[i - 1], f0);
            unpack8<T>(wC_[i - 1], f1);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = f0[e] * f1[e];
            unsigned char *g_slot = g_rm + (NK - 1 - i) * STEP * UROW;
            store_operand<T>(g_slot + rm_off, UROW, pf);
            dyq[NK - 1 - i] = wdy_[i - 1];
            __syncthreads();
            Au[NK - i] = M::load_operand(u_rm, UROW, w, j, q, false);
            Ag[NK - 1 - i] = M::load_operand(g_slot, UROW, w, j, q, true);
            __syncthreads();
        }
    }

    TR(5);
    int64_t s = s_lo;
    while (s < s_hi) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < s_hi) {
                const int slot_new = (ph + NK - 1) % NK;     // ring slot of step s+NK-1
                TR_IF(4 * (s - s_lo) == (s_hi - s_lo), 8);
                TR_IF(4 * (s - s_lo) == 2 * (s_hi - s_lo), 9);
                TR_IF(4 * (s - s_lo) == 3 * (s_hi - s_lo), 10);
                // rows of the next iteration; past the segment they fall outside the windows
                Row<T> xn, Bn, dyn, Cn;
                fetch(s + 1, xn, Bn, dyn, Cn);

                float xf[8], Bf[8], tf[8], cf[8], pf[8];
                unpack8<T>(xr, xf);
                unpack8<T>(Br, Bf);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = xf[e] * Bf[e];
                store_operand<T>(u_rm + rm_off, UROW, pf);
                unpack8<T>(dyr, tf);
                unpack8<T>(Cr, cf);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = tf[e] * cf[e];
                unsigned char *g_slot = g_rm + slot_new * STEP * UROW;
                store_operand<T>(g_slot + rm_off, UROW, pf);
                dyq[slot_new] = dyr;
                __syncthreads();
                Au[ph] = M::load_operand(u_rm, UROW, w, j, q, false);
                Ag[slot_new] = M::load_operand(g_slot, UROW, w, j, q, true);
                {
                    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
                    f32x4 dac0 = {0.f, 0.f, 0.f, 0.f}, dac1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < NK; ++i) {
                        acc0 = M::mfma(Au[(ph - i + NK) % NK], W0[i], acc0);
                        acc1 = M::mfma(Au[(ph - i + NK) % NK], W1[i], acc1);
                        dac0 = M::mfma(Ag[(ph + i) % NK], W1[i], dac0);   // output rows 0..15
                        dac1 = M::mfma(Ag[(ph + i) % NK], W0[i], dac1);   // output rows 16..31
                    }
                    *(f32x4 *)y_wr = acc0;
                    *(f32x4 *)(y_wr + 16 * YROW) = acc1;
                    *(f32x4 *)d_wr = dac0;
                    *(f32x4 *)(d_wr + 16 * YROW) = dac1;
                    // filter-gradient tiles: natural-layout operands (rows j and 16+j of a 32-row window)
                    const op_t un = M::load_natural(u_rm + j * UROW, u_rm + (16 + j) * UROW, UROW, w, q);
#pragma unroll
                    for (int dl = 0; dl < ND; ++dl) {
                        int row0 = STEP * ph + 16 * dl + j;              // ring rows of the window's two halves
                        int row1 = row0 + 16;
                        row0 = (row0 >= RING_ROWS) ? row0 - RING_ROWS : row0;
                        row1 = (row1 >= RING_ROWS) ? row1 - RING_ROWS : row1;
                        const op_t gn = M::load_natural(g_rm + row0 * UROW, g_rm + row1 * UROW, UROW, w, q);
                        P[dl] = M::mfma_aa(gn, un, P[dl]);
                    }
                }
                __syncthreads();
                {
                    const uint32_t o = lane_in + IM * step_off(s);
                    {
                        const f32x4 p0 = *(const f32x4 *)y_rd;
                        const f32x4 p1 = *(const f32x4 *)(y_rd + 16);
                        const float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                        float dyf[8], of[8];
                        unpack8<T>(dyq[ph], dyf);
#pragma unroll
                        for (int e = 0; e < 8; ++e) of[e] = dyf[e] * y2f[e];
                        if constexpr (GAP) idle_cycles<GCG_MFMA_BWD_ST_GAP>();
                        stw_row_policy<T, GCG_MFMA_BWD_ST_DC>(wdC, o, pack8<T>(of));
                    }
                    {
                        const f32x4 p0 = *(const f32x4 *)d_rd;
                        const f32x4 p1 = *(const f32x4 *)(d_rd + 16);
                        const float duf[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                        float of[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) of[e] = duf[e] * Bf[e];
                        if constexpr (GAP) idle_cycles<GCG_MFMA_BWD_ST_GAP>();
                        stw_row_policy<T, GCG_MFMA_BWD_ST>(wdx, o, pack8<T>(of));
#pragma unroll
                        for (int e = 0; e < 8; ++e) of[e] = duf[e] * xf[e];
                        if constexpr (GAP) idle_cycles<GCG_MFMA_BWD_ST_GAP>();
                        stw_row_policy<T, GCG_MFMA_BWD_ST>(wdB, o, pack8<T>(of));
                    }
                }
                xr = xn; Br = Bn; dyr = dyn; Cr = Cn;
                ++s;
            }
        }
    }

    TR(6);
    dh_finish<T, NW, ND>(P, smem, ws, dh, dm, pl, wg_id, cb, wave_valid);
    TR(7);
}

// Which element types take the two-kinds-of-waves backward below: 16-bit tensors in fp32 arithmetic (7B layer shape:
// bf16 232 -> 203 us, f16 311 -> 283 us).  Plain 16-bit tensors wait for memory, not for instructions (bf16: 181 us
// against 173 with mfma_bwd_kernel), and so do fp32 tensors, whose rows are twice as long (492 us against 460).
template <typename T> constexpr bool duo_type() { return std::is_same<T, bf16w_t>::value || std::is_same<T, f16w_t>::value; }

// --------------------------------------------------------------------------- backward, product waves and row waves
// The split-arithmetic backward is bound by instruction issue, not by memory (its 87 matrix instructions per step
// alone are 1600 cycles), and a SIMD runs matrix and vector instructions one after the other whether they come from
// one wave or from two (16 v_mfma_f32_16x16x32_bf16 take 312 cycles, 128 v_fma_f32 from a second wave 380, both 707).
// What a second wave per SIMD can hide is the waiting: LDS round trips, barriers, rows in flight.  The register state of
// mfma_bwd_kernel allows one wave per SIMD, so this kernel splits it over two kinds of waves in one workgroup of 512
// threads, one of each kind per SIMD, for the same 16 x 4 channels:
//   product waves (0..3): the Toeplitz operands, the u and g2 operand rings and the y2 / du products of a step;
//   row waves (4..7): global loads and stores, the gates before and after the products, and the filter-gradient
//     products (their operands are rows in natural order, which the row waves have just written).
// They meet at one barrier per step.  Iteration sigma: the product waves work on step sigma (operands written to LDS
// during iteration sigma-1, results to the y2 / du tiles of sigma's parity); the row waves finish step sigma-1 from
// the tiles of the other parity, prepare step sigma+1 (u into the tile of the other parity, g2 of step sigma+NK into
// a ring of NK+1 steps of g2, which both kinds of waves read) and accumulate the filter-gradient tiles of step sigma
// from the ring.
// Five-slice filters only (the rings' periods fix the unrolling: 2 NK for the product waves, NK+1 for the row waves).
template <typename T, bool PL = false>
__global__ __launch_bounds__(512) void mfma_bwd_duo_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                       const T *__restrict__ B, const T *__restrict__ C,
                                                       const T *__restrict__ h, T *__restrict__ dx,
                                                       T *__restrict__ dB, T *__restrict__ dC,
                                                       T *__restrict__ dh, float *__restrict__ ws, Dims dm,
                                                       MfmaPlan pl)
{
    typedef DuoGeo<T> D;
    typedef typename D::M M;
    typedef typename D::G G;
    constexpr int NK = D::NK, NW = D::NW, ND = D::ND, RSLOTS = D::RSLOTS;
    constexpr int CB = G::CB, UROW = D::UROW, YROW = D::YROW, ES = M::ES, USZ = D::USZ, YSZ = D::YSZ;
    constexpr int OFF_U = D::OFF_U, OFF_Y = D::OFF_Y, OFF_D = D::OFF_D;
    constexpr int LDS_MAIN = D::OFF_H + D::H_BYTES;
    constexpr int LDS_BYTES = LDS_MAIN > D::LDS_TAIL ? LDS_MAIN : D::LDS_TAIL;
    static_assert(LDS_BYTES <= 160 * 1024, "tiles do not fit the CU's LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_BYTES];
    unsigned char *const ring = smem + D::OFF_R;
    TR_INIT;
    TR(0);

    const uint32_t wg_id = xcd_contiguous_u32(blockIdx.x, gridDim.x);
    int cb, seg, bi;
    wg_place(wg_id, pl, cb, seg, bi);
    const int64_t b = bi;

    const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63;
    const bool row_wave = wv >= NW;
    const int w = wv & (NW - 1);                    // the wave's 16-channel block (either kind)
    const int vt = tid & (64 * NW - 1);             // row layout of the row waves: row r of the step, channels 8a..8a+7
    const int r = vt / G::LPR, a = vt % G::LPR;
    const int j = l & 15, q = l >> 4;               // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;
    const bool wave_valid = c0 + 16 * w < d;

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;

    f32x4 P[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i) P[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (!row_wave) {
        duo_product_waves<T>(smem, h, dm, pl, cb, w, l, wave_valid, s_lo, s_hi);
    } else {
        // ------------------------------------------------------------------ row waves
        // windows as in mfma_bwd_kernel: x, B and the outputs over rows [t0, t1), dy and C over [t0, t2)
        const int64_t t0 = (s_lo - (NK - 1)) * STEP > 0 ? (s_lo - (NK - 1)) * STEP : 0;
        const int64_t t1 = s_hi * STEP < L ? s_hi * STEP : L;
        const int64_t t2 = (s_hi + NK - 1) * STEP < L ? (s_hi + NK - 1) * STEP : L;
        const int64_t row_bytes = d * ES, origin = (b * L + t0) * d;
        const int64_t near_bytes = (t1 - t0) * row_bytes, far_bytes = (t2 - t0) * row_bytes;
        constexpr int IM = PL ? 3 : 1;                  // row stride of x, B, C, dx, dB, dC in rows of dy
        const win_t wx = make_window(x + IM * origin, IM * near_bytes), wB = make_window(B + IM * origin, IM * near_bytes);
        const win_t wdy = make_window(dy + origin, far_bytes), wC = make_window(C + IM * origin, IM * far_bytes);
        const win_t wdx = make_window(dx + IM * origin, IM * near_bytes), wdB = make_window(dB + IM * origin, IM * near_bytes);
        const win_t wdC = make_window(dC + IM * origin, IM * near_bytes);
        const uint32_t lane_off = (uint32_t)(r * row_bytes + (c0 + 8 * a) * ES) + (c0 + 8 * a < d ? 0u : WIN_OFF);
        const uint32_t lane_in = PL ? (uint32_t)(r * IM * row_bytes + (c0 + 8 * a) * ES) + (c0 + 8 * a < d ? 0u : WIN_OFF) : lane_off;
        auto step_off = [&](int64_t sg) { return (uint32_t)((sg * STEP - t0) * row_bytes); };
        const int rm_off = r * UROW + 8 * M::LES * a;
        const int yd_rd = r * YROW + 32 * a;

        // rows of iteration sg: x, B of step sg and dy, C of step sg+NK-1 (zero outside the windows)
        auto fetch = [&](int64_t sg, Row<T> &xo, Row<T> &Bo, Row<T> &dyo, Row<T> &Co) {
            const uint32_t o = lane_in + IM * step_off(sg), o2 = lane_off + step_off(sg + NK - 1);
            xo = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wx, o);
            Bo = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wB, o);
            dyo = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wdy, o2);
            Co = ldw_row_policy<T, GCG_MFMA_BWD_LD>(wC, PL ? lane_in + IM * step_off(sg + NK - 1) : o2);
        };
        // u = x * B into a u tile; g2 = dy * C into a slot of the ring
        auto gate_rows = [&](const Row<T> &xo, const Row<T> &Bo, const Row<T> &dyo, const Row<T> &Co, unsigned char *u_t,
                             unsigned char *g_ring) {
            float f0[8], f1[8], pf[8];
            unpack8<T>(xo, f0);
            unpack8<T>(Bo, f1);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = f0[e] * f1[e];
            store_operand<T>(u_t + rm_off, UROW, pf);
            unpack8<T>(dyo, f0);
            unpack8<T>(Co, f1);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = f0[e] * f1[e];
            store_operand<T>(g_ring + rm_off, UROW, pf);
        };
        // dC, dx, dB of step sg from its y2 / du tiles
        auto finish_step = [&](int64_t sg, bool live, const unsigned char *y_t, const unsigned char *d_t,
                               const Row<T> &dyo, const Row<T> &xo, const Row<T> &Bo) {
            const uint32_t o = live ? lane_in + IM * step_off(sg) : WIN_OFF;
            {
                const f32x4 p0 = *(const f32x4 *)(y_t + yd_rd);
                const f32x4 p1 = *(const f32x4 *)(y_t + yd_rd + 16);
                const float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                float dyf[8], of[8];
                unpack8<T>(dyo, dyf);
#pragma unroll
                for (int e = 0; e < 8; ++e) of[e] = dyf[e] * y2f[e];
                stw_row_policy<T, GCG_MFMA_BWD_ST_DC>(wdC, o, pack8<T>(of));
            }
            {
                const f32x4 p0 = *(const f32x4 *)(d_t + yd_rd);
                const f32x4 p1 = *(const f32x4 *)(d_t + yd_rd + 16);
                const float duf[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                float xf[8], Bf[8], of[8];
                unpack8<T>(xo, xf);
                unpack8<T>(Bo, Bf);
#pragma unroll
                for (int e = 0; e < 8; ++e) of[e] = duf[e] * Bf[e];
                stw_row_policy<T, GCG_MFMA_BWD_ST>(wdx, o, pack8<T>(of));
#pragma unroll
                for (int e = 0; e < 8; ++e) of[e] = duf[e] * xf[e];
                stw_row_policy<T, GCG_MFMA_BWD_ST>(wdB, o, pack8<T>(of));
            }
        };

        // Rings of the row waves, indexed by step - s_lo: x, B of three steps (the one being finished, the one in the
        // matrix cores, the one being prepared, whose slot the rows in flight take over once it is finished);
        // dy of NK+1 steps; dy, C of the rows in flight in one of two staging sets.
        Row<T> xh[3], Bh[3], dyq[RSLOTS], dy_st[2], C_st[2];
        Row<T> xp = zero_row<T>(), Bp = zero_row<T>(), dyp = zero_row<T>();   // x, B, dy of the step being finished
#pragma unroll
        for (int i = 0; i < 3; ++i) xh[i] = Bh[i] = zero_row<T>();
#pragma unroll
        for (int i = 0; i < RSLOTS; ++i) dyq[i] = zero_row<T>();
        Row<T> wx_[NK - 1], wB_[NK - 1], wdy_[NK - 1], wC_[NK - 1];
#pragma unroll
        for (int i = 1; i < NK; ++i) fetch(s_lo - i, wx_[i - 1], wB_[i - 1], wdy_[i - 1], wC_[i - 1]);
        fetch(s_lo, xh[0], Bh[0], dy_st[0], C_st[0]);
        fetch(s_lo + 1, xh[1], Bh[1], dy_st[1], C_st[1]);
        TR(1);
        __syncthreads();                                              // (A)
        __syncthreads();                                              // (A2)
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            // iteration s_lo-i carries u of step s_lo-i and g2 / dy of step s_lo+NK-1-i
            gate_rows(wx_[i - 1], wB_[i - 1], wdy_[i - 1], wC_[i - 1], smem + OFF_U,
                      ring + (NK - 1 - i) * USZ);
            dyq[NK - 1 - i] = wdy_[i - 1];
            __syncthreads();                                          // (B_i)
            __syncthreads();                                          // (C_i)
        }
        // step s_lo is prepared here, as an iteration s_lo-1 would have
        gate_rows(xh[0], Bh[0], dy_st[0], C_st[0], smem + OFF_U, ring + (NK - 1) * USZ);
        dyq[NK - 1] = dy_st[0];
        __syncthreads();                                              // (D)

        int64_t s = s_lo;
        auto row_step = [&](int pu) __attribute__((always_inline)) {
                    const int par = pu & 1;
                    const unsigned char *const u_cur = smem + OFF_U + par * USZ;
                    unsigned char *const u_nx = smem + OFF_U + (par ^ 1) * USZ;
                    const unsigned char *const y_old = smem + OFF_Y + (par ^ 1) * YSZ, *const d_old = smem + OFF_D + (par ^ 1) * YSZ;
                    // Order: the request for rows first, then the stores, then what needs the previous request's rows, the
                    // filter-gradient products last.  Measured at the 7B shape: products first 240 us, stores before the
                    // request 218, this order 203 - 205, the gating after the products 221.
                    // rows of iteration s+2 into the slots that step s-1 has left (past the segment: outside the windows)
                    fetch(s + 2, xh[(pu + 2) % 3], Bh[(pu + 2) % 3], dy_st[par], C_st[par]);
                    // step s-1: gate its tiles and store
                    finish_step(s - 1, s > s_lo, y_old, d_old, dyp, xp, Bp);
                    // step s+1: its rows arrived during the last iteration
                    dyq[(pu + RSLOTS - 1) % RSLOTS] = dy_st[par ^ 1];          // dy of step s+NK
                    gate_rows(xh[(pu + 1) % 3], Bh[(pu + 1) % 3], dy_st[par ^ 1], C_st[par ^ 1], u_nx,
                              ring + ((pu + RSLOTS - 1) % RSLOTS) * USZ);
                    duo_filter_gradient<T>(P, u_cur, ring, pu, w, l);    // filter-gradient tiles of step s
                    dyp = dyq[pu];                 // step s is finished during the next iteration
                    xp = xh[pu % 3];
                    Bp = Bh[pu % 3];
                    __syncthreads();
                    ++s;
        };
        // Every step can be the run's last, so the compiler's wait counts restart at each: a step's request for rows
        // then goes out once the previous request has been answered.  With the steps in straight-line groups the
        // counts are exact, two requests are in flight, and the kernel is 9 % slower (222 against 203 us at the 7B
        // shape): the memory system delivers less with more on the way, as in the other backward kernels.
        while (s < s_hi) {
#pragma unroll
            for (int pu = 0; pu < RSLOTS; ++pu)
                if (s < s_hi) row_step(pu);
        }
        // the last step of the segment: its tiles are those of parity (s_hi - 1 - s_lo) & 1
        {
            const int par = (int)((s_hi - 1 - s_lo) & 1);
            finish_step(s_hi - 1, true, smem + OFF_Y + par * YSZ, smem + OFF_D + par * YSZ, dyp, xp, Bp);
        }
    }

    TR(6);
    dh_finish<T, NW, ND, 512>(P, smem, ws, dh, dm, pl, wg_id, cb, wave_valid, row_wave, w);
    TR(7);
}

template <typename T, int NK, int NW>
int fwd_launch(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
               const Dims &dm, hipStream_t st)
{
    int e = 0;
    // 16-bit: ~112 registers, 4 waves per SIMD; fp32: ~200 registers, 2 waves per SIMD
    // runs down to 4 steps: on a tensor too small to fill the machine otherwise (a tensor-parallel rank's share, d = 1024)
    // more, shorter runs beat the lead-in they replay (35 -> 24 us at (1, 8192, 1024)); large tensors never get there
    MfmaPlan p = plan(dm, NW, 4, MT<T>::SPLIT ? 8 : 16, MT<T>::ES);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    // Workgroup order.  With 32 or more channel blocks per row the XCD-contiguous order gives an XCD whole rows;
    // with fewer, dealing the blocks round-robin measured 3-5 % faster in the forward (d = 2048, 4096) and the same
    // from d = 8192 on.  (The backward is 3 % faster XCD-contiguous at every width.)
    static const int order = env_int("GCG_MFMA_FWD_ORDER", -1);   // tuning override: 0 round-robin, 1 XCD-contiguous
    p.xcd = order >= 0 ? (order != 0) : (p.ncb >= 32);
    if constexpr (NK == 5) {
        // planar operands: instantiated for the five-slice walk only (fwd_t sends every filter length there)
        if (dm.planar)
            return (y2 || bx) ? (int)hipErrorInvalidValue
                              : launch_main((mfma_fwd_kernel<T, NK, NW, false, true>), dim3((unsigned)p.nwg), dim3(64 * NW), st,
                                            (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    }
    if (y2 || bx)
        e = launch_main((mfma_fwd_kernel<T, NK, NW, true>), dim3((unsigned)p.nwg), dim3(64 * NW), st,
                           (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    else
        e = launch_main((mfma_fwd_kernel<T, NK, NW, false>), dim3((unsigned)p.nwg), dim3(64 * NW), st,
                           (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    return e;
}

template <typename T, int NK>
int fwd_nk(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
           const Dims &dm, hipStream_t st)
{
    const int nw = choose_nw(dm, MT<T>::SPLIT);
    if constexpr (!MT<T>::SPLIT) {
        if (nw == 16) return fwd_launch<T, NK, 16>(x, B, C, h, y, y2, bx, dm, st);
    }
    if (nw == 8) return fwd_launch<T, NK, 8>(x, B, C, h, y, y2, bx, dm, st);
    return fwd_launch<T, NK, 4>(x, B, C, h, y, y2, bx, dm, st);
}

template <typename T>
int fwd_t(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
          const Dims &dm, hipStream_t st)
{
    switch (dm.planar ? 5 : nk_for(dm.hl)) {
    case 1: return fwd_nk<T, 1>(x, B, C, h, y, y2, bx, dm, st);
    case 2: return fwd_nk<T, 2>(x, B, C, h, y, y2, bx, dm, st);
    case 3: return fwd_nk<T, 3>(x, B, C, h, y, y2, bx, dm, st);
    case 4: return fwd_nk<T, 4>(x, B, C, h, y, y2, bx, dm, st);
    default: return fwd_nk<T, 5>(x, B, C, h, y, y2, bx, dm, st);
    }
}

} // namespace

bool mfma_supported(int dtype, const Dims &dm)
{
    (void)dtype;   // bf16, f16 and fp32 all have a matrix-core form
    // the shortest segment with its lead-in and look-ahead must fit one tensor window
    return dm.hl <= 128 && dm.dg % 16 == 0 && (int64_t)(1 + 2 * 5) * STEP * 3 * dm.d * 4 <= WIN_MAX_BYTES;
}

int mfma_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h, void *y,
                    void *y2, void *bx, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return fwd_t<bf16_t>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_F16) return fwd_t<f16_t>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_F32) return fwd_t<float>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_BF16_F32) return fwd_t<bf16w_t>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_F16_F32) return fwd_t<f16w_t>(x, B, C, h, y, y2, bx, dm, st);
    return (int)hipErrorInvalidValue;
}

bool mfma_bwd_available() { return true; }

#ifdef GCG_TRACE
} // namespace gcg
// trace builds only: device address and size of the timestamp table (16 slots of 8 bytes per workgroup)
extern "C" GCG_API void *gcg_trace_buffer(size_t *bytes)
{
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(gcg::g_trace)) != hipSuccess) return nullptr;
    if (bytes) *bytes = sizeof(gcg::g_trace);
    return p;
}
namespace gcg {
#endif

namespace {


template <typename T, int NK, int NW>
int bwd_launch(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
               void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    int e = 0;
    MfmaPlan p = plan_bwd(dm, MT<T>::SPLIT, MT<T>::ES);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (p.fuse_dh && (p.slot = dh_slot_for_stream(st)) < 0) p.fuse_dh = p.slot = 0;   // no ticket set: second launch
    auto launch = [&](auto kernel, int threads) {
        return launch_main(kernel, dim3((unsigned)p.nwg), dim3(threads), st, (const T *)dy, (const T *)x, (const T *)B,
                           (const T *)C, (const T *)h, (T *)dx, (T *)dB, (T *)dC, (T *)dh, (float *)ws, dm, p);
    };
    if constexpr (NK == 5 && duo_type<T>()) {
        // product waves and row waves in one workgroup: the types whose backward is bound by instruction issue
        e = dm.planar ? launch(mfma_bwd_duo_kernel<T, true>, 512) : launch(mfma_bwd_duo_kernel<T, false>, 512);
    } else if constexpr (NK == 5) {
        // planar operands: instantiated for the five-slice walk only (bwd_t sends every filter length there);
        // plain 16-bit tensors in runs of 32 steps and more: with the idle cycles in front of the stores
        if (dm.planar) e = launch(mfma_bwd_kernel<T, NK, NW, true>, 64 * NW);
        else if (!MT<T>::SPLIT && p.steps_per_seg >= 32) e = launch(mfma_bwd_kernel<T, NK, NW, false, !MT<T>::SPLIT>, 64 * NW);
        else e = launch(mfma_bwd_kernel<T, NK, NW>, 64 * NW);
    } else {
        e = launch(mfma_bwd_kernel<T, NK, NW>, 64 * NW);
    }
    if (e || p.fuse_dh) return e;
    const int64_t n = (int64_t)dm.g * (dm.fw ? dm.lc : dm.hl);
    e = launch_plain(mfma_dh_reduce_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), st,
                       (const float *)ws, (T *)dh, dm, p);
    return e;
}

template <typename T, int NK>
int bwd_nk(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
           void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    return bwd_launch<T, NK, BWD_NW>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
}

template <typename T>
int bwd_t(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
          void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    switch (dm.planar ? 5 : nk_for(dm.hl)) {
    case 1: return bwd_nk<T, 1>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case 2: return bwd_nk<T, 2>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case 3: return bwd_nk<T, 3>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case 4: return bwd_nk<T, 4>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    default: return bwd_nk<T, 5>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    }
}

} // namespace

size_t mfma_bwd_workspace(int dtype, const Dims &dm)
{
    const MfmaPlan p = plan_bwd(dm, dtype != GCG_BF16 && dtype != GCG_F16, dtype == GCG_F32 ? 4 : 2);
    return (size_t)p.nwg * p.nw * 128 * sizeof(float);
}

int mfma_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C, const void *h,
                    void *dx, void *dB, void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return bwd_t<bf16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dtype == GCG_F16) return bwd_t<f16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dtype == GCG_F32) return bwd_t<float>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dtype == GCG_BF16_F32) return bwd_t<bf16w_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dtype == GCG_F16_F32) return bwd_t<f16w_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
