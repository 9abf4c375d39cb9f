// Matrix-core kernels on interleaved operands: x, B, C are the thirds of one (bs, L, g, dg, 3)
// projected-features tensor, [..., 0] = C, [..., 1] = B, [..., 2] = x, and the backward writes
// dC, dB, dx in the same interleaved layout.
//
// The product side is the one of gcg_mfma.hip (same operand tiles, same order of operations,
// so y, dC, dB, dx agree bit for bit with the separate-tensor kernels, and dh up to the order in
// which the runs' partial sums are added).  The memory side differs: a
// row of the workgroup's 16*NW channels is 48*NW elements of (C, B, x) triples, and a lane
// takes 12 bytes of it per row -- two channels at 16 bits, one at fp32 -- so that the 64 lanes
// of a load or store cover one contiguous 768-byte run.  (Eight channels per lane, as in the
// separate-tensor kernels, would put lanes 48 bytes apart and make every access touch three
// times the cache lines it uses; measured at 0.72x the bandwidth.)  With 12 bytes per row a
// lane owns NR = 4 (16-bit) or 8 (fp32) rows of a 32-row step, RP = 32/NR rows apart.
#include "gcg_il_tile.h"

// Cache policy of the forward's output stores on 16-bit tensors (gcg_common.h: 2 = nontemporal, 16 = device scope:
// written through the XCD's L2).  As in gcg_mfma.hip the device-scope store measured faster: 96.5 against 98.5 us at
// the 7B layer shape.
#ifndef GCG_MFMA_IL_FWD_ST
#define GCG_MFMA_IL_FWD_ST 16
#endif

// Idle cycles in front of each output store of the 4-wave backward (tuning builds may override).  Measured at the
// 7B layer shape: bf16 174.0 us without, 170.4 - 170.9 with 8 - 12 cycles, 171.9 with 16, 178.7 with 24; f16 171.9,
// 168.4 - 169.1, 166.1, 167.3; 1 x 32768 x 8192 bf16: 663, 655 - 657, 665, 670.  (The kernel with product waves and
// row waves is bound by instruction issue and loses with any.)
#ifndef GCG_MFMA_IL_BWD_ST_GAP
#define GCG_MFMA_IL_BWD_ST_GAP 12
#endif
namespace gcg {
namespace {

// ---------------------------------------------------------------------------- forward
// KF > 0: `feat` is the projection output and wfeat the featurizer's filters (see above).
template <typename T, int NK, int NW, int KF>
__global__ __launch_bounds__(64 * NW) void mfma_il_fwd_kernel(const T *__restrict__ feat, const T *__restrict__ h,
                                                          const T *__restrict__ wfeat, T *__restrict__ y, Dims dm,
                                                          MfmaPlan pl, int kf)
{
    typedef MT<T> M;
    typedef typename M::op_t op_t;
    typedef typename M::hraw_t hraw_t;
    typedef Geo<T, NW> G;
    typedef GeoIL<T, NW> I;
    constexpr int CB = G::CB, UROW = G::UROW, YROW = G::YROW;
    constexpr int CH = I::CH, LPR = I::LPR, RP = I::RP, NR = I::NR;
    constexpr bool FEAT = KF > 0;
    constexpr int NH = FEAT ? KF - 1 : 0;           // rows fetched before the lane's own
    constexpr int KS = FEAT ? 1 : RP;               // rows between a lane's consecutive rows
    constexpr int NV = 3 * CH;                      // feature values of a lane's row piece
    __shared__ __attribute__((aligned(16))) unsigned char u_rm[STEP * UROW];
    __shared__ __attribute__((aligned(16))) unsigned char y_st[STEP * YROW];
    __shared__ hraw_t htab[NW][HTAB];

    int cb, seg, bi;
    wg_place(pl.xcd ? xcd_contiguous_u32(blockIdx.x, gridDim.x) : blockIdx.x, pl, cb, seg, bi);
    const int64_t b = bi;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int rr = tid / LPR, a = tid % LPR;        // memory layout: rows row0 + KS*k, channels CH*a ..
    const int row0 = FEAT ? NR * rr : rr;
    const int j = l & 15, q = l >> 4;               // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;

    // Windows over rows [t0, t1) of this batch row (12-byte pieces are only 4-byte aligned, which
    // buffer accesses take).  A lane's offset into y is lane_off + k * pass_off + step_off(s); into
    // the features three times that.  (With the featurizer the features' window starts NH rows earlier.)
    const int64_t t0 = (s_lo - (NK - 1)) * STEP > 0 ? (s_lo - (NK - 1)) * STEP : 0;
    const int64_t t1 = s_hi * STEP < L ? s_hi * STEP : L;
    const int64_t tf = t0 - NH > 0 ? t0 - NH : 0;
    const int64_t row_bytes = d * M::ES, win_bytes = (t1 - t0) * row_bytes;
    const int64_t origin = (b * L + t0) * d;
    const win_t wf = make_window(feat + 3 * (b * L + tf) * d, 3 * (t1 - tf) * row_bytes);
    const win_t wy = make_window(y + origin, win_bytes);
    const bool cvalid = c0 + CH * a < d;
    const uint32_t lane_off = (uint32_t)(row0 * row_bytes + (c0 + CH * a) * M::ES);
    const uint32_t feat_off = lane_off + (uint32_t)((t0 - tf) * row_bytes);
    const uint32_t pass_off = __builtin_amdgcn_readfirstlane((uint32_t)(KS * row_bytes)), bad = cvalid ? 0u : WIN_OFF;
    auto step_off = [&](int64_t s) { return (uint32_t)((s * STEP - t0) * row_bytes); };
    // The lane's part and the uniform part of a feature offset are tripled separately, and inside the loop the uniform
    // part is a running value (so3): written as 3 * (lane + uniform) each access costs a 64-bit multiply-add on the
    // vector unit.
    const uint32_t feat_off3 = 3 * feat_off + bad;
    const uint32_t pass_off3 = __builtin_amdgcn_readfirstlane(3 * pass_off);

    op_t A[NK];            // A[(ph - i + NK) % NK]: operand of step s-i while step s runs in phase ph
#pragma unroll
    for (int i = 0; i < NK; ++i) A[i] = M::zero_op();

    unsigned char *u_wr = u_rm + row0 * UROW + M::LES * CH * a;
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    const unsigned char *y_rd = y_st + row0 * YROW + 4 * CH * a;

    // rows of step s: the NH rows before the lane's own first, then its NR rows
    auto fetch = [&](uint32_t so3, u32x3 (&p)[NH + NR]) {
#pragma unroll
        for (int k = 0; k < NH + NR; ++k) p[k] = ldw12(wf, feat_off3 + (so3 + (uint32_t)(k - NH) * pass_off3));
    };
    auto store_u = [&](const float (&uf)[8]) {
#pragma unroll
        for (int k = 0; k < NR; ++k) store_operand_unit<T>(u_wr + KS * k * UROW, UROW, &uf[CH * k]);
    };
    float tap[FEAT ? KF : 1][NV];
    if constexpr (FEAT) load_feat_taps<T, KF, NV>(wfeat, cvalid ? 3 * (c0 + CH * a) : 0, kf, tap);
    // (C, B, x) of the lane's rows from the fetched pieces
    auto rows_of = [&](const u32x3 (&p)[NH + NR], float (&xf)[8], float (&Bf)[8], float (&Cf)[8]) {
        if constexpr (FEAT) featurized_rows<T, NR, KF>(p, tap, xf, Bf, Cf);
        else il_split<T, NR>(p, xf, Bf, Cf);
    };
    // The filter taps of this wave's group are requested before any row, so that the filter table and the
    // Toeplitz tiles are built while the rows are in flight (loads complete in order of issue).
    hraw_t hv[HTAB / 64];
    load_taps<T>(dm, h, (c0 + 16 * w < d) ? fdiv((uint32_t)(cb * NW + w), pl.q_dg16) : 0, l, hv);

    // A segment that starts inside the sequence first rebuilds the operands of the NK-1 steps
    // before it; their rows are requested together (one memory latency instead of NK-1) and
    // step s_lo-i lands in ring slot NK-i, where phase 0 expects it.  The rows of the first step
    // follow them: they are needed last.
    constexpr int NLEAD = NK > 1 ? NK - 1 : 1;
    u32x3 lead[NLEAD][NH + NR];
    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) fetch(3 * step_off(s_lo - i), lead[i - 1]);
    }
    u32x3 in[NH + NR];
    fetch(3 * step_off(s_lo), in);

    store_taps(htab[w], l, hv);
    __syncthreads();
    typename M::wop_t W0[NK], W1[NK];   // output rows 0..15 / 16..31 of the step against input step s-i
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = M::toeplitz(htab[w], 32 * i, j, q);
        W1[i] = M::toeplitz(htab[w], 32 * i + 16, j, q);
    }

    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            float xf[8], Bf[8], Cf[8], uf[8];
            rows_of(lead[i - 1], xf, Bf, Cf);
#pragma unroll
            for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
            store_u(uf);
            __syncthreads();
            A[NK - i] = M::load_operand(u_rm, UROW, w, j, q, false);
            __syncthreads();
        }
    }

    // the run's steps are counted from 0 in 32 bits, and so are their offsets (the values of step_off modulo 2^32)
    const int n_steps = (int)(s_hi - s_lo);
    const uint32_t step_b = __builtin_amdgcn_readfirstlane((uint32_t)(STEP * row_bytes));
    const uint32_t step_b3 = __builtin_amdgcn_readfirstlane(3 * step_b);
    uint32_t so = __builtin_amdgcn_readfirstlane(step_off(s_lo));            // of step s
    uint32_t so3 = __builtin_amdgcn_readfirstlane(3 * step_off(s_lo));
    int s = 0;
    while (s < n_steps) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < n_steps) {
                u32x3 nx[NH + NR];   // rows of the next step; past the segment they fall outside the window
                fetch(so3 + step_b3, nx);

                float xf[8], Bf[8], Cf[8], uf[8];
                rows_of(in, xf, Bf, Cf);
#pragma unroll
                for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
                store_u(uf);
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
                const uint32_t o = lane_off + so + bad;
#pragma unroll
                for (int k = 0; k < NR; ++k) {
                    float yf[CH];
#pragma unroll
                    for (int c = 0; c < CH; ++c)
                        yf[c] = Cf[CH * k + c] * *(const float *)(y_rd + KS * k * YROW + 4 * c);
                    // each store right behind its values, nothing scheduled across it: plain 16-bit tensors measure
                    // 97.4 -> 95.0 us at the 7B layer shape and 366.7 -> 358.9 us at 1 x 32768 x 8192 with this
                    // (8 - 16 more idle cycles: 96.1 - 96.2 us, 32: 97.2); the other element types measure the same
                    if constexpr (!M::SPLIT) idle_cycles<1>();
                    __builtin_amdgcn_raw_buffer_store_b32(pack_unit<T>(yf), wy, (int)(o + k * pass_off), 0,
                                                          M::ES == 2 ? GCG_MFMA_IL_FWD_ST : WIN_NT_ST);
                }
#pragma unroll
                for (int k = 0; k < NH + NR; ++k) in[k] = nx[k];
                ++s;
                so += step_b;
                so3 += step_b3;
            }
        }
    }
}

// --------------------------------------------------------------------------- backward
// Same schedule as the separate-tensor backward: iteration sigma produces the outputs of step
// sigma from u of steps sigma-NK+1..sigma and g2 = dy*C of steps sigma..sigma+NK-1.  In the
// interleaved tensor C of step sigma+NK-1 arrives together with x, B of that step, NK-1
// iterations before those are used, and the outputs of a row leave as one interleaved row.
// The early x, B values wait in LDS: each lane parks its own two row vectors in a ring of NK-1
// slots and reads them back itself, so the ring needs no barrier.
// KF > 0: `feat` is the projection output and wfeat the featurizer's filters (see above); dfeat is still the
// gradient of the featurized features, which the featurizer's own backward then takes.
template <typename T, int NK, int NW, bool KEEP, int KF>
__global__ __launch_bounds__(64 * NW) void mfma_il_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ feat,
                                                          const T *__restrict__ h, const T *__restrict__ wfeat,
                                                          int kf, T *__restrict__ dfeat,
                                                          T *__restrict__ dh, float *__restrict__ ws, Dims dm,
                                                          MfmaPlan pl)
{
    typedef MT<T> M;
    typedef typename M::op_t op_t;
    typedef typename M::hraw_t hraw_t;
    typedef Geo<T, NW> G;
    typedef GeoIL<T, NW> I;
    constexpr int CB = G::CB, UROW = G::UROW, YROW = G::YROW;
    constexpr int CH = I::CH, LPR = I::LPR, RP = I::RP, NR = I::NR;
    constexpr bool FEAT = KF > 0;
    constexpr int NH = FEAT ? KF - 1 : 0;           // rows fetched before the lane's own
    constexpr int KS = FEAT ? 1 : RP;               // rows between a lane's consecutive rows
    constexpr int NV = 3 * CH;                      // feature values of a lane's row piece
    constexpr int ND = 2 * NK - 1;
    constexpr int RING_ROWS = STEP * NK;
    constexpr int OFF_U = 0;                                // u of the current step, row-major
    constexpr int OFF_G = OFF_U + STEP * UROW;              // g2 ring, NK steps, row-major
    constexpr int OFF_Y = OFF_G + RING_ROWS * UROW;         // y2 tile, fp32, row-major
    constexpr int OFF_D = OFF_Y + STEP * YROW;              // du tile, fp32, row-major
    constexpr int OFF_H = OFF_D + STEP * YROW;              // filter tables: dead once the Toeplitz tiles are built,
    constexpr int OFF_XB = OFF_H;                           // so the waiting x, B values take the same place
    constexpr int XB_SLOTS = NK > 1 ? NK - 1 : 0;
    constexpr int XB_VEC = G::NT * 16 * M::RW;              // one row vector of every lane
    constexpr int XB_BYTES = XB_SLOTS * 2 * XB_VEC, H_BYTES = NW * HTAB * (int)sizeof(hraw_t);
    constexpr int LDS_MAIN = OFF_XB + (XB_BYTES > H_BYTES ? XB_BYTES : H_BYTES);
    constexpr int LDS_TAIL = NW * (16 * ND + 16) * 17 * 4;  // P tiles at the end (dh_finish)
    // a 4-wave workgroup at 16 bits asks for more than half of the CU's 160 KB, so that a CU holds one
    constexpr int LDS_NEED = LDS_MAIN > LDS_TAIL ? LDS_MAIN : LDS_TAIL;
    constexpr int LDS_ALONE = (NW == 4 && M::ES == 2) ? 82 * 1024 : 0;
    constexpr int LDS_BYTES = LDS_NEED > LDS_ALONE ? LDS_NEED : LDS_ALONE;
    static_assert(LDS_BYTES <= 160 * 1024, "workgroup exceeds the 160 KB of LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_BYTES];
    unsigned char *u_rm = smem + OFF_U, *g_rm = smem + OFF_G, *y_st = smem + OFF_Y, *d_st = smem + OFF_D;
    hraw_t *htab = (hraw_t *)(smem + OFF_H);

    const uint32_t wg_id = xcd_contiguous_u32(blockIdx.x, gridDim.x);
    int cb, seg, bi;
    wg_place(wg_id, pl, cb, seg, bi);
    const int64_t b = bi;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int rr = tid / LPR, a = tid % LPR;        // memory layout: rows row0 + KS*k, channels CH*a ..
    const int row0 = FEAT ? NR * rr : rr;
    const int j = l & 15, q = l >> 4;               // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;
    const bool wave_valid = c0 + 16 * w < d;

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;

    // Windows of this batch row: the outputs over rows [t0, t1), the features and dy over
    // [t0, t2) (the backward looks NK-1 steps ahead for g2).
    const int64_t t0 = (s_lo - (NK - 1)) * STEP > 0 ? (s_lo - (NK - 1)) * STEP : 0;
    const int64_t t1 = s_hi * STEP < L ? s_hi * STEP : L;
    const int64_t t2 = (s_hi + NK - 1) * STEP < L ? (s_hi + NK - 1) * STEP : L;
    const int64_t tf = t0 - NH > 0 ? t0 - NH : 0;        // the featurizer looks NH rows further back
    const int64_t row_bytes = d * M::ES, origin = (b * L + t0) * d;
    const win_t wf = make_window(feat + 3 * (b * L + tf) * d, 3 * (t2 - tf) * row_bytes);
    const win_t wdyw = make_window(dy + origin, (t2 - t0) * row_bytes);
    const win_t wdf = make_window(dfeat + 3 * origin, 3 * (t1 - t0) * row_bytes);
    const bool cvalid = c0 + CH * a < d;
    const uint32_t lane_off = (uint32_t)(row0 * row_bytes + (c0 + CH * a) * M::ES);
    const uint32_t feat_off = lane_off + (uint32_t)((t0 - tf) * row_bytes);
    const uint32_t pass_off = __builtin_amdgcn_readfirstlane((uint32_t)(KS * row_bytes)), bad = cvalid ? 0u : WIN_OFF;
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
    const int rm_off = row0 * UROW + M::LES * CH * a;                                  // memory layout, row row0
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    unsigned char *d_wr = d_st + (15 - j) * YROW + (16 * w + 4 * q) * 4;      // columns come out reversed
    const unsigned char *y_rd = y_st + row0 * YROW + 4 * CH * a;
    const unsigned char *d_rd = d_st + row0 * YROW + 4 * CH * a;
    unsigned char *xb_own = smem + OFF_XB + tid * 16 * M::RW;                 // slot k at + k * 2 * XB_VEC

    // interleaved rows and dy of one step (zero outside the sequence)
    // (with the featurizer: the NH rows before the lane's own first, then its NR rows)
    // (so3: three times the step's offset step_off(step).  The lane's part and the uniform part of an offset are
    // tripled separately and the uniform one is a running value inside the loop: written as 3 * (lane + uniform)
    // each access costs a 64-bit multiply-add on the vector unit.)
    const uint32_t feat_off3 = 3 * feat_off + bad, lane_off3 = 3 * lane_off + bad;
    const uint32_t pass_off3 = __builtin_amdgcn_readfirstlane(3 * pass_off);
    // x, B rows straight from the pieces (il_split_rows): not for plain f16, whose conversions through fp32 the compiler
    // removes by itself, and whose backward measures 10 us slower with the explicit form (7B layer shape)
    constexpr bool SPLIT_ROWS = !std::is_same<T, f16_t>::value;
    auto fetch_feat = [&](uint32_t so3, u32x3 (&p)[NH + NR]) {
#pragma unroll
        for (int k = 0; k < NH + NR; ++k) p[k] = ldw12(wf, feat_off3 + (so3 + (uint32_t)(k - NH) * pass_off3));
    };
    float tap[FEAT ? KF : 1][NV];
    if constexpr (FEAT) load_feat_taps<T, KF, NV>(wfeat, cvalid ? 3 * (c0 + CH * a) : 0, kf, tap);
    // x, B, C of the lane's rows from the fetched pieces
    auto rows_of = [&](const u32x3 (&p)[NH + NR], float (&xo)[8], float (&Bo)[8], float (&Co)[8]) {
        if constexpr (FEAT) featurized_rows<T, NR, KF>(p, tap, xo, Bo, Co);
        else il_split<T, NR>(p, xo, Bo, Co);
    };
    auto fetch_dy = [&](uint32_t so, Row<T> &out) {
        const uint32_t o = lane_off + so + bad;
        uint32_t u[NR];
#pragma unroll
        for (int k = 0; k < NR; ++k) u[k] = ldw4(wdyw, o + k * pass_off);
        out = units_row<T, NR>(u);
    };
    auto store_rows = [&](unsigned char *tile, const float (&f)[8]) {
#pragma unroll
        for (int k = 0; k < NR; ++k) store_operand_unit<T>(tile + rm_off + KS * k * UROW, UROW, &f[CH * k]);
    };

    // iteration sigma brings the interleaved rows and dy of step sigma+NK-1
    u32x3 in[NH + NR];
    Row<T> dyr;
    // The filter taps of this wave's group are requested before any row (loads complete in order of issue).
    hraw_t hv[HTAB / 64];
    load_taps<T>(dm, h, wave_valid ? fdiv((uint32_t)(cb * NW + w), pl.q_dg16) : 0, l, hv);

    // Lead-in: the rows of the NK-1 steps before the segment (for u) and of its first NK-1 steps
    // (for g2, and x, B to wait in the ring), i.e. what iterations s_lo-NK+1 .. s_lo-1 would have
    // brought.  Requested together, so the lead-in costs one memory latency instead of NK-1; the rows
    // of the first iteration follow them (needed last).
    constexpr int NLEAD = NK > 1 ? NK - 1 : 1;
    u32x3 past[NLEAD][NH + NR], lead[NLEAD][NH + NR];
    Row<T> wdy[NLEAD];
    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            fetch_feat(3 * step_off(s_lo - i), past[i - 1]);
            fetch_feat(3 * step_off(s_lo + NK - 1 - i), lead[i - 1]);
            fetch_dy(step_off(s_lo + NK - 1 - i), wdy[i - 1]);
        }
    }
    fetch_feat(3 * step_off(s_lo + NK - 1), in);
    fetch_dy(step_off(s_lo + NK - 1), dyr);

    store_taps(htab + w * HTAB, l, hv);
    __syncthreads();
    typename M::wop_t W0[NK], W1[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = M::toeplitz(htab + w * HTAB, 32 * i, j, q);
        W1[i] = M::toeplitz(htab + w * HTAB, 32 * i + 16, j, q);
    }
    __syncthreads();      // the filter tables have been read: their place now holds the waiting x, B values

    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            // iteration s_lo-i carries u of step s_lo-i and g2 / dy of step s_lo+NK-1-i
            float f0[8], f1[8], f2[8], tf[8], pf[8];
            rows_of(past[i - 1], f0, f1, f2);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = f0[e] * f1[e];
            store_rows(u_rm, pf);
            // x, B of step s_lo+NK-1-i wait in ring slot (NK-1-i) % (NK-1) for iteration s_lo+NK-1-i
            rows_of(lead[i - 1], f0, f1, f2);
            unsigned char *slot = xb_own + ((NK - 1 - i) % (NK - 1)) * 2 * XB_VEC;
            lds_store_row<T>(slot, pack8<T>(f0));
            lds_store_row<T>(slot + XB_VEC, pack8<T>(f1));
            unpack8<T>(wdy[i - 1], tf);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = tf[e] * f2[e];
            unsigned char *g_slot = g_rm + (NK - 1 - i) * STEP * UROW;
            store_rows(g_slot, pf);
            dyq[NK - 1 - i] = wdy[i - 1];
            __syncthreads();
            Au[NK - i] = M::load_operand(u_rm, UROW, w, j, q, false);
            Ag[NK - 1 - i] = M::load_operand(g_slot, UROW, w, j, q, true);
            __syncthreads();
        }
    }

    int xb_slot = 0;      // ring slot of step s (step s_lo+k sits in slot k % (NK-1))
    // the run's steps are counted from 0 in 32 bits, and so are their offsets (the values of step_off modulo 2^32)
    const int n_steps = (int)(s_hi - s_lo);
    const uint32_t step_b = __builtin_amdgcn_readfirstlane((uint32_t)(STEP * row_bytes));
    uint32_t so = __builtin_amdgcn_readfirstlane(step_off(s_lo));        // of step s
    uint32_t so3 = __builtin_amdgcn_readfirstlane(3 * step_off(s_lo));
    const uint32_t step_b3 = __builtin_amdgcn_readfirstlane(3 * step_b);
    int s = 0;
    while (s < n_steps) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < n_steps) {
                const int slot_new = (ph + NK - 1) % NK;     // ring slot of step s+NK-1
                u32x3 nx[NH + NR];   // rows of the next iteration; past the segment's reach they are
                Row<T> dyn;          // outside the windows
                fetch_feat(so3 + (uint32_t)NK * step_b3, nx);
                fetch_dy(so + (uint32_t)NK * step_b, dyn);

                float xf[8], Bf[8], tf[8], cf[8], pf[8];
                if constexpr (SPLIT_ROWS && NK > 1 && !FEAT && M::ES == 2) {
                    // x, B of step s+NK-1 go to the ring as they are; C as fp32
                    Row<T> xa, Ba;
                    il_split_rows<T>(in, xa, Ba, cf);
                    unsigned char *slot = xb_own + xb_slot * 2 * XB_VEC;
                    const Row<T> xw = lds_load_row<T>(slot), Bw = lds_load_row<T>(slot + XB_VEC);
                    lds_store_row<T>(slot, xa);
                    lds_store_row<T>(slot + XB_VEC, Ba);
                    xb_slot = (xb_slot + 1 == NK - 1) ? 0 : xb_slot + 1;
                    unpack8<T>(xw, xf);
                    unpack8<T>(Bw, Bf);
                } else {
                    float xa[8], Ba[8];
                    rows_of(in, xa, Ba, cf);                  // x, B, C of step s+NK-1
                    if constexpr (NK > 1) {
                        unsigned char *slot = xb_own + xb_slot * 2 * XB_VEC;
                        const Row<T> xw = lds_load_row<T>(slot), Bw = lds_load_row<T>(slot + XB_VEC);
                        lds_store_row<T>(slot, pack8<T>(xa));
                        lds_store_row<T>(slot + XB_VEC, pack8<T>(Ba));
                        xb_slot = (xb_slot + 1 == NK - 1) ? 0 : xb_slot + 1;
                        unpack8<T>(xw, xf);
                        unpack8<T>(Bw, Bf);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) { xf[e] = xa[e]; Bf[e] = Ba[e]; }
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = xf[e] * Bf[e];
                store_rows(u_rm, pf);
                unpack8<T>(dyr, tf);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = tf[e] * cf[e];
                unsigned char *g_slot = g_rm + slot_new * STEP * UROW;
                store_rows(g_slot, pf);
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
                    float dyf[8], oC[8], ox[8], oB[8];
                    unpack8<T>(dyq[ph], dyf);
#pragma unroll
                    for (int k = 0; k < NR; ++k)
#pragma unroll
                        for (int c = 0; c < CH; ++c) {
                            const int e = CH * k + c;
                            const float y2v = *(const float *)(y_rd + KS * k * YROW + 4 * c);
                            const float duv = *(const float *)(d_rd + KS * k * YROW + 4 * c);
                            oC[e] = dyf[e] * y2v;
                            ox[e] = duv * Bf[e];
                            oB[e] = duv * xf[e];
                        }
                    u32x3 po[NR];
                    il_join<T, NR>(ox, oB, oC, po);
#pragma unroll
                    for (int k = 0; k < NR; ++k) {
                        if constexpr (GCG_MFMA_IL_BWD_ST_GAP > 0 && M::ES == 2 && !M::SPLIT) idle_cycles<GCG_MFMA_IL_BWD_ST_GAP>();
                        win_store_as<KEEP>(wdf, lane_off3 + (so3 + (uint32_t)k * pass_off3), po[k]);
                    }
                }
#pragma unroll
                for (int k = 0; k < NH + NR; ++k) in[k] = nx[k];
                dyr = dyn;
                ++s;
                so += step_b;
                so3 += step_b3;
            }
        }
    }

    dh_finish<T, NW, ND>(P, smem, ws, dh, dm, pl, wg_id, cb, wave_valid);
}

// bf16 tensors in fp32 arithmetic only: with f16's three-plane operand tiles the waiting x, B values no longer fit
// beside them (174 KB of LDS)
template <typename T> constexpr bool il_duo_type() { return std::is_same<T, bf16w_t>::value; }

// --------------------------------------------------------------------------- backward, product waves and row waves
// The interleaved-features form of mfma_bwd_duo_kernel (gcg_mfma.hip) for the element types whose backward is bound
// by instruction issue: four product waves (duo_product_waves) and four row waves in one workgroup, one barrier per
// step.  The rows of a step arrive as one interleaved piece per lane and row: C of step s+NK goes into g2 at once,
// x and B of that step wait in a lane-private ring in LDS until step s+NK is the one being prepared.  Iteration s of
// the row waves: request the rows of step s+NK+1; finish step s-1 (gate its y2 / du tiles, store its interleaved
// gradient rows); prepare step s+1 (u from the ring, g2 of step s+NK from the rows that arrived); the filter-gradient
// products of step s.
template <typename T, bool KEEP, int KF>
__global__ __launch_bounds__(512) void mfma_il_bwd_duo_kernel(const T *__restrict__ dy, const T *__restrict__ feat,
                                                          const T *__restrict__ h, const T *__restrict__ wfeat,
                                                          int kf, T *__restrict__ dfeat, T *__restrict__ dh,
                                                          float *__restrict__ ws, Dims dm, MfmaPlan pl)
{
    typedef DuoGeo<T> D;
    typedef typename D::M M;
    typedef typename D::G G;
    typedef GeoIL<T, D::NW> I;
    constexpr int NK = D::NK, NW = D::NW, ND = D::ND, RSLOTS = D::RSLOTS;
    constexpr int CB = G::CB, UROW = D::UROW, YROW = D::YROW, USZ = D::USZ, YSZ = D::YSZ;
    constexpr int CH = I::CH, LPR = I::LPR, RP = I::RP, NR = I::NR;
    constexpr bool FEAT = KF > 0;
    constexpr int NH = FEAT ? KF - 1 : 0;           // rows fetched before the lane's own
    constexpr int KS = FEAT ? 1 : RP;               // rows between a lane's consecutive rows
    constexpr int NV = 3 * CH;                      // feature values of a lane's row piece
    // the waiting x, B values take the place of the filter tables, which are dead after barrier (A2)
    constexpr int OFF_XB = D::OFF_H;
    constexpr int XB_VEC = 64 * NW * 16 * M::RW;    // one row vector of every lane of the row waves
    constexpr int XB_BYTES = (NK - 1) * 2 * XB_VEC;
    constexpr int LDS_MAIN = OFF_XB + (XB_BYTES > D::H_BYTES ? XB_BYTES : D::H_BYTES);
    constexpr int LDS_BYTES = LDS_MAIN > D::LDS_TAIL ? LDS_MAIN : D::LDS_TAIL;
    static_assert(LDS_BYTES <= 160 * 1024, "tiles do not fit the CU's LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_BYTES];
    unsigned char *const ring = smem + D::OFF_R;

    const uint32_t wg_id = xcd_contiguous_u32(blockIdx.x, gridDim.x);
    int cb, seg, bi;
    wg_place(wg_id, pl, cb, seg, bi);
    const int64_t b = bi;

    const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63;
    const bool row_wave = wv >= NW;
    const int w = wv & (NW - 1);                    // the wave's 16-channel block (either kind)
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
        const int vt = tid & (64 * NW - 1);
        const int rr = vt / LPR, a = vt % LPR;      // memory layout: rows row0 + KS*k, channels CH*a ..
        const int row0 = FEAT ? NR * rr : rr;
        // windows of this batch row: the outputs over rows [t0, t1), the features and dy over [t0, t2)
        const int64_t t0 = (s_lo - (NK - 1)) * STEP > 0 ? (s_lo - (NK - 1)) * STEP : 0;
        const int64_t t1 = s_hi * STEP < L ? s_hi * STEP : L;
        const int64_t t2 = (s_hi + NK - 1) * STEP < L ? (s_hi + NK - 1) * STEP : L;
        const int64_t tf = t0 - NH > 0 ? t0 - NH : 0;        // the featurizer looks NH rows further back
        const int64_t row_bytes = d * M::ES, origin = (b * L + t0) * d;
        const win_t wf = make_window(feat + 3 * (b * L + tf) * d, 3 * (t2 - tf) * row_bytes);
        const win_t wdyw = make_window(dy + origin, (t2 - t0) * row_bytes);
        const win_t wdf = make_window(dfeat + 3 * origin, 3 * (t1 - t0) * row_bytes);
        const bool cvalid = c0 + CH * a < d;
        const uint32_t lane_off = (uint32_t)(row0 * row_bytes + (c0 + CH * a) * M::ES);
        const uint32_t feat_off = lane_off + (uint32_t)((t0 - tf) * row_bytes);
        const uint32_t pass_off = __builtin_amdgcn_readfirstlane((uint32_t)(KS * row_bytes)), bad = cvalid ? 0u : WIN_OFF;
        auto step_off = [&](int64_t sg) { return (uint32_t)((sg * STEP - t0) * row_bytes); };
        const int rm_off = row0 * UROW + M::LES * CH * a;
        const int yd_rd = row0 * YROW + 4 * CH * a;
        unsigned char *const xb_own = smem + OFF_XB + vt * 16 * M::RW;           // slot k at + k * 2 * XB_VEC

        // the interleaved rows and dy of one step (zero outside the sequence); with the featurizer the NH rows
        // before the lane's own come first
        struct Rows { u32x3 p[NH + NR]; Row<T> dy; };
        // (so: the step's offset, step_off(step), and so3 three times that; inside the loop running 32-bit values.  The
        // lane's part and the uniform part of an offset are tripled separately: written as 3 * (lane + uniform) each
        // access costs a 64-bit multiply-add on the vector unit.)
        const uint32_t feat_off3 = 3 * feat_off + bad, lane_off3 = 3 * lane_off + bad;
        const uint32_t pass_off3 = __builtin_amdgcn_readfirstlane(3 * pass_off);
        auto fetch_feat = [&](uint32_t so3, u32x3 (&p)[NH + NR]) {
#pragma unroll
            for (int k = 0; k < NH + NR; ++k) p[k] = ldw12(wf, feat_off3 + (so3 + (uint32_t)(k - NH) * pass_off3));
        };
        auto fetch = [&](uint32_t so, uint32_t so3, Rows &r) {
            fetch_feat(so3, r.p);
            const uint32_t o = lane_off + so + bad;
            uint32_t u[NR];
#pragma unroll
            for (int k = 0; k < NR; ++k) u[k] = ldw4(wdyw, o + k * pass_off);
            r.dy = units_row<T, NR>(u);
        };
        float tap[FEAT ? KF : 1][NV];
        if constexpr (FEAT) load_feat_taps<T, KF, NV>(wfeat, cvalid ? 3 * (c0 + CH * a) : 0, kf, tap);
        auto rows_of = [&](const u32x3 (&p)[NH + NR], float (&xo)[8], float (&Bo)[8], float (&Co)[8]) {
            if constexpr (FEAT) featurized_rows<T, NR, KF>(p, tap, xo, Bo, Co);
            else il_split<T, NR>(p, xo, Bo, Co);
        };
        auto store_rows = [&](unsigned char *tile, const float (&f)[8]) {
#pragma unroll
            for (int k = 0; k < NR; ++k) store_operand_unit<T>(tile + rm_off + KS * k * UROW, UROW, &f[CH * k]);
        };
        // g2 = dy * C of a step into its slot of the ring
        auto store_g2 = [&](const Row<T> &dyo, const float (&Cf)[8], unsigned char *g_ring) {
            float tf8[8], pf[8];
            unpack8<T>(dyo, tf8);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = tf8[e] * Cf[e];
            store_rows(g_ring, pf);
        };
        auto store_u = [&](const float (&xf)[8], const float (&Bf)[8], unsigned char *u_t) {
            float pf[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = xf[e] * Bf[e];
            store_rows(u_t, pf);
        };
        // the interleaved gradient rows of step sg from its y2 / du tiles
        auto finish_step = [&](uint32_t so3, bool live, const unsigned char *y_t, const unsigned char *d_t,
                               const Row<T> &dyo, const Row<T> &xo, const Row<T> &Bo) {
            float dyf[8], xf[8], Bf[8], oC[8], ox[8], oB[8];
            unpack8<T>(dyo, dyf);
            unpack8<T>(xo, xf);
            unpack8<T>(Bo, Bf);
#pragma unroll
            for (int k = 0; k < NR; ++k)
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    const int e = CH * k + c;
                    const float y2v = *(const float *)(y_t + yd_rd + KS * k * YROW + 4 * c);
                    const float duv = *(const float *)(d_t + yd_rd + KS * k * YROW + 4 * c);
                    oC[e] = dyf[e] * y2v;
                    ox[e] = duv * Bf[e];
                    oB[e] = duv * xf[e];
                }
            u32x3 po[NR];
            il_join<T, NR>(ox, oB, oC, po);
            const uint32_t o3 = live ? lane_off3 + so3 : WIN_OFF;
#pragma unroll
            for (int k = 0; k < NR; ++k) win_store_as<KEEP>(wdf, o3 + (uint32_t)k * pass_off3, po[k]);
        };

        // Rings of the row waves, indexed by step - s_lo: x, B (as row vectors of the tensors' type) of the step being
        // finished, the one in the matrix cores and the one being prepared; dy of NK+1 steps; two sets of rows in
        // turn for the request on its way.
        Row<T> xh[3], Bh[3], dyq[RSLOTS];
#pragma unroll
        for (int i = 0; i < 3; ++i) xh[i] = Bh[i] = zero_row<T>();
#pragma unroll
        for (int i = 0; i < RSLOTS; ++i) dyq[i] = zero_row<T>();
        Rows st[2];
        {
            // Lead-in: the rows of the NK-1 steps before the run (for u) and of its first NK steps (g2; x, B to wait in
            // the ring), requested together; the rows of step s_lo+NK follow them.
            u32x3 past[NK - 1][NH + NR];
            Rows lead[NK];
#pragma unroll
            for (int i = 1; i < NK; ++i) fetch_feat(3 * step_off(s_lo - i), past[i - 1]);
#pragma unroll
            for (int jj = NK - 2; jj >= 0; --jj) fetch(step_off(s_lo + jj), 3 * step_off(s_lo + jj), lead[jj]);
            fetch(step_off(s_lo + NK - 1), 3 * step_off(s_lo + NK - 1), lead[NK - 1]);
            fetch(step_off(s_lo + NK), 3 * step_off(s_lo + NK), st[1]);
            __syncthreads();                                          // (A)
            __syncthreads();                                          // (A2): the filter tables' place is free
            float f0[8], f1[8], f2[8];
#pragma unroll
            for (int i = 1; i < NK; ++i) {
                // iteration s_lo-i carries u of step s_lo-i and g2 / dy of step s_lo+NK-1-i
                rows_of(past[i - 1], f0, f1, f2);
                store_u(f0, f1, smem + D::OFF_U);
                const int jj = NK - 1 - i;
                rows_of(lead[jj].p, f0, f1, f2);
                if (jj >= 1) {           // x, B of step s_lo+jj wait in ring slot jj % (NK-1)
                    unsigned char *slot = xb_own + (jj % (NK - 1)) * 2 * XB_VEC;
                    lds_store_row<T>(slot, pack8<T>(f0));
                    lds_store_row<T>(slot + XB_VEC, pack8<T>(f1));
                } else {                 // step s_lo itself is prepared below
                    xh[0] = pack8<T>(f0);
                    Bh[0] = pack8<T>(f1);
                }
                store_g2(lead[jj].dy, f2, ring + jj * USZ);
                dyq[jj] = lead[jj].dy;
                __syncthreads();                                      // (B_i)
                __syncthreads();                                      // (C_i)
            }
            // step s_lo is prepared here, as an iteration s_lo-1 would have: u of step s_lo, g2 of step s_lo+NK-1
            {
                float xf[8], Bf[8];
                unpack8<T>(xh[0], xf);
                unpack8<T>(Bh[0], Bf);
                store_u(xf, Bf, smem + D::OFF_U);
                rows_of(lead[NK - 1].p, f0, f1, f2);
                unsigned char *slot = xb_own + ((NK - 1) % (NK - 1)) * 2 * XB_VEC;
                lds_store_row<T>(slot, pack8<T>(f0));
                lds_store_row<T>(slot + XB_VEC, pack8<T>(f1));
                store_g2(lead[NK - 1].dy, f2, ring + (NK - 1) * USZ);
                dyq[NK - 1] = lead[NK - 1].dy;
            }
            __syncthreads();                                          // (D)
        }

        int xb_slot = 1 % (NK - 1);          // ring slot of step s+1
        // the run's steps are counted from 0 in 32 bits, and so are their offsets (the same values modulo 2^32 as
        // step_off gives): 64-bit multiplications per step are a tenth of the row waves' vector cycles otherwise
        const int n_steps = (int)(s_hi - s_lo);
        const uint32_t step_b = __builtin_amdgcn_readfirstlane((uint32_t)(STEP * row_bytes));
        const uint32_t step_b3 = __builtin_amdgcn_readfirstlane(3 * step_b);
        uint32_t so = __builtin_amdgcn_readfirstlane(step_off(s_lo));        // of step s
        uint32_t so3 = __builtin_amdgcn_readfirstlane(3 * step_off(s_lo));
        int s = 0;
        auto row_step = [&](int pu) __attribute__((always_inline)) {
            const int par = pu & 1;
            const unsigned char *const u_cur = smem + D::OFF_U + par * USZ;
            unsigned char *const u_nx = smem + D::OFF_U + (par ^ 1) * USZ;
            const unsigned char *const y_old = smem + D::OFF_Y + (par ^ 1) * YSZ, *const d_old = smem + D::OFF_D + (par ^ 1) * YSZ;
            // Order as in mfma_bwd_duo_kernel: the request for rows first, then the stores, then what needs the previous
            // request's rows, the filter-gradient products last.
            fetch(so + (uint32_t)(NK + 1) * step_b, so3 + (uint32_t)(NK + 1) * step_b3, st[par]);
            finish_step(so3 - step_b3, s > 0, y_old, d_old, dyq[(pu + RSLOTS - 1) % RSLOTS], xh[(pu + 2) % 3], Bh[(pu + 2) % 3]);
            {
                // step s+1: x, B from the ring; C and dy of step s+NK from the rows that arrived, whose x, B take the slot
                float cf[8], xf[8], Bf[8];
                Row<T> xa, Ba;
                if constexpr (FEAT || M::ES == 4) {
                    float xv[8], Bv[8];
                    rows_of(st[par ^ 1].p, xv, Bv, cf);
                    xa = pack8<T>(xv);
                    Ba = pack8<T>(Bv);
                } else {
                    il_split_rows<T>(st[par ^ 1].p, xa, Ba, cf);
                }
                unsigned char *slot = xb_own + xb_slot * 2 * XB_VEC;
                const Row<T> xw = lds_load_row<T>(slot), Bw = lds_load_row<T>(slot + XB_VEC);
                lds_store_row<T>(slot, xa);
                lds_store_row<T>(slot + XB_VEC, Ba);
                xb_slot = (xb_slot + 1 == NK - 1) ? 0 : xb_slot + 1;
                unpack8<T>(xw, xf);
                unpack8<T>(Bw, Bf);
                store_u(xf, Bf, u_nx);
                store_g2(st[par ^ 1].dy, cf, ring + ((pu + RSLOTS - 1) % RSLOTS) * USZ);
                dyq[(pu + RSLOTS - 1) % RSLOTS] = st[par ^ 1].dy;               // dy of step s+NK
                xh[(pu + 1) % 3] = xw;
                Bh[(pu + 1) % 3] = Bw;
            }
            duo_filter_gradient<T>(P, u_cur, ring, pu, w, l);    // filter-gradient tiles of step s
            __syncthreads();
            ++s;
            so += step_b;
            so3 += step_b3;
        };
        // Every step can be the run's last (see mfma_bwd_duo_kernel for why the steps are not grouped); the run's
        // last step is finished where the loop leaves, so that the rings keep compile-time indices.
        bool done = false;
        while (!done) {
#pragma unroll
            for (int pu = 0; pu < RSLOTS; ++pu) {
                if (!done) {
                    if (s < n_steps) {
                        row_step(pu);
                    } else {
                        const int par = (pu & 1) ^ 1;         // of step n_steps-1
                        finish_step(so3 - step_b3, true, smem + D::OFF_Y + par * YSZ, smem + D::OFF_D + par * YSZ,
                                    dyq[(pu + RSLOTS - 1) % RSLOTS], xh[(pu + 2) % 3], Bh[(pu + 2) % 3]);
                        done = true;
                    }
                }
            }
        }
    }

    dh_finish<T, NW, ND, 512>(P, smem, ws, dh, dm, pl, wg_id, cb, wave_valid, row_wave, w);
}

// ---------------------------------------------------------------------------- launch
template <typename T, int NK, int NW>
int fwd_launch(const void *feat, const void *h, void *y, const Dims &dm, hipStream_t st)
{
    int e = 0;
    MfmaPlan p = plan(dm, NW, 4, MT<T>::SPLIT ? 8 : 16, MT<T>::ES);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    // Workgroup order: dealing the channel blocks to the XCDs round-robin measured 3-4 % faster than XCD-contiguous
    // runs on interleaved operands at every width (d = 4096: 102.5 against 105.4 us, d = 8192: 376 against 389 us,
    // d = 16384: 361 against 375 us).
    static const int order = env_int("GCG_MFMA_FWD_ORDER", -1);   // tuning override: 0 round-robin, 1 XCD-contiguous
    p.xcd = order >= 0 ? (order != 0) : 0;
    e = launch_main((mfma_il_fwd_kernel<T, NK, NW, 0>), dim3((unsigned)p.nwg), dim3(64 * NW), st, (const T *)feat,
                       (const T *)h, (const T *)nullptr, (T *)y, dm, p, 0);
    return e;
}

// the forward with the featurizer in front: full-length filters only (the five-slice walk), up to FEAT_KF taps
constexpr int FEAT_KF = 3;
template <typename T, int NW>
int fwd_feat_launch(const void *raw, const void *wfeat, int kf, const void *h, void *y, const Dims &dm, hipStream_t st)
{
    MfmaPlan p = plan(dm, NW, 4, MT<T>::SPLIT ? 8 : 16, MT<T>::ES);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    static const int order = env_int("GCG_MFMA_FWD_ORDER", -1);
    p.xcd = order >= 0 ? (order != 0) : 0;
    return launch_main((mfma_il_fwd_kernel<T, 5, NW, FEAT_KF>), dim3((unsigned)p.nwg), dim3(64 * NW), st,
                       (const T *)raw, (const T *)h, (const T *)wfeat, (T *)y, dm, p, kf);
}
template <typename T>
int fwd_feat_t(const void *raw, const void *wfeat, int kf, const void *h, void *y, const Dims &dm, hipStream_t st)
{
    static const int forced = env_int("GCG_MFMA_FEAT_NW", 0);   // tuning override: 4, 8 or 16
    // the featurizer's registers leave room for three waves per SIMD: 8-wave workgroups at most (16 spill)
    int nw = choose_nw(dm, MT<T>::SPLIT);
    if (nw > 8) nw = 8;
    if (forced == 4 || forced == 8 || (forced == 16 && !MT<T>::SPLIT)) nw = forced;
    if constexpr (!MT<T>::SPLIT) {
        if (nw == 16) return fwd_feat_launch<T, 16>(raw, wfeat, kf, h, y, dm, st);
    }
    if (nw == 8) return fwd_feat_launch<T, 8>(raw, wfeat, kf, h, y, dm, st);
    return fwd_feat_launch<T, 4>(raw, wfeat, kf, h, y, dm, st);
}

template <typename T, int NK> int fwd_nk(const void *feat, const void *h, void *y, const Dims &dm, hipStream_t st)
{
    const int nw = choose_nw(dm, MT<T>::SPLIT);
    if constexpr (!MT<T>::SPLIT) {
        if (nw == 16) return fwd_launch<T, NK, 16>(feat, h, y, dm, st);
    }
    if (nw == 8) return fwd_launch<T, NK, 8>(feat, h, y, dm, st);
    return fwd_launch<T, NK, 4>(feat, h, y, dm, st);
}

template <typename T> int fwd_t(const void *feat, const void *h, void *y, const Dims &dm, hipStream_t st)
{
    switch (nk_for(dm.hl)) {
    case 1: return fwd_nk<T, 1>(feat, h, y, dm, st);
    case 2: return fwd_nk<T, 2>(feat, h, y, dm, st);
    case 3: return fwd_nk<T, 3>(feat, h, y, dm, st);
    case 4: return fwd_nk<T, 4>(feat, h, y, dm, st);
    default: return fwd_nk<T, 5>(feat, h, y, dm, st);
    }
}

// same plan as the separate-tensor backward, so gcg_bwd_workspace_bytes covers both
template <typename T, int NK, int NW>
int bwd_launch(const void *dy, const void *feat, const void *h, void *dfeat, void *dh, void *ws, const Dims &dm,
               hipStream_t st)
{
    int e = 0;
    MfmaPlan p = plan_bwd(dm, MT<T>::SPLIT, MT<T>::ES);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (p.fuse_dh && (p.slot = dh_slot_for_stream(st)) < 0) p.fuse_dh = p.slot = 0;   // no ticket set: second launch
    auto launch = [&](auto kernel, int threads) {
        return launch_main(kernel, dim3((unsigned)p.nwg), dim3(threads), st, (const T *)dy, (const T *)feat, (const T *)h,
                           (const T *)nullptr, 0, (T *)dfeat, (T *)dh, (float *)ws, dm, p);
    };
    if constexpr (NK == 5 && il_duo_type<T>()) {
        // product waves and row waves in one workgroup: the types whose backward is bound by instruction issue
        e = dm.keep_out ? launch(mfma_il_bwd_duo_kernel<T, true, 0>, 512) : launch(mfma_il_bwd_duo_kernel<T, false, 0>, 512);
    } else {
        e = dm.keep_out ? launch(mfma_il_bwd_kernel<T, NK, NW, true, 0>, 64 * NW)
                        : launch(mfma_il_bwd_kernel<T, NK, NW, false, 0>, 64 * NW);
    }
    if (e || p.fuse_dh) return e;
    const int64_t n = (int64_t)dm.g * (dm.fw ? dm.lc : dm.hl);
    e = launch_plain(mfma_dh_reduce_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), st,
                       (const float *)ws, (T *)dh, dm, p);
    return e;
}

// the backward from the projection output (full-length filters; 4-wave workgroups; dfeat goes to the featurizer's
// backward next, so it is stored through the cache)
template <typename T, int NW>
int bwd_feat_launch(const void *dy, const void *raw, const void *wfeat, int kf, const void *h, void *dfeat, void *dh,
                    void *ws, const Dims &dm, MfmaPlan p, hipStream_t st)
{
    int e;
    if constexpr (NW == 4 && il_duo_type<T>())
        e = launch_main((mfma_il_bwd_duo_kernel<T, true, FEAT_KF>), dim3((unsigned)p.nwg), dim3(512), st,
                        (const T *)dy, (const T *)raw, (const T *)h, (const T *)wfeat, kf, (T *)dfeat, (T *)dh,
                        (float *)ws, dm, p);
    else
        e = launch_main((mfma_il_bwd_kernel<T, 5, NW, true, FEAT_KF>), dim3((unsigned)p.nwg), dim3(64 * NW), st,
                        (const T *)dy, (const T *)raw, (const T *)h, (const T *)wfeat, kf, (T *)dfeat, (T *)dh,
                        (float *)ws, dm, p);
    if (e || p.fuse_dh) return e;
    const int64_t n = (int64_t)dm.g * (dm.fw ? dm.lc : dm.hl);
    return launch_plain(mfma_dh_reduce_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), st,
                        (const float *)ws, (T *)dh, dm, p);
}
template <typename T>
int bwd_feat_t(const void *dy, const void *raw, const void *wfeat, int kf, const void *h, void *dfeat, void *dh,
               void *ws, const Dims &dm, hipStream_t st)
{
    MfmaPlan p = plan_bwd_nw(dm, choose_nw_bwd_feat(MT<T>::SPLIT), MT<T>::ES);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (p.fuse_dh && (p.slot = dh_slot_for_stream(st)) < 0) p.fuse_dh = p.slot = 0;   // no ticket set: second launch
    if constexpr (!MT<T>::SPLIT) {
        if (p.nw == 8) return bwd_feat_launch<T, 8>(dy, raw, wfeat, kf, h, dfeat, dh, ws, dm, p, st);
    }
    return bwd_feat_launch<T, 4>(dy, raw, wfeat, kf, h, dfeat, dh, ws, dm, p, st);
}

template <typename T, int NK>
int bwd_nk(const void *dy, const void *feat, const void *h, void *dfeat, void *dh, void *ws, const Dims &dm,
           hipStream_t st)
{
    return bwd_launch<T, NK, BWD_NW>(dy, feat, h, dfeat, dh, ws, dm, st);
}

template <typename T>
int bwd_t(const void *dy, const void *feat, const void *h, void *dfeat, void *dh, void *ws, const Dims &dm,
          hipStream_t st)
{
    switch (nk_for(dm.hl)) {
    case 1: return bwd_nk<T, 1>(dy, feat, h, dfeat, dh, ws, dm, st);
    case 2: return bwd_nk<T, 2>(dy, feat, h, dfeat, dh, ws, dm, st);
    case 3: return bwd_nk<T, 3>(dy, feat, h, dfeat, dh, ws, dm, st);
    case 4: return bwd_nk<T, 4>(dy, feat, h, dfeat, dh, ws, dm, st);
    default: return bwd_nk<T, 5>(dy, feat, h, dfeat, dh, ws, dm, st);
    }
}

} // namespace

int mfma_il_fwd_launch(int dtype, const void *feat, const void *h, void *y, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return fwd_t<bf16_t>(feat, h, y, dm, st);
    if (dtype == GCG_F16) return fwd_t<f16_t>(feat, h, y, dm, st);
    if (dtype == GCG_F32) return fwd_t<float>(feat, h, y, dm, st);
    if (dtype == GCG_BF16_F32) return fwd_t<bf16w_t>(feat, h, y, dm, st);
    if (dtype == GCG_F16_F32) return fwd_t<f16w_t>(feat, h, y, dm, st);
    return (int)hipErrorInvalidValue;
}

size_t mfma_feat_bwd_workspace(int dtype, const Dims &dm)
{
    const bool split = dtype != GCG_BF16 && dtype != GCG_F16;
    const MfmaPlan p = plan_bwd_nw(dm, choose_nw_bwd_feat(split), dtype == GCG_F32 ? 4 : 2);
    return (size_t)p.nwg * p.nw * 128 * sizeof(float);
}

bool mfma_feat_supported(int dtype, const Dims &dm, int kf)
{
    // (the kernels walk five slices of the banded matrix whatever hl is: a shorter filter leaves the far ones zero)
    return kf >= 1 && kf <= FEAT_KF && mfma_supported(dtype, dm);
}

int mfma_il_fwd_feat_launch(int dtype, const void *raw, const void *wfeat, int kf, const void *h, void *y,
                            const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return fwd_feat_t<bf16_t>(raw, wfeat, kf, h, y, dm, st);
    if (dtype == GCG_F16) return fwd_feat_t<f16_t>(raw, wfeat, kf, h, y, dm, st);
    if (dtype == GCG_F32) return fwd_feat_t<float>(raw, wfeat, kf, h, y, dm, st);
    if (dtype == GCG_BF16_F32) return fwd_feat_t<bf16w_t>(raw, wfeat, kf, h, y, dm, st);
    if (dtype == GCG_F16_F32) return fwd_feat_t<f16w_t>(raw, wfeat, kf, h, y, dm, st);
    return (int)hipErrorInvalidValue;
}

int mfma_il_bwd_feat_launch(int dtype, const void *dy, const void *raw, const void *wfeat, int kf, const void *h,
                            void *dfeat, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return bwd_feat_t<bf16_t>(dy, raw, wfeat, kf, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_F16) return bwd_feat_t<f16_t>(dy, raw, wfeat, kf, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_F32) return bwd_feat_t<float>(dy, raw, wfeat, kf, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_BF16_F32) return bwd_feat_t<bf16w_t>(dy, raw, wfeat, kf, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_F16_F32) return bwd_feat_t<f16w_t>(dy, raw, wfeat, kf, h, dfeat, dh, ws, dm, st);
    return (int)hipErrorInvalidValue;
}

int mfma_il_bwd_launch(int dtype, const void *dy, const void *feat, const void *h, void *dfeat, void *dh,
                       void *ws, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return bwd_t<bf16_t>(dy, feat, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_F16) return bwd_t<f16_t>(dy, feat, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_F32) return bwd_t<float>(dy, feat, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_BF16_F32) return bwd_t<bf16w_t>(dy, feat, h, dfeat, dh, ws, dm, st);
    if (dtype == GCG_F16_F32) return bwd_t<f16w_t>(dy, feat, h, dfeat, dh, ws, dm, st);
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
