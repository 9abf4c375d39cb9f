// Backward of (featurizer conv -> Hyena-MR operator) in one kernel: from dy and the projection output `raw`
// straight to d raw, d wf and dh.  Neither the featurized tensor nor its gradient exists in memory: the
// features are made again from the raw rows (rounded like the featurizer's output), the gradient of the
// features is rounded like the operator's backward would have stored it and handed on through LDS to the
// featurizer's backward.  Per element the kernel moves 7 values (dy and 3 of raw in, 3 of d raw out).
//
// Nearly all of that is vector arithmetic on row pieces, and a SIMD issues one vector or matrix instruction at a
// time, so the instruction count is what bounds the kernel.  A workgroup splits its eight waves by role, one wave
// of each kind per SIMD, so that neither kind holds the other's registers (Toeplitz tiles, operand rings and
// filter-gradient tiles on one side; rows in flight, taps, queues and accumulators on the other) and both fit
// two waves per SIMD:
//   memory waves (0..3)  own the rows: a lane holds 4 consecutive time rows of 2 channels -- one 12-byte piece
//                        (C0 B0 | x0 C1 | B1 x1) per row, 384 contiguous bytes per row across 32 lanes -- loads
//                        them, makes features, operands and the gradient of the features, and accumulates d wf;
//   matrix waves (4..7)  own 16 channels each for the products y2 = T u, du = T' g2 and the filter-gradient tiles
//                        (operands from LDS, results to LDS), and in the row layout turn the gradient of the
//                        features into d raw and store it.
//
// Step k of a run (32 rows x 64 channels) has two barriers:
//   before the first   memory: gradient of the features of step k-1 from y2, du (LDS) -> LDS; x, B of step k from
//                              the raw ring -> u(k); g2(k+4) -> ring
//                      matrix: d raw of step k-2 from the gradient rows in LDS (its rows two back, which need the
//                              two rows after them) -> memory
//   between the two    matrix: operands of u(k), g2(k+4), 20 products -> y2(k), du(k), 9 filter-gradient products
//                      memory: rows of step k+5 arrive -> C and g2 of that step, raw ring; rows of step k+7
//                              requested; d wf of step k-1
// The raw rows wait in an LDS ring (7 steps) from their arrival, 5 steps ahead for the anti-causal product, to
// the step after their own, where d wf needs them again; dy waits in registers; the gradient rows of two steps
// are in LDS at a time.  A run goes one step beyond its end (products only, nothing accumulated) because its last
// two rows of d raw need the first two gradient rows of the next run.
#include "gcg_il_tile.h"
#include "gcg_rowvec.h"

#include <type_traits>

namespace gcg {
namespace {

constexpr int MR_KF = 3;          // featurizer taps the kernel is built for; shorter filters are zero-padded in front

template <typename T> struct MixGeo {
    typedef MT<T> M;
    static_assert(!M::SPLIT && M::ES == 2, "16-bit tensors with 16-bit arithmetic operands");
    static constexpr int XW = 4, MW = 4, NT = 64 * (XW + MW);
    static constexpr int NK = 5, ND = 2 * NK - 1;
    static constexpr int CB = 16 * XW;                          // channels per workgroup
    static constexpr int UROW = CB * 2 + 16, YROW = CB * 4 + 16;    // LDS rows of u / g2 and of y2 / du (padded)
    static constexpr int LPR = CB / 2;                          // row lanes per row
    static constexpr int NR = 4, NG = STEP / NR;                // rows per lane, row groups
    static constexpr int NH = MR_KF - 1;                        // rows before a lane's own that its features need
    static constexpr int BLK = NR * 12;                         // a lane's rows of one step in a slot
    static constexpr int PRE = NG * LPR * BLK;                  // offset of the NH rows before the step (24 bytes a lane)
    static constexpr int PRE_BYTES = LPR * NH * 12;
    static constexpr int SLOT = PRE + PRE_BYTES;                // raw ring: a step's rows and the NH before them
    static constexpr int RAW_SLOTS = NK + 2;
    static constexpr int OFF_U = 0;
    static constexpr int OFF_G = OFF_U + STEP * UROW;
    static constexpr int OFF_Y = OFF_G + NK * STEP * UROW;
    static constexpr int OFF_D = OFF_Y + STEP * YROW;
    static constexpr int OFF_RAW = OFF_D + STEP * YROW;
    static constexpr int OFF_DF = OFF_RAW + RAW_SLOTS * SLOT;   // gradient rows of two steps, then three sets of a step's last NH rows
    static constexpr int OFF_DFP = OFF_DF + 2 * PRE;
    static constexpr int LDS_BYTES = OFF_DFP + 3 * PRE_BYTES;
    static constexpr int OFF_H = OFF_DF;                        // filter tables: read before the first gradient rows are written
    static constexpr int OFF_P = OFF_RAW;                       // tail: gradient tiles, then the d wf accumulators
    static constexpr int OFF_W = OFF_P + XW * ND * 1024;
    static constexpr int NACC = MR_KF * 6;
    static_assert(OFF_W + MW * 64 * NACC * 4 <= LDS_BYTES, "tail fits");
    static_assert(XW * HTAB * 2 <= PRE, "filter tables fit");
    static_assert(LDS_BYTES <= 160 * 1024, "workgroup exceeds the 160 KB of LDS");
    static_assert(OFF_RAW % 16 == 0 && SLOT % 16 == 0 && BLK % 16 == 0, "16-byte LDS accesses");
};

// Accesses without the streaming hint: the rows before a lane's own are its neighbour's rows, requested by both, and
// read twice from memory when the first request marks them for early eviction (measured: forward 116 -> 107 us,
// backward 4 % faster; for the stores it makes no difference in the backward and 3 us in the forward).
__device__ __forceinline__ u32x3 ldw12_cached(win_t w, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b96(w, (int)off, 0, 0);
}
__device__ __forceinline__ uint32_t ldw4_cached(win_t w, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b32(w, (int)off, 0, 0);
}
__device__ __forceinline__ void stw4_cached(win_t w, uint32_t off, uint32_t v)
{
    __builtin_amdgcn_raw_buffer_store_b32(v, w, (int)off, 0, 0);
}

// Planar features (PL; Dims::planar, the split without interleaving of block.py:881-884): a row holds the planes
// C | B | x one after the other, d elements each.  A lane's piece is then three words one plane apart, and its six
// values come plane by plane, C0 C1 | B0 B1 | x0 x1, instead of C0 B0 | x0 C1 | B1 x1.  That changes where a value
// sits in a piece (vi), which feature channel it is (feature_channel), and how a piece is loaded and stored; the
// rings, the featurizer's sums and the pairing of rows treat the six values alike.
template <bool PL> __device__ __forceinline__ constexpr int vi(int ch, int p) { return PL ? 2 * p + ch : 3 * ch + p; }
template <bool PL> __device__ __forceinline__ int64_t feature_channel(int64_t c, int v, int64_t d)
{
    return PL ? (int64_t)(v / 2) * d + c + v % 2 : 3 * c + v;
}
// off: the piece's offset in an interleaved row, or that of its first word in a planar one; plane: bytes of a plane
template <bool PL> __device__ __forceinline__ u32x3 piece_load_cached(win_t w, uint32_t off, uint32_t plane)
{
    if constexpr (PL)
        return u32x3{ldw4_cached(w, off), ldw4_cached(w, off + plane), ldw4_cached(w, off + 2 * plane)};
    else
        return ldw12_cached(w, off);
}
template <bool PL> __device__ __forceinline__ void piece_store(win_t w, uint32_t off, uint32_t plane, const u32x3 &v)
{
    if constexpr (PL) {
        stw4(w, off, v[0]);
        stw4(w, off + plane, v[1]);
        stw4(w, off + 2 * plane, v[2]);
    } else {
        stw12(w, off, v);
    }
}
// taps of a lane's six feature channels, oldest sample first, zero-padded in front to KF taps
template <typename T, int KF, bool PL>
__device__ __forceinline__ void lane_feat_taps(const T *wfeat, int64_t c, bool valid, int64_t d, int kf, float (&tap)[KF][6])
{
    if constexpr (PL) {
#pragma unroll
        for (int v = 0; v < 6; ++v) {
            const T *wp = wfeat + (valid ? feature_channel<true>(c, v, d) : 0) * kf;
#pragma unroll
            for (int m = 0; m < KF; ++m) {
                const int kk = m - (KF - kf);                // index into the kf taps of the filter
                const float t = Elem<T>::load(wp + (kk >= 0 ? kk : 0));
                tap[m][v] = kk >= 0 ? t : 0.f;
            }
        }
    } else {
        load_feat_taps<T, KF, 6>(wfeat, valid ? 3 * c : 0, kf, tap);
    }
}

struct Blk { uint4 w[3]; };       // four 12-byte pieces
struct Halo { uint2 w[3]; };      // two 12-byte pieces

__device__ __forceinline__ void blk_pieces(const Blk &b, u32x3 *p)
{
    const uint32_t v[12] = {b.w[0].x, b.w[0].y, b.w[0].z, b.w[0].w, b.w[1].x, b.w[1].y,
                            b.w[1].z, b.w[1].w, b.w[2].x, b.w[2].y, b.w[2].z, b.w[2].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = u32x3{v[3 * i], v[3 * i + 1], v[3 * i + 2]};
}
__device__ __forceinline__ Blk pieces_blk(const u32x3 *p)
{
    Blk b;
    b.w[0] = make_uint4(p[0][0], p[0][1], p[0][2], p[1][0]);
    b.w[1] = make_uint4(p[1][1], p[1][2], p[2][0], p[2][1]);
    b.w[2] = make_uint4(p[2][2], p[3][0], p[3][1], p[3][2]);
    return b;
}
__device__ __forceinline__ void halo_pieces(const Halo &h, u32x3 *p)
{
    p[0] = u32x3{h.w[0].x, h.w[0].y, h.w[1].x};
    p[1] = u32x3{h.w[1].y, h.w[2].x, h.w[2].y};
}
__device__ __forceinline__ Halo pieces_halo(const u32x3 *p)
{
    Halo h;
    h.w[0] = make_uint2(p[0][0], p[0][1]);
    h.w[1] = make_uint2(p[0][2], p[1][0]);
    h.w[2] = make_uint2(p[1][1], p[1][2]);
    return h;
}
__device__ __forceinline__ Blk lds_load_blk(const unsigned char *p)
{
    Blk b;
#pragma unroll
    for (int i = 0; i < 3; ++i) b.w[i] = *(const uint4 *)(p + 16 * i);
    return b;
}
__device__ __forceinline__ void lds_store_blk(unsigned char *p, const Blk &b)
{
#pragma unroll
    for (int i = 0; i < 3; ++i) *(uint4 *)(p + 16 * i) = b.w[i];
}
__device__ __forceinline__ Halo lds_load_halo(const unsigned char *p)
{
    Halo h;
#pragma unroll
    for (int i = 0; i < 3; ++i) h.w[i] = *(const uint2 *)(p + 8 * i);
    return h;
}
__device__ __forceinline__ void lds_store_halo(unsigned char *p, const Halo &h)
{
#pragma unroll
    for (int i = 0; i < 3; ++i) *(uint2 *)(p + 8 * i) = h.w[i];
}
// values of a piece in its own order: C0 B0 x0 C1 B1 x1
template <typename T> __device__ __forceinline__ void piece_values(const u32x3 &p, float (&v)[6])
{
    MT<T>::unpack2(p[0], v[0], v[1]);
    MT<T>::unpack2(p[1], v[2], v[3]);
    MT<T>::unpack2(p[2], v[4], v[5]);
}
template <typename T> __device__ __forceinline__ u32x3 values_piece(const float (&v)[6])
{
    return u32x3{MT<T>::pack2(v[0], v[1]), MT<T>::pack2(v[2], v[3]), MT<T>::pack2(v[4], v[5])};
}
// a.lo * b.lo + a.hi * b.hi + c on packed 16-bit pairs (the sum may differ from two fused multiply-adds in the
// last place of fp32: used where partial sums are added in another order anyway)
template <typename T> __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c);
template <> __device__ __forceinline__ float dot2<bf16_t>(uint32_t a, uint32_t b, float c)
{
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    return __builtin_amdgcn_fdot2_f32_bf16(x, y, c, false);
}
template <> __device__ __forceinline__ float dot2<f16_t>(uint32_t a, uint32_t b, float c)
{
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    return __builtin_amdgcn_fdot2(x, y, c, false);
}
// the low (high) halves of two dwords as one pair: first dword's in the low half
__device__ __forceinline__ uint32_t pair_lo(uint32_t first, uint32_t second)
{
    return __builtin_amdgcn_perm(second, first, 0x05040100u);
}
__device__ __forceinline__ uint32_t pair_hi(uint32_t first, uint32_t second)
{
    return __builtin_amdgcn_perm(second, first, 0x07060302u);
}

// one feature value: the featurizer kernel's order of summation (oldest sample first, fp32)
__device__ __forceinline__ float feat_sum(const float (&tap)[MR_KF][6], const float (&rv)[MR_KF - 1 + 4][6], int k, int v)
{
    float acc = 0.f;
#pragma unroll
    for (int m = 0; m < MR_KF; ++m) acc = fmaf(tap[m][v], rv[k + m][v], acc);
    return acc;
}

// Tail of the backward, run by every wave: the workgroup that finishes a channel block's last run adds the block's
// partial sums of dh and d wf in a fixed order (so the results do not depend on which workgroup that is) and writes
// the gradients; without pl.fuse_dh two small launches do it.
template <typename T, bool PL>
__device__ __forceinline__ void mixer_bwd_finish(const float *ws, const float *wsf, T *__restrict__ dh,
                                                 T *__restrict__ dwf, const Dims &dm, const MfmaPlan &pl, int cb, int kf)
{
    typedef MixGeo<T> G;
    if (!pl.fuse_dh) return;
    const int tid = threadIdx.x;
    if (!dh_arrive_last(pl, cb, (unsigned int)(dm.bs * pl.nseg))) return;
    const int64_t np = dm.bs * pl.nseg;
    {
        const int gpc = G::CB / dm.dg, bpg = dm.dg / 16;   // filter groups per channel block, 16-channel blocks per group
        const int row = dm.fw ? dm.lc : dm.hl;              // taps per group in the output
        for (int idx = tid; idx < gpc * row; idx += G::NT) {
            const int gl = idx / row, k = idx % row;
            const int64_t grp = (int64_t)cb * gpc + gl;
            if (grp >= dm.g) continue;
            if (k >= dm.hl) {                                // the parameter's taps beyond the filter in use
                ((float *)dh)[grp * row + k] = 0.f;
                continue;
            }
            const int lag = dm.hl - 1 - k;
            float sum = 0.f;
            for (int64_t p = 0; p < np; ++p)
                for (int kk = 0; kk < bpg; ++kk)
                    sum += __hip_atomic_load(ws + ((p * pl.ncb + cb) * G::XW + gl * bpg + kk) * 128 + lag, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
            store_dh<T>(dh, dm, grp, k, sum);
        }
    }
    const int64_t nf = 3 * dm.d;
    for (int idx = tid; idx < kf * 3 * G::CB; idx += G::NT) {
        const int kk = idx / (3 * G::CB), col = idx % (3 * G::CB);
        // the block's feature channels: 3 * CB consecutive ones, or CB of each plane
        const int64_t f = PL ? (int64_t)(col / G::CB) * dm.d + (int64_t)cb * G::CB + col % G::CB : (int64_t)cb * 3 * G::CB + col;
        if (PL ? (int64_t)cb * G::CB + col % G::CB >= dm.d : f >= nf) continue;
        float sum = 0.f;
        for (int64_t p = 0; p < np; ++p)
            sum += __hip_atomic_load(wsf + ((size_t)kk * np + p) * nf + f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        Elem<T>::store(dwf + f * kf + kk, sum);
    }
}

template <typename T, bool PL = false>
__global__ __launch_bounds__(MixGeo<T>::NT) void mixer_mr_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ raw,
                                                                    const T *__restrict__ h, const T *__restrict__ wfeat,
                                                                    int kf, T *__restrict__ draw, T *__restrict__ dh,
                                                                    T *__restrict__ dwf, float *__restrict__ ws,
                                                                    float *__restrict__ wsf, Dims dm, MfmaPlan pl)
{
    typedef MT<T> M;
    typedef typename M::op_t op_t;
    typedef typename M::hraw_t hraw_t;
    typedef MixGeo<T> G;
    constexpr int NK = G::NK, ND = G::ND, XW = G::XW, MW = G::MW, CB = G::CB, UROW = G::UROW, YROW = G::YROW;
    constexpr int LPR = G::LPR, NR = G::NR, NH = G::NH, KF = MR_KF, NV = 6;
    constexpr int RING_ROWS = STEP * NK;
    __shared__ __attribute__((aligned(16))) unsigned char smem[G::LDS_BYTES];
    unsigned char *u_rm = smem + G::OFF_U, *g_rm = smem + G::OFF_G, *y_st = smem + G::OFF_Y, *d_st = smem + G::OFF_D;
    unsigned char *raw_rg = smem + G::OFF_RAW, *df_rg = smem + G::OFF_DF;
    hraw_t *htab = (hraw_t *)(smem + G::OFF_H);

    const int64_t wg_id = xcd_contiguous_id(blockIdx.x, gridDim.x);
    int64_t wg = wg_id;
    const int cb = (int)(wg % pl.ncb); wg /= pl.ncb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const bool is_m = w < MW;
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;
    const int64_t s_end = s_hi + 1;      // one step beyond the run: its first gradient rows complete the run's last rows of d raw
    const int64_t k_first = s_lo - (NK - 1);                    // u of the NK-1 steps before the run is made again

    // Row layout, used by the memory waves for everything and by the matrix waves for d raw: lane (rr, a) of its
    // kind owns rows NR*rr .. NR*rr+3 of a step and channels c0 + 2a, 2a+1.
    const int rt = tid & (64 * MW - 1), rr = rt / LPR, a = rt % LPR;
    const bool cvalid = c0 + 2 * a < d;
    const int64_t row_bytes = d * 2;
    const int64_t T0 = s_lo * STEP, T1 = s_hi * STEP < L ? s_hi * STEP : L;
    // Offsets are 32-bit sums of a lane part, a step part (uniform, advanced by one step's bytes per iteration) and
    // a row part; positions before a window's origin wrap to offsets far outside it, where loads return zero and
    // stores are dropped, and lanes whose channels lie beyond the tensor add WIN_OFF.
    const uint32_t rb = (uint32_t)row_bytes, bad = cvalid ? 0u : WIN_OFF, step_b = (uint32_t)STEP * rb;
    const uint32_t col_b = (uint32_t)((c0 + 2 * a) * 2);
    const uint32_t lane_raw = PL ? 3u * ((uint32_t)(NR * rr - NH) * rb) + col_b + bad
                                 : 3u * ((uint32_t)(NR * rr - NH) * rb + col_b) + bad;     // row NR*rr-NH of a step
    auto step_base = [&](int64_t step, int64_t origin) { return (uint32_t)((step * STEP - origin) * row_bytes); };
    float tap[KF][NV];
    lane_feat_taps<T, KF, PL>(wfeat, c0 + 2 * a, cvalid, d, kf, tap);
    const int own_off = (rr * LPR + a) * G::BLK;                                   // own rows in a slot
    const int halo_off = rr ? ((rr - 1) * LPR + a) * G::BLK + 24 : G::PRE + a * 24;    // the NH rows before them

    if (!is_m) {
        // ------------------------------------------------------------------ matrix waves
        const int xw = w - MW, j = l & 15, q = l >> 4;
        const bool wave_valid = c0 + 16 * xw < d;
        hraw_t hv[HTAB / 64];
        load_taps<T>(dm, h, wave_valid ? (c0 + 16 * xw) / dm.dg : 0, l, hv);
        store_taps(htab + xw * HTAB, l, hv);
        __syncthreads();
        typename M::wop_t W0[NK], W1[NK];
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            W0[i] = M::toeplitz(htab + xw * HTAB, 32 * i, j, q);
            W1[i] = M::toeplitz(htab + xw * HTAB, 32 * i + 16, j, q);
        }
        __syncthreads();      // the filter tables have been read: their place becomes the gradient rows

        op_t Au[NK], Ag[NK];
        f32x4 P[ND];
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            Au[i] = M::zero_op();
            Ag[i] = M::zero_op();
        }
#pragma unroll
        for (int i = 0; i < ND; ++i) P[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        unsigned char *y_wr = y_st + j * YROW + (16 * xw + 4 * q) * 4;
        unsigned char *d_wr = d_st + (15 - j) * YROW + (16 * xw + 4 * q) * 4;      // columns come out reversed
        // d raw, from the gradient rows the memory waves leave in LDS, two steps behind the products
        const win_t wdr = make_window(draw + 3 * (b * L + T0) * d, 3 * (T1 - T0) * row_bytes);
        uint32_t dr_b = 3u * step_base(s_lo, T0);      // of step k-2
        const unsigned char *df_own = df_rg + own_off;
        const unsigned char *df_halo = rr ? df_rg + halo_off : smem + G::OFF_DFP + a * 24;
        int dfb = 0;                                    // which of the two sets of gradient rows step k-2 lies in
        int dfp = 2 * G::PRE_BYTES;                     // where the NH rows before step k-2 lie (row group 0 only)
        u32x3 dro[NR];                                  // the rows of d raw stored last
#pragma unroll
        for (int r = 0; r < NR; ++r) dro[r] = u32x3{0u, 0u, 0u};

        // While step k runs in phase ph:  Au[(ph - i + NK) % NK] is the u operand of step k-i,
        // Ag[(ph + i) % NK] the time-reversed g2 operand of step k+i (ring slot (ph + i) % NK).
        int64_t k = k_first;
        while (k <= s_end + 1) {
#pragma unroll
            for (int ph = 0; ph < NK; ++ph) {
                if (k <= s_end + 1) {
                    if (k - 2 >= s_lo) {
                        // d raw of rows NR*rr-NH .. NR*rr+NR-NH-1 of step k-2: each needs the gradient rows from its own on
                        u32x3 pg[NH + NR];
                        halo_pieces(lds_load_halo(df_halo + (rr ? dfb : dfp)), pg);
                        blk_pieces(lds_load_blk(df_own + dfb), pg + NH);
                        float gv[NH + NR][NV];
#pragma unroll
                        for (int i = 0; i < NH + NR; ++i) piece_values<T>(pg[i], gv[i]);
                        // The stored rows keep registers of their own until here, one step later: a register that is
                        // written again while its store is still on the way makes the wave wait for that store.
#pragma unroll
                        for (int i = 0; i < NR; ++i) asm volatile("" ::"v"(dro[i][0]), "v"(dro[i][1]), "v"(dro[i][2]));
#pragma unroll
                        for (int i = 0; i < NR; ++i) {
                            float o[NV];
#pragma unroll
                            for (int v = 0; v < NV; ++v) {
                                float acc = 0.f;             // the featurizer backward's order: nearest row first
#pragma unroll
                                for (int m = KF - 1; m >= 0; --m) acc = fmaf(tap[m][v], gv[i + KF - 1 - m][v], acc);
                                o[v] = acc;
                            }
                            dro[i] = values_piece<T>(o);
                        }
#pragma unroll
                        for (int i = 0; i < NR; ++i) piece_store<PL>(wdr, lane_raw + dr_b + 3u * (uint32_t)i * rb, rb, dro[i]);
                        dr_b += 3u * step_b;
                        dfb ^= G::PRE;
                        dfp = dfp == 2 * G::PRE_BYTES ? 0 : dfp + G::PRE_BYTES;
                    }
                    __syncthreads();
                    if (k < s_end) {
                        const int slot_new = (ph + NK - 1) % NK;
                        Au[ph] = M::load_operand(u_rm, UROW, xw, j, q, false);
                        Ag[slot_new] = M::load_operand(g_rm + slot_new * STEP * UROW, UROW, xw, j, q, true);
                        if (k >= s_lo) {
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
                            if (k < s_hi) {
                                // filter-gradient tiles: natural-layout operands (rows j and 16+j of a 32-row window)
                                const op_t un = M::load_natural(u_rm + j * UROW, u_rm + (16 + j) * UROW, UROW, xw, q);
#pragma unroll
                                for (int dl = 0; dl < ND; ++dl) {
                                    int row0 = STEP * ph + 16 * dl + j;          // ring rows of the window's two halves
                                    int row1 = row0 + 16;
                                    row0 = (row0 >= RING_ROWS) ? row0 - RING_ROWS : row0;
                                    row1 = (row1 >= RING_ROWS) ? row1 - RING_ROWS : row1;
                                    const op_t gn = M::load_natural(g_rm + row0 * UROW, g_rm + row1 * UROW, UROW, xw, q);
                                    P[dl] = M::mfma_aa(gn, un, P[dl]);
                                }
                            }
                        }
                    }
                    __syncthreads();
                    ++k;
                }
            }
        }
        // gradient tiles -> LDS for the diagonal sums
        float *pt = (float *)(smem + G::OFF_P) + xw * ND * 256;
#pragma unroll
        for (int dl = 0; dl < ND; ++dl)
#pragma unroll
            for (int v = 0; v < 4; ++v) pt[dl * 256 + (4 * q + v) * 16 + j] = P[dl][v];
        __syncthreads();
        if (wave_valid) {
            float *out = ws + ((size_t)wg_id * XW + xw) * 128;
            for (int lag = l; lag < 128; lag += 64) {
                const int d0 = lag >> 4, r = lag & 15;
                float sum = 0.f;
                if (d0 < ND)
                    for (int jj = 0; jj + r < 16; ++jj) sum += pt[d0 * 256 + (jj + r) * 16 + jj];
                if (d0 + 1 < ND)
                    for (int ii = 0; ii < r; ++ii) sum += pt[(d0 + 1) * 256 + ii * 16 + ii + 16 - r];
                __hip_atomic_store(out + lag, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        mixer_bwd_finish<T, PL>(ws, wsf, dh, dwf, dm, pl, cb, kf);
        return;
    }

    // ---------------------------------------------------------------------- memory waves
    // the rows read: from the NK-1 steps before the run (and the NH rows before those) to the NK-1 steps after
    // the last step worked on; what lies outside reads as zero
    const int64_t t0 = k_first * STEP > 0 ? k_first * STEP : 0;
    const int64_t tf = t0 - NH > 0 ? t0 - NH : 0;
    const int64_t t2 = (s_end + NK - 1) * STEP < L ? (s_end + NK - 1) * STEP : L;
    const win_t wraw = make_window(raw + 3 * (b * L + tf) * d, 3 * (t2 - tf) * row_bytes);
    const win_t wdy = make_window(dy + (b * L + t0) * d, (t2 - t0) * row_bytes);
    const uint32_t lane_dy = (uint32_t)(NR * rr) * rb + col_b + bad;                    // row NR*rr

    // LDS addresses of this lane
    unsigned char *u_own = u_rm + NR * rr * UROW + 4 * a;
    unsigned char *g_own = g_rm + NR * rr * UROW + 4 * a;
    const unsigned char *y_rd = y_st + NR * rr * YROW + 8 * a;
    const unsigned char *d_rd = d_st + NR * rr * YROW + 8 * a;
    unsigned char *raw_own = raw_rg + own_off, *raw_halo = raw_rg + halo_off;
    unsigned char *df_own = df_rg + own_off, *df_last = smem + G::OFF_DFP + a * 24;

    // rows of a step: the NH rows before the lane's own, its NR rows, and dy of those
    struct Rows { u32x3 p[NH + NR]; uint32_t dy[NR]; };
    auto fetch = [&](Rows &r, uint32_t raw_base, uint32_t dy_base) {
#pragma unroll
        for (int i = 0; i < NH + NR; ++i) r.p[i] = piece_load_cached<PL>(wraw, lane_raw + 3u * (raw_base + (uint32_t)i * rb), rb);
#pragma unroll
        for (int i = 0; i < NR; ++i) r.dy[i] = ldw4_cached(wdy, lane_dy + dy_base + (uint32_t)i * rb);
    };

    uint32_t dq[NK + 1][NR];          // dy of the steps between arrival and their own gradient, oldest first
    uint32_t g2n[NR];                 // g2 of the step that arrived last, as it goes into the ring
#pragma unroll
    for (int i = 0; i <= NK; ++i)
#pragma unroll
        for (int r = 0; r < NR; ++r) dq[i][r] = 0u;

    // what arrived rows bring: the rows into the ring slot at byte offset `slot`, C of the step and with it g2
    auto arrive = [&](const Rows &r, int slot) {
        float rv[NH + NR][NV];
#pragma unroll
        for (int i = 0; i < NH + NR; ++i) piece_values<T>(r.p[i], rv[i]);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            float c0r, c1r, d0, d1;
            M::unpack2(M::pack2(feat_sum(tap, rv, i, vi<PL>(0, 0)), feat_sum(tap, rv, i, vi<PL>(1, 0))), c0r, c1r);
            M::unpack2(r.dy[i], d0, d1);
            g2n[i] = M::pack2(d0 * c0r, d1 * c1r);
        }
#pragma unroll
        for (int q = 0; q < NK; ++q)
#pragma unroll
            for (int i = 0; i < NR; ++i) dq[q][i] = dq[q + 1][i];
#pragma unroll
        for (int i = 0; i < NR; ++i) dq[NK][i] = r.dy[i];
        // (the ring is written after the arithmetic: the matrix waves read their operands at the same time)
        lds_store_blk(raw_own + slot, pieces_blk(r.p + NH));
        if (rr == 0) lds_store_halo(raw_halo + slot, pieces_halo(r.p));
    };

    // Lead-in: the steps k_first .. s_lo are requested together and arrive in order (their dy too, though the g2 of
    // the NK-1 steps before the run is never used), then the rows of steps s_lo+1 and s_lo+2 are requested.
    uint32_t raw_b = step_base(k_first, tf), dy_b = step_base(k_first, t0);    // of the step requested next
    Rows in0, in1;                    // rows on the way, requested two steps before they are taken up
    {
        Rows lead[NK];
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            fetch(lead[i], raw_b, dy_b);
            raw_b += step_b;
            dy_b += step_b;
        }
        fetch(in0, raw_b, dy_b);
        raw_b += step_b;
        dy_b += step_b;
        fetch(in1, raw_b, dy_b);
        raw_b += step_b;
        dy_b += step_b;
#pragma unroll
        for (int i = 0; i < NK; ++i) arrive(lead[i], i * G::SLOT);
    }
    __syncthreads();
    __syncthreads();

    float dwa[KF][NV];                // d wf of the lane's 6 feature channels
#pragma unroll
    for (int m = 0; m < KF; ++m)
#pragma unroll
        for (int v = 0; v < NV; ++v) dwa[m][v] = 0.f;
    float xk[NR][2], Bk[NR][2];       // x, B of the step whose products are under way
#pragma unroll
    for (int r = 0; r < NR; ++r) { xk[r][0] = xk[r][1] = 0.f; Bk[r][0] = Bk[r][1] = 0.f; }

    constexpr int RING_END = (G::RAW_SLOTS - 1) * G::SLOT;
    int rs = 0;                       // byte offset of the raw ring slot of step k
    int ra = NK * G::SLOT;            // ... of step k+NK, which arrives during step k (two slots behind step k)
    int gs = (NK - 1) * STEP * UROW;  // byte offset of the g2 ring slot of step k+NK-1
    int dfb = 0;                      // which of the two sets of gradient rows step k-1 goes into
    int dfp = 0;                      // where the last row group leaves its last NH rows of step k-1 for the step after

    // One step.  PREV: step k-1 has products (gradient of its features); DWF: it also counts for d wf (it lies
    // inside the run); MAKE: step k gets its u and step k+NK-1 its g2.  The variants are separate straight-line
    // bodies, so that within each the LDS reads can all be requested before the first use.
    auto iter = [&](auto prev_c, auto dwf_c, auto make_c, Rows &in) {
        constexpr bool PREV = decltype(prev_c)::value, DWF = decltype(dwf_c)::value, MAKE = decltype(make_c)::value;
        const int rs_prev = rs ? rs - G::SLOT : RING_END;
        float2 y2v[NR], duv[NR];
        u32x3 prc[NH + NR], po[NR];
        if constexpr (PREV) {
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                y2v[i] = *(const float2 *)(y_rd + i * YROW);
                duv[i] = *(const float2 *)(d_rd + i * YROW);
            }
        }
        if constexpr (MAKE) {
            halo_pieces(lds_load_halo(raw_halo + rs), prc);
            blk_pieces(lds_load_blk(raw_own + rs), prc + NH);
        }
        if constexpr (PREV) {
            // gradient of the features of step k-1 -> LDS, where the matrix waves turn it into d raw
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                float dv[2], o[NV];
                M::unpack2(dq[0][i], dv[0], dv[1]);
                o[vi<PL>(0, 0)] = dv[0] * y2v[i].x; o[vi<PL>(0, 1)] = duv[i].x * xk[i][0]; o[vi<PL>(0, 2)] = duv[i].x * Bk[i][0];
                o[vi<PL>(1, 0)] = dv[1] * y2v[i].y; o[vi<PL>(1, 1)] = duv[i].y * xk[i][1]; o[vi<PL>(1, 2)] = duv[i].y * Bk[i][1];
                po[i] = values_piece<T>(o);
            }
            lds_store_blk(df_own + dfb, pieces_blk(po));
            if (rr == G::NG - 1) lds_store_halo(df_last + dfp, pieces_halo(po + NR - NH));
            dfb ^= G::PRE;
            dfp = dfp == 2 * G::PRE_BYTES ? 0 : dfp + G::PRE_BYTES;
        }
        if constexpr (MAKE) {
            // x, B of step k -> u; g2 of step k+NK-1 -> ring
            float rv[NH + NR][NV];
#pragma unroll
            for (int i = 0; i < NH + NR; ++i) piece_values<T>(prc[i], rv[i]);
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                // rounded to the tensors' type like the featurizer's output, then kept as fp32 for the gradient
                M::unpack2(M::pack2(feat_sum(tap, rv, i, vi<PL>(0, 1)), feat_sum(tap, rv, i, vi<PL>(1, 1))), Bk[i][0], Bk[i][1]);
                M::unpack2(M::pack2(feat_sum(tap, rv, i, vi<PL>(0, 2)), feat_sum(tap, rv, i, vi<PL>(1, 2))), xk[i][0], xk[i][1]);
                *(uint32_t *)(u_own + i * UROW) = M::pack2(xk[i][0] * Bk[i][0], xk[i][1] * Bk[i][1]);
                *(uint32_t *)(g_own + gs + i * UROW) = g2n[i];
            }
        }
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);           // what follows runs beside the matrix waves' products, not before them
        // The rows of step k+NK arrive (the ring slot two behind step k).  They are taken up before anything else is
        // sent to memory, so that waiting for them does not wait for younger accesses; then the rows of step
        // k+NK+2 are requested into the same registers.
        arrive(in, ra);
#pragma unroll
        for (int i = 0; i < NR; ++i) asm volatile("" : "+v"(g2n[i]), "+v"(dq[NK][i]));
        __builtin_amdgcn_sched_barrier(0);
        fetch(in, raw_b, dy_b);
        raw_b += step_b;
        dy_b += step_b;
        if constexpr (DWF) {
            // d wf: each gradient row of step k-1 with the raw rows its feature was made of, two rows per product:
            // value v of rows (i, i+1) of the gradient with value v of rows (i+m, i+m+1)
            u32x3 prp[NH + NR];
            halo_pieces(lds_load_halo(raw_halo + rs_prev), prp);
            blk_pieces(lds_load_blk(raw_own + rs_prev), prp + NH);
            uint32_t rp[NH + NR - 1][NV], gp[NR / 2][NV];
#pragma unroll
            for (int i = 0; i < NH + NR - 1; ++i)
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    rp[i][2 * c] = pair_lo(prp[i][c], prp[i + 1][c]);
                    rp[i][2 * c + 1] = pair_hi(prp[i][c], prp[i + 1][c]);
                }
#pragma unroll
            for (int i = 0; i < NR / 2; ++i)
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    gp[i][2 * c] = pair_lo(po[2 * i][c], po[2 * i + 1][c]);
                    gp[i][2 * c + 1] = pair_hi(po[2 * i][c], po[2 * i + 1][c]);
                }
#pragma unroll
            for (int i = 0; i < NR / 2; ++i)
#pragma unroll
                for (int m = 0; m < KF; ++m)
#pragma unroll
                    for (int v = 0; v < NV; ++v) dwa[m][v] = dot2<T>(gp[i][v], rp[2 * i + m][v], dwa[m][v]);
        }
        rs = rs == RING_END ? 0 : rs + G::SLOT;
        ra = ra == RING_END ? 0 : ra + G::SLOT;
        gs = gs == (NK - 1) * STEP * UROW ? 0 : gs + STEP * UROW;
        __syncthreads();
    };
    {
        const std::true_type yes;
        const std::false_type no;
        int64_t k = k_first;
        bool odd = false;             // which of in0, in1 holds the rows that arrive in this step
        for (; k <= s_lo; ++k, odd = !odd) {                // the steps before the run: operands only
            if (odd) iter(no, no, yes, in1);
            else iter(no, no, yes, in0);
        }
        if (odd && k < s_end) {
            iter(yes, yes, yes, in1);
            ++k;
            odd = false;
        }
        for (; k + 1 < s_end; k += 2) {
            iter(yes, yes, yes, in0);
            iter(yes, yes, yes, in1);
        }
        if (k < s_end) {
            iter(yes, yes, yes, in0);
            odd = true;
        }
        if (odd) iter(yes, no, no, in1);                        // the step beyond the run gives its gradient rows
        else iter(yes, no, no, in0);
        __syncthreads();                                    // one more step of the matrix waves: d raw lags two steps
        __syncthreads();
    }
    // d wf: the row groups' sums, then one partial row per run (the first barrier is the one of the matrix waves' tail)
    float *wacc = (float *)(smem + G::OFF_W);
#pragma unroll
    for (int m = 0; m < KF; ++m)
#pragma unroll
        for (int v = 0; v < NV; ++v) wacc[(m * G::NG + rr) * (LPR * NV) + a * NV + v] = dwa[m][v];
    __syncthreads();
    const int64_t prow = b * pl.nseg + seg, nprow = dm.bs * pl.nseg;
    for (int idx = tid; idx < KF * LPR * NV; idx += 64 * MW) {
        const int m = idx / (LPR * NV), col = idx % (LPR * NV);
        const int kk = m - (KF - kf);                           // index into the kf taps of the filter
        // column a * NV + v: value v of the lane that owns channels c0 + 2a, 2a+1
        const int64_t f = PL ? feature_channel<true>(c0 + 2 * (col / NV), col % NV, d) : 3 * c0 + col;
        if (kk < 0 || (PL ? c0 + 2 * (col / NV) + (col % NV) % 2 >= d : f >= 3 * d)) continue;
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < G::NG; ++r) sum += wacc[(m * G::NG + r) * (LPR * NV) + col];
        __hip_atomic_store(wsf + ((size_t)kk * nprow + prow) * (3 * d) + f, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    mixer_bwd_finish<T, PL>(ws, wsf, dh, dwf, dm, pl, cb, kf);
}

// ---------------------------------------------------------------------------- forward
// The same division of labour for y = C * (T u), u = x * B, with the features made from the projection output on
// the way.  The forward has no ring to keep and few registers per wave, so a workgroup takes sixteen waves and 128
// channels: rows of 768 bytes in, 256 bytes out (with 64 channels and two workgroups per CU, 130 us at the 7B shape
// against 118: the 128-byte pieces of y are what costs).  Step k (32 rows):
//   before the first barrier   memory: u(k) (made during the step before) -> LDS; y of step k-1 = C * y2 -> memory
//   between the two            matrix: operand of u(k), 10 products -> y2(k)
//                              memory: the rows of step k+1 arrive -> its features, u and C; rows of step k+3 requested
template <typename T> struct MixFwdGeo {
    typedef MT<T> M;
    static_assert(!M::SPLIT && M::ES == 2, "16-bit tensors with 16-bit arithmetic operands");
    static constexpr int XW = 8, MW = 8, NT = 64 * (XW + MW);
    static constexpr int NK = 5;
    static constexpr int CB = 16 * XW;
    static constexpr int UROW = CB * 2 + 16, YROW = CB * 4 + 16;
    static constexpr int LPR = CB / 2, NR = 4, NH = MR_KF - 1;
    static constexpr int OFF_U = 0;
    static constexpr int OFF_Y = OFF_U + STEP * UROW;
    static constexpr int OFF_H = OFF_Y;                         // filter tables: read before the first y2 tile is written
    static constexpr int LDS_BYTES = OFF_Y + STEP * YROW;
    static_assert(XW * HTAB * 2 <= STEP * YROW, "filter tables fit");
};

template <typename T, bool PL = false>
__global__ __launch_bounds__(MixFwdGeo<T>::NT) void mixer_mr_fwd_kernel(const T *__restrict__ raw, const T *__restrict__ h,
                                                                       const T *__restrict__ wfeat, int kf,
                                                                       T *__restrict__ y, Dims dm, MfmaPlan pl)
{
    typedef MT<T> M;
    typedef typename M::op_t op_t;
    typedef typename M::hraw_t hraw_t;
    typedef MixFwdGeo<T> G;
    constexpr int NK = G::NK, MW = G::MW, CB = G::CB, UROW = G::UROW, YROW = G::YROW;
    constexpr int LPR = G::LPR, NR = G::NR, NH = G::NH, KF = MR_KF, NV = 6;
    __shared__ __attribute__((aligned(16))) unsigned char smem[G::LDS_BYTES];
    unsigned char *u_rm = smem + G::OFF_U, *y_st = smem + G::OFF_Y;
    hraw_t *htab = (hraw_t *)(smem + G::OFF_H);

    const int64_t wg_id = xcd_contiguous_id(blockIdx.x, gridDim.x);
    int64_t wg = wg_id;
    const int cb = (int)(wg % pl.ncb); wg /= pl.ncb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;
    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;
    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;
    const int64_t k_first = s_lo - (NK - 1);                    // u of the NK-1 steps before the run is made again

    if (w >= MW) {
        // ------------------------------------------------------------------ matrix waves
        const int xw = w - MW, j = l & 15, q = l >> 4;
        hraw_t hv[HTAB / 64];
        load_taps<T>(dm, h, (c0 + 16 * xw < d) ? (c0 + 16 * xw) / dm.dg : 0, l, hv);
        store_taps(htab + xw * HTAB, l, hv);
        __syncthreads();
        typename M::wop_t W0[NK], W1[NK];   // output rows 0..15 / 16..31 of the step against input step k-i
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            W0[i] = M::toeplitz(htab + xw * HTAB, 32 * i, j, q);
            W1[i] = M::toeplitz(htab + xw * HTAB, 32 * i + 16, j, q);
        }
        __syncthreads();      // the filter tables have been read: their place becomes the y2 tile
        op_t Au[NK];
#pragma unroll
        for (int i = 0; i < NK; ++i) Au[i] = M::zero_op();
        unsigned char *y_wr = y_st + j * YROW + (16 * xw + 4 * q) * 4;
        int64_t k = k_first;
        while (k <= s_hi) {
#pragma unroll
            for (int ph = 0; ph < NK; ++ph) {
                if (k <= s_hi) {
                    __syncthreads();
                    if (k < s_hi) {
                        Au[ph] = M::load_operand(u_rm, UROW, xw, j, q, false);
                        if (k >= s_lo) {
                            f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                            for (int i = 0; i < NK; ++i) {
                                acc0 = M::mfma(Au[(ph - i + NK) % NK], W0[i], acc0);
                                acc1 = M::mfma(Au[(ph - i + NK) % NK], W1[i], acc1);
                            }
                            *(f32x4 *)y_wr = acc0;
                            *(f32x4 *)(y_wr + 16 * YROW) = acc1;
                        }
                    }
                    __syncthreads();
                    ++k;
                }
            }
        }
        return;
    }

    // ---------------------------------------------------------------------- memory waves
    const int rr = tid / LPR, a = tid % LPR;        // rows NR*rr .. NR*rr+3, channels c0 + 2a, 2a+1
    const bool cvalid = c0 + 2 * a < d;
    const int64_t row_bytes = d * 2;
    const int64_t T0 = s_lo * STEP, T1 = s_hi * STEP < L ? s_hi * STEP : L;
    const int64_t t0 = k_first * STEP > 0 ? k_first * STEP : 0;
    const int64_t tf = t0 - NH > 0 ? t0 - NH : 0;
    const win_t wraw = make_window(raw + 3 * (b * L + tf) * d, 3 * (T1 - tf) * row_bytes);
    const win_t wy = make_window(y + (b * L + T0) * d, (T1 - T0) * row_bytes);
    const uint32_t rb = (uint32_t)row_bytes, bad = cvalid ? 0u : WIN_OFF, step_b = (uint32_t)STEP * rb;
    const uint32_t col_b = (uint32_t)((c0 + 2 * a) * 2);
    const uint32_t lane_raw = PL ? 3u * ((uint32_t)(NR * rr - NH) * rb) + col_b + bad
                                 : 3u * ((uint32_t)(NR * rr - NH) * rb + col_b) + bad;     // row NR*rr-NH of a step
    const uint32_t lane_y = (uint32_t)(NR * rr) * rb + col_b + bad;                     // row NR*rr
    auto step_base = [&](int64_t step, int64_t origin) { return (uint32_t)((step * STEP - origin) * row_bytes); };
    float tap[KF][NV];
    lane_feat_taps<T, KF, PL>(wfeat, c0 + 2 * a, cvalid, d, kf, tap);
    unsigned char *u_own = u_rm + NR * rr * UROW + 4 * a;
    const unsigned char *y_rd = y_st + NR * rr * YROW + 8 * a;

    struct Rows { u32x3 p[NH + NR]; };
    auto fetch = [&](Rows &r, uint32_t raw_base) {
#pragma unroll
        for (int i = 0; i < NH + NR; ++i) r.p[i] = piece_load_cached<PL>(wraw, lane_raw + 3u * (raw_base + (uint32_t)i * rb), rb);
    };
    uint32_t un[NR], cn[NR];          // u and C of the step that arrived last
    // what arrived rows bring: the features, rounded like the featurizer's output, and with them u and C
    auto arrive = [&](const Rows &r) {
        float rv[NH + NR][NV];
#pragma unroll
        for (int i = 0; i < NH + NR; ++i) piece_values<T>(r.p[i], rv[i]);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            float x0, x1, B0, B1;
            cn[i] = M::pack2(feat_sum(tap, rv, i, vi<PL>(0, 0)), feat_sum(tap, rv, i, vi<PL>(1, 0)));
            M::unpack2(M::pack2(feat_sum(tap, rv, i, vi<PL>(0, 1)), feat_sum(tap, rv, i, vi<PL>(1, 1))), B0, B1);
            M::unpack2(M::pack2(feat_sum(tap, rv, i, vi<PL>(0, 2)), feat_sum(tap, rv, i, vi<PL>(1, 2))), x0, x1);
            un[i] = M::pack2(x0 * B0, x1 * B1);
        }
#pragma unroll
        for (int i = 0; i < NR; ++i) asm volatile("" : "+v"(un[i]), "+v"(cn[i]));     // made here, not after younger loads
        __builtin_amdgcn_sched_barrier(0);
    };

    uint32_t raw_b = step_base(k_first, tf);        // of the step requested next
    Rows in0, in1;                                   // rows on the way, requested two steps before they are taken up
    fetch(in0, raw_b);
    raw_b += step_b;
    fetch(in1, raw_b);
    raw_b += step_b;
    __syncthreads();
    __syncthreads();
    arrive(in0);                                     // step k_first
    fetch(in0, raw_b);
    raw_b += step_b;

    uint32_t cp[NR], yo[NR];          // C of the step whose products are under way; the rows of y stored last
#pragma unroll
    for (int i = 0; i < NR; ++i) { cp[i] = 0u; yo[i] = 0u; }
    uint32_t y_b = step_base(s_lo, T0);              // of step k-1

    auto iter = [&](int64_t k, Rows &in) {
        if (k < s_hi) {
#pragma unroll
            for (int i = 0; i < NR; ++i) *(uint32_t *)(u_own + i * UROW) = un[i];
        }
        if (k > s_lo) {
            // y of step k-1
            float2 y2v[NR];
#pragma unroll
            for (int i = 0; i < NR; ++i) y2v[i] = *(const float2 *)(y_rd + i * YROW);
#pragma unroll
            for (int i = 0; i < NR; ++i) asm volatile("" ::"v"(yo[i]));       // (stored a step ago: see the backward)
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                float c0v, c1v;
                M::unpack2(cp[i], c0v, c1v);
                yo[i] = M::pack2(c0v * y2v[i].x, c1v * y2v[i].y);
            }
#pragma unroll
            for (int i = 0; i < NR; ++i) stw4_cached(wy, lane_y + y_b + (uint32_t)i * rb, yo[i]);
            y_b += step_b;
        }
#pragma unroll
        for (int i = 0; i < NR; ++i) cp[i] = cn[i];
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);           // what follows runs beside the matrix waves' products, not before them
        arrive(in);                                  // step k+1
        fetch(in, raw_b);                            // step k+3
        raw_b += step_b;
        __syncthreads();
    };
    int64_t k = k_first;
    for (; k + 1 <= s_hi; k += 2) {
        iter(k, in1);
        iter(k + 1, in0);
    }
    if (k <= s_hi) iter(k, in1);
}

} // namespace

// ---------------------------------------------------------------------------- launch
namespace {

MfmaPlan mixer_plan(const Dims &dm)
{
    MfmaPlan p = plan(dm, MixGeo<bf16_t>::XW, 16, MixGeo<bf16_t>::XW, 2);
    // the kernel adds the partials itself when a filter group lies within one channel block
    p.fuse_dh = MixGeo<bf16_t>::CB % dm.dg == 0 && p.ncb <= DH_UNITS;
    return p;
}

// a run with NK-1 steps and two rows before it, and one step plus NK-1 after it, stays inside one window
bool windows_fit(const Dims &dm, const MfmaPlan &p)
{
    return (int64_t)(p.steps_per_seg + 2 * 5 + 2) * STEP * 3 * dm.d * 2 <= WIN_MAX_BYTES;
}

template <typename T>
int bwd_t(const void *dy, const void *raw, const void *wfeat, int kf, const void *h, void *draw, void *dwf, void *dh,
          void *ws, const Dims &dm, hipStream_t st)
{
    typedef MixGeo<T> G;
    MfmaPlan p = mixer_plan(dm);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (p.fuse_dh && (p.slot = dh_slot_for_stream(st)) < 0) p.fuse_dh = p.slot = 0;   // no ticket set: second launches
    float *ws_dh = (float *)ws;
    float *ws_f = ws_dh + (size_t)p.nwg * G::XW * 128;
    int e = dm.planar
                ? launch_main((mixer_mr_bwd_kernel<T, true>), dim3((unsigned)p.nwg), dim3(G::NT), st, (const T *)dy,
                              (const T *)raw, (const T *)h, (const T *)wfeat, kf, (T *)draw, (T *)dh, (T *)dwf, ws_dh, ws_f,
                              dm, p)
                : launch_main((mixer_mr_bwd_kernel<T>), dim3((unsigned)p.nwg), dim3(G::NT), st, (const T *)dy,
                              (const T *)raw, (const T *)h, (const T *)wfeat, kf, (T *)draw, (T *)dh, (T *)dwf, ws_dh, ws_f,
                              dm, p);
    if (e || p.fuse_dh) return e;
    const int64_t n = (int64_t)dm.g * (dm.fw ? dm.lc : dm.hl);
    e = launch_plain(mfma_dh_reduce_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), st, (const float *)ws_dh,
                     (T *)dh, dm, p);
    if (e) return e;
    // partials are wsf[tap][(batch, run)][feature channel]
    return launch_colsum_reduce<T>(ws_f, (T *)dwf, dm.bs * p.nseg, 3 * dm.d, 1, (int)(3 * dm.d), kf, st);
}

} // namespace

namespace {
MfmaPlan mixer_fwd_plan(const Dims &dm)
{
    return plan(dm, MixFwdGeo<bf16_t>::XW, 4, MixFwdGeo<bf16_t>::XW, 2);
}
template <typename T>
int fwd_t(const void *raw, const void *wfeat, int kf, const void *h, void *y, const Dims &dm, hipStream_t st)
{
    const MfmaPlan p = mixer_fwd_plan(dm);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (dm.planar)
        return launch_main((mixer_mr_fwd_kernel<T, true>), dim3((unsigned)p.nwg), dim3(MixFwdGeo<T>::NT), st,
                           (const T *)raw, (const T *)h, (const T *)wfeat, kf, (T *)y, dm, p);
    return launch_main((mixer_mr_fwd_kernel<T>), dim3((unsigned)p.nwg), dim3(MixFwdGeo<T>::NT), st, (const T *)raw,
                       (const T *)h, (const T *)wfeat, kf, (T *)y, dm, p);
}
} // namespace

int mixer_mr_fused_fwd_launch(int dtype, const void *raw, const void *wfeat, int kf, const void *h, void *y,
                              const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return fwd_t<bf16_t>(raw, wfeat, kf, h, y, dm, st);
    if (dtype == GCG_F16) return fwd_t<f16_t>(raw, wfeat, kf, h, y, dm, st);
    return (int)hipErrorInvalidValue;
}

// 16-bit tensors with arithmetic in their own type, filters of up to 128 taps, a featurizer of at most 3
bool mixer_mr_fused_supported(int dtype, const Dims &dm, int kf)
{
    if (dtype != GCG_BF16 && dtype != GCG_F16) return false;
    if (!mfma_feat_supported(dtype, dm, kf) || 3 * dm.d > 0x7fffffffLL) return false;
    // both launches: the forward plans its runs by itself (shorter ones), the backward by its own
    return windows_fit(dm, mixer_plan(dm)) && windows_fit(dm, mixer_fwd_plan(dm));
}

size_t mixer_mr_fused_workspace(const Dims &dm, int kf)
{
    const MfmaPlan p = mixer_plan(dm);
    return ((size_t)p.nwg * MixGeo<bf16_t>::XW * 128 + (size_t)kf * dm.bs * p.nseg * 3 * dm.d) * sizeof(float);
}

int mixer_mr_fused_bwd_launch(int dtype, const void *dy, const void *raw, const void *wfeat, int kf, const void *h,
                              void *draw, void *dwf, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return bwd_t<bf16_t>(dy, raw, wfeat, kf, h, draw, dwf, dh, ws, dm, st);
    if (dtype == GCG_F16) return bwd_t<f16_t>(dy, raw, wfeat, kf, h, draw, dwf, dh, ws, dm, st);
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
