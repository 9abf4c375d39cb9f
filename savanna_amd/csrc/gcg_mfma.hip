// Banded Toeplitz GEMM on the matrix cores (bf16 / f16 I/O, fp32 accumulate, hl <= 128).
//
// Streaming form of the two-pass chunked convolution.  A workgroup of four waves owns 64
// adjacent channels of one batch row and walks a run of time steps of 32 rows.  Wave w owns
// the 16 channels [16w, 16w+16) -- one filter -- and computes, per step, the transposed
// output tile  Y2^T (16 channels x 32 times) = sum_i  U_{s-i}^T (16 x 32)  *  W_i (32 x 32)
// with v_mfma_f32_16x16x32, where U_{s-i} is the pre-gate product of step s-i and W_i the
// slice of the banded Toeplitz matrix of the filter at time offset 32*i.  The NK = 5 slices
// (10 operand tiles of 16 output times) live in registers for the whole walk, and the last
// NK operand tiles of U are carried in registers, so the "carry from the previous chunk" of
// the two-pass form never goes back to memory: q, k, v are read once and y written once.
//
// Memory side: the four waves load each 32 x 64 tile with full 128-byte rows, form
// u = bf16(x*B) in registers, park it row-major in LDS, and every wave fetches its matrix
// operand from there with the transposing LDS read (ds_read_b64_tr_b16), which hands a lane
// four consecutive time samples of one channel.  The fp32 result tile returns through LDS to
// the row layout, is gated with C in fp32 and stored with full 128-byte rows.
#include "gcg_common.h"

#include <cstdlib>

namespace gcg {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int STEP = 32;          // time rows per step (K of one MFMA)
// A workgroup of NW waves owns CB = 16*NW adjacent channels; its LDS rows are padded so that
// consecutive time rows start 8 (u, 2-byte elements) or 4 (y2, fp32) banks apart.
template <int NW> struct Geo {
    static constexpr int CB = 16 * NW;          // channels per workgroup
    static constexpr int LPR = CB / 8;          // lanes per row in the row layout (8 channels each)
    static constexpr int UROW = CB * 2 + 32;    // bytes per LDS row of u
    static constexpr int YROW = CB * 4 + 16;    // bytes per LDS row of y2
    static constexpr int NT = 64 * NW;          // threads
};
constexpr int HPAD = 32;          // filter table holds lags [-32, 160)
constexpr int HTAB = 192;

template <typename T> struct MT;
template <> struct MT<bf16_t> {
    typedef bf16x8 op_t;
    static __device__ __forceinline__ f32x4 mfma(op_t a, op_t b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void unpack2(uint32_t p, float &lo, float &hi)
    {
        lo = __uint_as_float(p << 16);
        hi = __uint_as_float(p & 0xffff0000u);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
};
template <> struct MT<f16_t> {
    typedef f16x8 op_t;
    static __device__ __forceinline__ f32x4 mfma(op_t a, op_t b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void unpack2(uint32_t p, float &lo, float &hi)
    {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v;
        __builtin_memcpy(&v, &p, 4);
        lo = (float)v[0];
        hi = (float)v[1];
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_f16x2(lo, hi); }
};

template <typename T> __device__ __forceinline__ void unpack8(const uint4 &r, float (&f)[8])
{
    MT<T>::unpack2(r.x, f[0], f[1]);
    MT<T>::unpack2(r.y, f[2], f[3]);
    MT<T>::unpack2(r.z, f[4], f[5]);
    MT<T>::unpack2(r.w, f[6], f[7]);
}
template <typename T> __device__ __forceinline__ uint4 pack8(const float (&f)[8])
{
    return make_uint4(MT<T>::pack2(f[0], f[1]), MT<T>::pack2(f[2], f[3]), MT<T>::pack2(f[4], f[5]),
                      MT<T>::pack2(f[6], f[7]));
}

// Transposing LDS read: within each block of 16 lanes, lane i receives element (i % 4) of
// the 8-byte rows addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4 of that block.
__device__ __forceinline__ s16x4 lds_read_tr(const unsigned char *p)
{
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
}

// Streaming accesses: every tensor element is touched once, so loads and stores carry the
// nontemporal hint (GCG_MFMA_NT=0 at build time turns it off for comparison).
#ifndef GCG_XCD_SWIZZLE
#define GCG_XCD_SWIZZLE 1
#endif
#ifndef GCG_MFMA_NT
#define GCG_MFMA_NT 3
#endif
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <typename T> __device__ __forceinline__ uint4 ldg16(const T *p)
{
#if GCG_MFMA_NT & 1
    const u32x4 v = __builtin_nontemporal_load((const u32x4 *)p);
    return make_uint4(v[0], v[1], v[2], v[3]);
#else
    return *(const uint4 *)p;
#endif
}
template <typename T> __device__ __forceinline__ void stg16(T *p, const uint4 &v)
{
#if GCG_MFMA_NT & 2
    const u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (u32x4 *)p);
#else
    *(uint4 *)p = v;
#endif
}

// Workgroups are dealt to the 8 XCDs round-robin by index.  Re-labelling them so that each XCD
// receives a contiguous run of (batch, segment, channel-block) triples makes the workgroups of
// one XCD cover whole tensor rows between them, which its L2 and the memory channels prefer.
__device__ __forceinline__ int64_t xcd_contiguous_id(int64_t id, int64_t n)
{
#if GCG_XCD_SWIZZLE
    if ((n & 7) == 0) return (id & 7) * (n >> 3) + (id >> 3);
#endif
    return id;
}

struct MfmaPlan { int ncb, nseg, steps_per_seg, nw; int64_t nsteps, nwg; };

// Operand tile of the banded Toeplitz matrix at row offset doff = (out time) - (in time) of
// the tile origins: element e of lane (j, q) is the tap for lag doff + j - 8q - e.
template <typename T>
__device__ __forceinline__ typename MT<T>::op_t toeplitz_operand(const uint16_t *htab, int doff, int j, int q)
{
    uint16_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = htab[doff + j - 8 * q - e + HPAD];
    typename MT<T>::op_t r;
    __builtin_memcpy(&r, v, 16);
    return r;
}

// ---------------------------------------------------------------------------- forward
template <typename T, int NK, int NW>
__global__ __launch_bounds__(64 * NW) void mfma_fwd_kernel(const T *__restrict__ x, const T *__restrict__ B,
                                                       const T *__restrict__ C, const T *__restrict__ h,
                                                       T *__restrict__ y, T *__restrict__ y2o,
                                                       T *__restrict__ bxo, Dims dm, MfmaPlan pl)
{
    typedef typename MT<T>::op_t op_t;
    typedef Geo<NW> G;
    constexpr int CB = G::CB, UROW = G::UROW, YROW = G::YROW;
    __shared__ __attribute__((aligned(16))) unsigned char u_rm[STEP * UROW];
    __shared__ __attribute__((aligned(16))) unsigned char y_st[STEP * YROW];
    __shared__ uint16_t htab[NW][HTAB];

    int64_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int cb = (int)(wg % pl.ncb); wg /= pl.ncb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int r = tid / G::LPR, a = tid % G::LPR;   // row layout: row r of the step, channels 8a..8a+7
    const int j = l & 15, q = l >> 4;    // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;
    const int hl = dm.hl;

    // filter table of this wave's group: htab[lag + 32] = h[hl-1-lag] for 0 <= lag < hl, else 0
    {
        const int64_t cw = c0 + 16 * w;
        const int64_t grp = (cw < d) ? cw / dm.dg : 0;
        const uint16_t *hg = (const uint16_t *)h + grp * hl;
        for (int i = l; i < HTAB; i += 64) {
            const int lag = i - HPAD;
            htab[w][i] = (lag >= 0 && lag < hl) ? hg[hl - 1 - lag] : (uint16_t)0;
        }
    }
    __syncthreads();
    op_t W0[NK], W1[NK];   // output rows 0..15 / 16..31 of the step against input step s-i
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = toeplitz_operand<T>(htab[w], 32 * i, j, q);
        W1[i] = toeplitz_operand<T>(htab[w], 32 * i + 16, j, q);
    }

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;
    const int64_t s_first = (s_lo - (NK - 1) > 0) ? s_lo - (NK - 1) : 0;

    const bool cvalid = c0 + 8 * a < d;
    const int64_t col = b * L * d + c0 + 8 * a;            // element offset of this lane's columns
    const int row_in_step = r;

    op_t A[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        uint4 z = make_uint4(0u, 0u, 0u, 0u);
        __builtin_memcpy(&A[i], &z, 16);
    }

    unsigned char *u_wr = u_rm + row_in_step * UROW + 16 * a;
    const unsigned char *u_rd = u_rm + (8 * q + (j >> 2)) * UROW + (16 * w + 4 * (j & 3)) * 2;
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    const unsigned char *y_rd = y_st + row_in_step * YROW + 32 * a;

    uint4 xr, Br, Cr;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    auto fetch = [&](int64_t s, uint4 &xo, uint4 &Bo, uint4 &Co) {
        const int64_t t = s * STEP + row_in_step;
        xo = zero4; Bo = zero4; Co = zero4;
        if (cvalid && t < L) {
            const int64_t o = col + t * d;
            xo = ldg16(x + o);
            Bo = ldg16(B + o);
            if (s >= s_lo) Co = ldg16(C + o);
        }
    };
    fetch(s_first, xr, Br, Cr);

    int64_t s = s_first;
    while (s < s_hi) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < s_hi) {
                const bool main_step = s >= s_lo;
                uint4 xn = zero4, Bn = zero4, Cn = zero4;
                if (s + 1 < s_hi) fetch(s + 1, xn, Bn, Cn);

                float xf[8], Bf[8], uf[8];
                unpack8<T>(xr, xf);
                unpack8<T>(Br, Bf);
#pragma unroll
                for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
                const uint4 up = pack8<T>(uf);
                *(uint4 *)u_wr = up;
                const int64_t t = s * STEP + row_in_step;
                const bool store_ok = main_step && cvalid && t < L;
                if (bxo && store_ok) stg16(bxo + col + t * d, up);
                __syncthreads();
                {
                    const s16x4 lo = lds_read_tr(u_rd);
                    const s16x4 hi = lds_read_tr(u_rd + 4 * UROW);
                    short v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    __builtin_memcpy(&A[ph], v, 16);
                }
                if (main_step) {
                    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < NK; ++i) {
                        acc0 = MT<T>::mfma(A[(ph - i + NK) % NK], W0[i], acc0);
                        acc1 = MT<T>::mfma(A[(ph - i + NK) % NK], W1[i], acc1);
                    }
                    *(f32x4 *)y_wr = acc0;
                    *(f32x4 *)(y_wr + 16 * YROW) = acc1;
                }
                __syncthreads();
                if (store_ok) {
                    const f32x4 p0 = *(const f32x4 *)y_rd;
                    const f32x4 p1 = *(const f32x4 *)(y_rd + 16);
                    float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                    float Cf[8], yf[8];
                    unpack8<T>(Cr, Cf);
#pragma unroll
                    for (int e = 0; e < 8; ++e) yf[e] = Cf[e] * y2f[e];
                    stg16(y + col + t * d, pack8<T>(yf));
                    if (y2o) stg16(y2o + col + t * d, pack8<T>(y2f));
                }
                xr = xn; Br = Bn; Cr = Cn;
                ++s;
            }
        }
    }
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
// (a 16x16x32 MFMA contracts 16 channels x 2 row-halves), lag = 16*delta + i - j.  At the
// end the diagonals of the P tiles are summed in a fixed order into per-wave partials in
// the workspace, and a second kernel adds the partials in a fixed order.
template <typename T, int NK, int NW>
__global__ __launch_bounds__(64 * NW) void mfma_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                       const T *__restrict__ B, const T *__restrict__ C,
                                                       const T *__restrict__ h, T *__restrict__ dx,
                                                       T *__restrict__ dB, T *__restrict__ dC,
                                                       float *__restrict__ ws, Dims dm, MfmaPlan pl)
{
    typedef typename MT<T>::op_t op_t;
    typedef Geo<NW> G;
    constexpr int CB = G::CB, UROW = G::UROW, YROW = G::YROW;
    constexpr int ND = 2 * NK - 1;
    constexpr int RING_ROWS = STEP * NK;
    constexpr int OFF_U = 0;                                // u of the current step, row-major
    constexpr int OFF_G = OFF_U + STEP * UROW;              // g2 ring, NK steps, row-major
    constexpr int OFF_Y = OFF_G + RING_ROWS * UROW;         // y2 tile, fp32, row-major
    constexpr int OFF_D = OFF_Y + STEP * YROW;              // du tile, fp32, row-major
    constexpr int OFF_H = OFF_D + STEP * YROW;              // filter tables
    constexpr int LDS_MAIN = OFF_H + NW * HTAB * 2;
    constexpr int LDS_TAIL = NW * ND * 256 * 4;             // P tiles at the end
    constexpr int LDS_BYTES = LDS_MAIN > LDS_TAIL ? LDS_MAIN : LDS_TAIL;
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_BYTES];
    unsigned char *u_rm = smem + OFF_U, *g_rm = smem + OFF_G, *y_st = smem + OFF_Y, *d_st = smem + OFF_D;
    uint16_t *htab = (uint16_t *)(smem + OFF_H);

    int64_t wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int cb = (int)(wg % pl.ncb); wg /= pl.ncb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int r = tid / G::LPR, a = tid % G::LPR;   // row layout: row r of the step, channels 8a..8a+7
    const int j = l & 15, q = l >> 4;               // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;
    const int hl = dm.hl;
    const bool wave_valid = c0 + 16 * w < d;

    {
        const int64_t grp = wave_valid ? (c0 + 16 * w) / dm.dg : 0;
        const uint16_t *hg = (const uint16_t *)h + grp * hl;
        for (int i = l; i < HTAB; i += 64) {
            const int lag = i - HPAD;
            htab[w * HTAB + i] = (lag >= 0 && lag < hl) ? hg[hl - 1 - lag] : (uint16_t)0;
        }
    }
    __syncthreads();
    op_t W0[NK], W1[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = toeplitz_operand<T>(htab + w * HTAB, 32 * i, j, q);
        W1[i] = toeplitz_operand<T>(htab + w * HTAB, 32 * i + 16, j, q);
    }

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;
    const int64_t s_first = s_lo - (NK - 1);                // may be negative: those rows read as zero

    const bool cvalid = c0 + 8 * a < d;
    const int64_t col = b * L * d + c0 + 8 * a;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    op_t Au[NK], Ag[NK];      // Au[k]: u operand of a step; Ag[k]: time-reversed g2 operand of a step
    uint4 dyq[NK];            // dy rows (row layout) waiting for their y2
    f32x4 P[ND];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        __builtin_memcpy(&Au[i], &zero4, 16);
        __builtin_memcpy(&Ag[i], &zero4, 16);
        dyq[i] = zero4;
    }
#pragma unroll
    for (int i = 0; i < ND; ++i) P[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // LDS addresses of this lane
    unsigned char *u_wr = u_rm + r * UROW + 16 * a;
    const int g_wr_off = r * UROW + 16 * a;                                   // + slot * STEP * UROW
    const int tr_col = (16 * w + 4 * (j & 3)) * 2;
    const unsigned char *u_tr = u_rm + (8 * q + (j >> 2)) * UROW + tr_col;
    const int g_tr_off = (31 - 8 * q - (j >> 2)) * UROW + tr_col;             // reversed time order
    const int nat_col = (16 * w + 8 * (q & 1)) * 2;                           // natural operand: 8 channels
    const int nat_row = 16 * (q >> 1) + j;                                    // row half by lane quad
    const unsigned char *u_nat = u_rm + nat_row * UROW + nat_col;
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    unsigned char *d_wr = d_st + (15 - j) * YROW + (16 * w + 4 * q) * 4;      // columns come out reversed
    const unsigned char *y_rd = y_st + r * YROW + 32 * a;
    const unsigned char *d_rd = d_st + r * YROW + 32 * a;

    auto fetch = [&](int64_t sg, uint4 &xo, uint4 &Bo, uint4 &dyo, uint4 &Co) {
        xo = zero4; Bo = zero4; dyo = zero4; Co = zero4;
        if (cvalid) {
            const int64_t t = sg * STEP + r;
            if (t >= 0 && t < L) {
                xo = ldg16(x + col + t * d);
                Bo = ldg16(B + col + t * d);
            }
            const int64_t t2 = t + (NK - 1) * STEP;
            if (t2 >= 0 && t2 < L) {
                dyo = ldg16(dy + col + t2 * d);
                Co = ldg16(C + col + t2 * d);
            }
        }
    };
    uint4 xr, Br, dyr, Cr;
    fetch(s_first, xr, Br, dyr, Cr);

    int64_t s = s_first;
    while (s < s_hi) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < s_hi) {
                const bool main_step = s >= s_lo;
                const int slot_new = (ph + NK - 1) % NK;     // ring slot of step s+NK-1
                uint4 xn = zero4, Bn = zero4, dyn = zero4, Cn = zero4;
                if (s + 1 < s_hi) fetch(s + 1, xn, Bn, dyn, Cn);

                float xf[8], Bf[8], tf[8], cf[8], pf[8];
                unpack8<T>(xr, xf);
                unpack8<T>(Br, Bf);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = xf[e] * Bf[e];
                *(uint4 *)u_wr = pack8<T>(pf);
                unpack8<T>(dyr, tf);
                unpack8<T>(Cr, cf);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = tf[e] * cf[e];
                *(uint4 *)(g_rm + slot_new * STEP * UROW + g_wr_off) = pack8<T>(pf);
                dyq[slot_new] = dyr;
                __syncthreads();
                {
                    const s16x4 lo = lds_read_tr(u_tr);
                    const s16x4 hi = lds_read_tr(u_tr + 4 * UROW);
                    short v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    __builtin_memcpy(&Au[ph], v, 16);
                    const unsigned char *gp = g_rm + slot_new * STEP * UROW + g_tr_off;
                    const s16x4 glo = lds_read_tr(gp);
                    const s16x4 ghi = lds_read_tr(gp - 4 * UROW);
                    short gv[8] = {glo[0], glo[1], glo[2], glo[3], ghi[0], ghi[1], ghi[2], ghi[3]};
                    __builtin_memcpy(&Ag[slot_new], gv, 16);
                }
                if (main_step) {
                    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
                    f32x4 dac0 = {0.f, 0.f, 0.f, 0.f}, dac1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < NK; ++i) {
                        acc0 = MT<T>::mfma(Au[(ph - i + NK) % NK], W0[i], acc0);
                        acc1 = MT<T>::mfma(Au[(ph - i + NK) % NK], W1[i], acc1);
                        // g2 of step s+i sits in slot (ph+i) % NK
                        dac0 = MT<T>::mfma(Ag[(ph + i) % NK], W1[i], dac0);   // output rows 0..15
                        dac1 = MT<T>::mfma(Ag[(ph + i) % NK], W0[i], dac1);   // output rows 16..31
                    }
                    *(f32x4 *)y_wr = acc0;
                    *(f32x4 *)(y_wr + 16 * YROW) = acc1;
                    *(f32x4 *)d_wr = dac0;
                    *(f32x4 *)(d_wr + 16 * YROW) = dac1;
                    // filter-gradient tiles: natural-layout operands, 8 channels of two row halves
                    op_t un;
                    {
                        const uint4 t4 = *(const uint4 *)u_nat;
                        __builtin_memcpy(&un, &t4, 16);
                    }
#pragma unroll
                    for (int dl = 0; dl < ND; ++dl) {
                        int row = STEP * ph + 16 * dl + nat_row;           // ring row of this lane's g2 row
                        row = (row >= RING_ROWS) ? row - RING_ROWS : row;
                        const uint4 t4 = *(const uint4 *)(g_rm + row * UROW + nat_col);
                        op_t gn;
                        __builtin_memcpy(&gn, &t4, 16);
                        P[dl] = MT<T>::mfma(gn, un, P[dl]);
                    }
                }
                __syncthreads();
                const int64_t t = s * STEP + r;
                if (main_step && cvalid && t < L) {
                    const int64_t o = col + t * d;
                    {
                        const f32x4 p0 = *(const f32x4 *)y_rd;
                        const f32x4 p1 = *(const f32x4 *)(y_rd + 16);
                        const float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                        float dyf[8], of[8];
                        unpack8<T>(dyq[ph], dyf);
#pragma unroll
                        for (int e = 0; e < 8; ++e) of[e] = dyf[e] * y2f[e];
                        stg16(dC + o, pack8<T>(of));
                    }
                    {
                        const f32x4 p0 = *(const f32x4 *)d_rd;
                        const f32x4 p1 = *(const f32x4 *)(d_rd + 16);
                        const float duf[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                        float of[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) of[e] = duf[e] * Bf[e];
                        stg16(dx + o, pack8<T>(of));
#pragma unroll
                        for (int e = 0; e < 8; ++e) of[e] = duf[e] * xf[e];
                        stg16(dB + o, pack8<T>(of));
                    }
                }
                xr = xn; Br = Bn; dyr = dyn; Cr = Cn;
                ++s;
            }
        }
    }

    // diagonal sums of the P tiles -> per-wave filter-gradient partials
    __syncthreads();
    float *pt = (float *)smem + w * ND * 256;
#pragma unroll
    for (int dl = 0; dl < ND; ++dl)
#pragma unroll
        for (int v = 0; v < 4; ++v) pt[dl * 256 + (4 * q + v) * 16 + j] = P[dl][v];
    __syncthreads();
    if (wave_valid) {
        float *out = ws + ((size_t)xcd_contiguous_id(blockIdx.x, gridDim.x) * NW + w) * 128;
        for (int lag = l; lag < 128; lag += 64) {
            const int d0 = lag >> 4, rr = lag & 15;
            float sum = 0.f;
            if (d0 < ND)
                for (int jj = 0; jj + rr < 16; ++jj) sum += pt[d0 * 256 + (jj + rr) * 16 + jj];
            if (d0 + 1 < ND)
                for (int ii = 0; ii < rr; ++ii) sum += pt[(d0 + 1) * 256 + ii * 16 + ii + 16 - rr];
            out[lag] = sum;
        }
    }
}

// dh[grp][k] = sum of the per-wave partials of the 16-channel blocks of the group
template <typename T>
__global__ __launch_bounds__(256) void mfma_dh_reduce_kernel(const float *__restrict__ ws, T *__restrict__ dh,
                                                             Dims dm, MfmaPlan pl)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)dm.g * dm.hl) return;
    const int64_t grp = i / dm.hl;
    const int lag = dm.hl - 1 - (int)(i % dm.hl);
    const int bpg = dm.dg / 16;                          // 16-channel blocks per group
    const int64_t slots = (int64_t)pl.ncb * pl.nw;       // block slots per (batch, segment)
    float sum = 0.f;
    for (int64_t p = 0; p < dm.bs * pl.nseg; ++p)
        for (int k = 0; k < bpg; ++k)
            sum += ws[(p * slots + grp * bpg + k) * 128 + lag];
    Elem<T>::store(dh + i, sum);
}

int cu_count()
{
    static int n = 0;
    if (n == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            n = v;
        else
            n = 256;
    }
    return n;
}

int env_int(const char *name, int dflt)
{
    const char *v = getenv(name);
    return (v && atoi(v) > 0) ? atoi(v) : dflt;
}

// Waves per workgroup: wider workgroups read wider rows (16*NW channels, 32*NW bytes), which
// the memory system rewards; narrow tensors fall back to what their width fills.
int choose_nw(const Dims &dm)
{
    static const int forced = env_int("GCG_MFMA_NW", 0);   // tuning override: 4, 8 or 16
    if (forced == 4 || forced == 8 || forced == 16) return forced;
    if (dm.d >= 256) return 16;
    if (dm.d >= 128) return 8;
    return 4;
}

MfmaPlan plan(const Dims &dm, int nw, int min_steps, int waves_per_cu)
{
    MfmaPlan p;
    const int cb = 16 * nw;
    p.nw = nw;
    p.ncb = (int)((dm.d + cb - 1) / cb);
    p.nsteps = (dm.L + STEP - 1) / STEP;
    const int wg_per_cu = waves_per_cu / nw > 0 ? waves_per_cu / nw : 1;
    int64_t cols = dm.bs * p.ncb;
    int64_t want = ((int64_t)cu_count() * wg_per_cu + cols - 1) / cols;   // segments to fill the chip
    int64_t max_seg = p.nsteps / min_steps;
    if (max_seg < 1) max_seg = 1;
    if (want > max_seg) want = max_seg;
    if (want < 1) want = 1;
    static const int forced = env_int("GCG_MFMA_STEPS_PER_SEG", 0);        // tuning override
    int64_t sps = (p.nsteps + want - 1) / want;
    if (forced > 0) sps = forced;
    p.steps_per_seg = (int)sps;
    p.nseg = (int)((p.nsteps + sps - 1) / sps);
    p.nwg = dm.bs * p.nseg * p.ncb;
    return p;
}

// input steps an output step reaches back over: lags up to hl-1 from rows 0..31 of the step
int nk_for(int hl) { const int n = (hl + 30) / 32 + 1; return n > 5 ? 5 : n; }

template <typename T, int NK, int NW>
int fwd_launch(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
               const Dims &dm, hipStream_t st)
{
    const MfmaPlan p = plan(dm, NW, 16, 16);   // ~124 registers: 4 waves per SIMD
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((mfma_fwd_kernel<T, NK, NW>), dim3((unsigned)p.nwg), dim3(64 * NW), 0, st, (const T *)x,
                       (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    return (int)hipGetLastError();
}

template <typename T, int NK>
int fwd_nk(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
           const Dims &dm, hipStream_t st)
{
    switch (choose_nw(dm)) {
    case 16: return fwd_launch<T, NK, 16>(x, B, C, h, y, y2, bx, dm, st);
    case 8:  return fwd_launch<T, NK, 8>(x, B, C, h, y, y2, bx, dm, st);
    default: return fwd_launch<T, NK, 4>(x, B, C, h, y, y2, bx, dm, st);
    }
}

template <typename T>
int fwd_t(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
          const Dims &dm, hipStream_t st)
{
    switch (nk_for(dm.hl)) {
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
    return (dtype == GCG_BF16 || dtype == GCG_F16) && dm.hl <= 128 && dm.dg % 16 == 0;
}

int mfma_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h, void *y,
                    void *y2, void *bx, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return fwd_t<bf16_t>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_F16) return fwd_t<f16_t>(x, B, C, h, y, y2, bx, dm, st);
    return (int)hipErrorInvalidValue;
}

bool mfma_bwd_available() { return true; }

namespace {

// The backward holds about twice the forward's register state per wave, so it runs two
// waves per SIMD and at most 8 waves (128 channels, 256-byte rows) per workgroup.
int choose_nw_bwd(const Dims &dm)
{
    static const int forced = env_int("GCG_MFMA_BWD_NW", 0);   // tuning override: 4 or 8
    if (forced == 4 || forced == 8) return forced;
    return dm.d >= 128 ? 8 : 4;
}

MfmaPlan plan_bwd(const Dims &dm) { return plan(dm, choose_nw_bwd(dm), 16, 8); }

template <typename T, int NK, int NW>
int bwd_launch(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
               void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    const MfmaPlan p = plan_bwd(dm);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((mfma_bwd_kernel<T, NK, NW>), dim3((unsigned)p.nwg), dim3(64 * NW), 0, st, (const T *)dy,
                       (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)dx, (T *)dB, (T *)dC,
                       (float *)ws, dm, p);
    int e = (int)hipGetLastError();
    if (e) return e;
    const int64_t n = (int64_t)dm.g * dm.hl;
    hipLaunchKernelGGL(mfma_dh_reduce_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const float *)ws, (T *)dh, dm, p);
    return (int)hipGetLastError();
}

template <typename T, int NK>
int bwd_nk(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
           void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    if (choose_nw_bwd(dm) == 8) return bwd_launch<T, NK, 8>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    return bwd_launch<T, NK, 4>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
}

template <typename T>
int bwd_t(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
          void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    switch (nk_for(dm.hl)) {
    case 1: return bwd_nk<T, 1>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case 2: return bwd_nk<T, 2>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case 3: return bwd_nk<T, 3>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    case 4: return bwd_nk<T, 4>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    default: return bwd_nk<T, 5>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    }
}

} // namespace

size_t mfma_bwd_workspace(const Dims &dm)
{
    const MfmaPlan p = plan_bwd(dm);
    return (size_t)p.nwg * p.nw * 128 * sizeof(float);
}

int mfma_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C, const void *h,
                    void *dx, void *dB, void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return bwd_t<bf16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dtype == GCG_F16) return bwd_t<f16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
