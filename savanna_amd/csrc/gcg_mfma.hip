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
// one channel per lane) comes from the transposing LDS read ds_read_b64_tr_b16.  fp32: the
// same 32-deep product is eight v_mfma_f32_16x16x4_f32 (exact fp32 multiply-add, so the fp32
// path keeps fp32 accuracy); a lane's eight operand values are time samples q, q+4, ... of one
// channel, read straight from the row-major tile.
#include "gcg_common.h"

#include <cstdlib>

namespace gcg {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int STEP = 32;          // time rows per step (contraction depth of one product)
constexpr int HPAD = 32;          // filter table holds lags [-32, 160)
constexpr int HTAB = 192;

// Transposing LDS read: within each block of 16 lanes, lane i receives element (i % 4) of
// the 8-byte rows addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4 of that block.
__device__ __forceinline__ s16x4 lds_read_tr(const unsigned char *p)
{
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
}

// Per element type: the matrix operand, how it is fetched from a row-major LDS tile of
// `urow` bytes per time row, and the 32-deep product.  Operand element e of the lane in
// quad q stands for contraction index kmap(q, e); both factors of a product use the same map.
template <typename T> struct MT;

template <typename OP> struct MT16 {
    static constexpr int ES = 2;                 // bytes per element
    static constexpr int RW = 1;                 // 16-byte words per 8-channel row vector
    static constexpr int UPAD = 32;              // row padding: consecutive rows start 8 banks apart
    typedef OP op_t;
    typedef uint16_t hraw_t;
    static __device__ __forceinline__ int kmap(int q, int e) { return 8 * q + e; }
    static __device__ __forceinline__ op_t zero_op()
    {
        op_t r;
        const uint4 z = make_uint4(0u, 0u, 0u, 0u);
        __builtin_memcpy(&r, &z, 16);
        return r;
    }
    // time samples kmap(q, .) of channel 16w+j from rows row0 .. row0+31 (reversed: 31-k)
    static __device__ __forceinline__ op_t load_operand(const unsigned char *tile, int urow, int w, int j, int q,
                                                        bool reversed)
    {
        const int col = (16 * w + 4 * (j & 3)) * 2;
        const int r0 = reversed ? 31 - 8 * q - (j >> 2) : 8 * q + (j >> 2);
        const int r1 = reversed ? r0 - 4 : r0 + 4;
        const s16x4 lo = lds_read_tr(tile + r0 * urow + col);
        const s16x4 hi = lds_read_tr(tile + r1 * urow + col);
        const short v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        op_t r;
        __builtin_memcpy(&r, v, 16);
        return r;
    }
    // natural-layout operand of the filter-gradient product: 8 channels of one of two rows;
    // lane quad q takes row half q>>1 and channels 8*(q&1)..+7 of the wave's 16
    static __device__ __forceinline__ op_t load_natural(const unsigned char *row_half0,
                                                        const unsigned char *row_half1, int w, int q)
    {
        const unsigned char *p = ((q >> 1) ? row_half1 : row_half0) + (16 * w + 8 * (q & 1)) * 2;
        const uint4 t4 = *(const uint4 *)p;
        op_t r;
        __builtin_memcpy(&r, &t4, 16);
        return r;
    }
    static __device__ __forceinline__ op_t toeplitz(const hraw_t *htab, int doff, int j, int q)
    {
        uint16_t v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = htab[doff + j - kmap(q, e) + HPAD];
        op_t r;
        __builtin_memcpy(&r, v, 16);
        return r;
    }
};

template <> struct MT<bf16_t> : MT16<bf16x8> {
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
template <> struct MT<f16_t> : MT16<f16x8> {
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

struct F32x8 { float v[8]; };
template <> struct MT<float> {
    static constexpr int ES = 4;
    static constexpr int RW = 2;
    static constexpr int UPAD = 64;              // consecutive rows start 16 banks apart
    typedef F32x8 op_t;
    typedef float hraw_t;
    // instruction e of the eight contracts time samples 4e .. 4e+3, one per lane quad
    static __device__ __forceinline__ int kmap(int q, int e) { return 4 * e + q; }
    static __device__ __forceinline__ op_t zero_op()
    {
        op_t r;
#pragma unroll
        for (int e = 0; e < 8; ++e) r.v[e] = 0.f;
        return r;
    }
    static __device__ __forceinline__ op_t load_operand(const unsigned char *tile, int urow, int w, int j, int q,
                                                        bool reversed)
    {
        op_t r;
        const int col = (16 * w + j) * 4;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int k = kmap(q, e);
            r.v[e] = *(const float *)(tile + (reversed ? 31 - k : k) * urow + col);
        }
        return r;
    }
    // element e: row half e>>2, channel 4q + (e&3) of the wave's 16
    static __device__ __forceinline__ op_t load_natural(const unsigned char *row_half0,
                                                        const unsigned char *row_half1, int w, int q)
    {
        const int col = (16 * w + 4 * q) * 4;
        const f32x4 a = *(const f32x4 *)(row_half0 + col), b = *(const f32x4 *)(row_half1 + col);
        op_t r;
        r.v[0] = a[0]; r.v[1] = a[1]; r.v[2] = a[2]; r.v[3] = a[3];
        r.v[4] = b[0]; r.v[5] = b[1]; r.v[6] = b[2]; r.v[7] = b[3];
        return r;
    }
    static __device__ __forceinline__ op_t toeplitz(const hraw_t *htab, int doff, int j, int q)
    {
        op_t r;
#pragma unroll
        for (int e = 0; e < 8; ++e) r.v[e] = htab[doff + j - kmap(q, e) + HPAD];
        return r;
    }
    static __device__ __forceinline__ f32x4 mfma(const op_t &a, const op_t &b, f32x4 c)
    {
#pragma unroll
        for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[e], b.v[e], c, 0, 0, 0);
        return c;
    }
};

// A workgroup of NW waves owns CB = 16*NW adjacent channels; LDS rows are padded (see UPAD;
// the fp32 result tile: consecutive rows start 4 banks apart).
template <typename T, int NW> struct Geo {
    static constexpr int CB = 16 * NW;                          // channels per workgroup
    static constexpr int LPR = CB / 8;                          // lanes per row in the row layout (8 channels each)
    static constexpr int UROW = CB * MT<T>::ES + MT<T>::UPAD;   // bytes per LDS row of u / g2
    static constexpr int YROW = CB * 4 + 16;                    // bytes per LDS row of y2 / du
    static constexpr int NT = 64 * NW;                          // threads
};

// A lane's 8 channels of one row: RW 16-byte words.
template <typename T> struct Row { uint4 w[MT<T>::RW]; };

template <typename T> __device__ __forceinline__ void unpack8(const Row<T> &r, float (&f)[8])
{
    if constexpr (MT<T>::ES == 4) {
        f[0] = __uint_as_float(r.w[0].x); f[1] = __uint_as_float(r.w[0].y);
        f[2] = __uint_as_float(r.w[0].z); f[3] = __uint_as_float(r.w[0].w);
        f[4] = __uint_as_float(r.w[1].x); f[5] = __uint_as_float(r.w[1].y);
        f[6] = __uint_as_float(r.w[1].z); f[7] = __uint_as_float(r.w[1].w);
    } else {
        MT<T>::unpack2(r.w[0].x, f[0], f[1]);
        MT<T>::unpack2(r.w[0].y, f[2], f[3]);
        MT<T>::unpack2(r.w[0].z, f[4], f[5]);
        MT<T>::unpack2(r.w[0].w, f[6], f[7]);
    }
}
template <typename T> __device__ __forceinline__ Row<T> pack8(const float (&f)[8])
{
    Row<T> r;
    if constexpr (MT<T>::ES == 4) {
        r.w[0] = make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
        r.w[1] = make_uint4(__float_as_uint(f[4]), __float_as_uint(f[5]), __float_as_uint(f[6]), __float_as_uint(f[7]));
    } else {
        r.w[0] = make_uint4(MT<T>::pack2(f[0], f[1]), MT<T>::pack2(f[2], f[3]), MT<T>::pack2(f[4], f[5]),
                            MT<T>::pack2(f[6], f[7]));
    }
    return r;
}
template <typename T> __device__ __forceinline__ Row<T> zero_row()
{
    Row<T> r;
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) r.w[i] = make_uint4(0u, 0u, 0u, 0u);
    return r;
}
template <typename T> __device__ __forceinline__ void lds_store_row(unsigned char *p, const Row<T> &r)
{
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) *(uint4 *)(p + 16 * i) = r.w[i];
}

template <typename T> __device__ __forceinline__ Row<T> lds_load_row(const unsigned char *p)
{
    Row<T> r;
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) r.w[i] = *(const uint4 *)(p + 16 * i);
    return r;
}

// Interleaved operands (element stride 3): a lane's 8 channels of one row are 24 consecutive
// elements, (C, B, x) per channel, i.e. three row vectors.  split_rows / join_rows convert
// between that order and per-tensor channel vectors; every index is a compile-time constant.
template <typename T>
__device__ __forceinline__ void split_rows(const Row<T> (&p)[3], float (&xf)[8], float (&Bf)[8], float (&Cf)[8])
{
    float f[3][8];
#pragma unroll
    for (int i = 0; i < 3; ++i) unpack8<T>(p[i], f[i]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        Cf[e] = f[(3 * e) / 8][(3 * e) % 8];
        Bf[e] = f[(3 * e + 1) / 8][(3 * e + 1) % 8];
        xf[e] = f[(3 * e + 2) / 8][(3 * e + 2) % 8];
    }
}
template <typename T>
__device__ __forceinline__ void join_rows(const float (&xf)[8], const float (&Bf)[8], const float (&Cf)[8],
                                          Row<T> (&p)[3])
{
    float f[3][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        f[(3 * e) / 8][(3 * e) % 8] = Cf[e];
        f[(3 * e + 1) / 8][(3 * e + 1) % 8] = Bf[e];
        f[(3 * e + 2) / 8][(3 * e + 2) % 8] = xf[e];
    }
#pragma unroll
    for (int i = 0; i < 3; ++i) p[i] = pack8<T>(f[i]);
}
// One input row of a lane as three row vectors: (x, B, C) of separate tensors, or the three
// thirds of the interleaved row.
template <typename T, bool PK>
__device__ __forceinline__ void in_floats(const Row<T> (&p)[3], float (&xf)[8], float (&Bf)[8], float (&Cf)[8])
{
    if constexpr (PK) {
        split_rows<T>(p, xf, Bf, Cf);
    } else {
        unpack8<T>(p[0], xf);
        unpack8<T>(p[1], Bf);
        unpack8<T>(p[2], Cf);
    }
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
template <typename T> __device__ __forceinline__ uint4 ldg16(const T *p);
template <typename T> __device__ __forceinline__ void stg16(T *p, const uint4 &v);
template <typename T> __device__ __forceinline__ Row<T> ldg_row(const T *p)
{
    Row<T> r;
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) r.w[i] = ldg16((const unsigned char *)p + 16 * i);
    return r;
}
template <typename T> __device__ __forceinline__ void stg_row(T *p, const Row<T> &r)
{
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) stg16((unsigned char *)p + 16 * i, r.w[i]);
}
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

// Operand tile of the banded Toeplitz matrix at row offset doff = (out time) - (in time) of the
// tile origins: element e of lane (j, q) is the tap for lag doff + j - kmap(q, e)  (MT<T>::toeplitz).

// ---------------------------------------------------------------------------- forward
// PK: x, B, C are interleaved in one tensor that starts at C (element stride 3).
template <typename T, int NK, int NW, bool PK>
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
    __shared__ __attribute__((aligned(16))) unsigned char u_rm[STEP * UROW];
    __shared__ __attribute__((aligned(16))) unsigned char y_st[STEP * YROW];
    __shared__ hraw_t htab[NW][HTAB];

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

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;

    const bool cvalid = c0 + 8 * a < d;
    const int64_t col = b * L * d + c0 + 8 * a;            // element offset of this lane's columns

    op_t A[NK];            // A[(ph - i + NK) % NK]: operand of step s-i while step s runs in phase ph
#pragma unroll
    for (int i = 0; i < NK; ++i) A[i] = M::zero_op();

    unsigned char *u_wr = u_rm + r * UROW + 8 * ES * a;
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    const unsigned char *y_rd = y_st + r * YROW + 32 * a;

    // a lane's input row: x, B, C vectors, or the three thirds of the interleaved row
    auto load_in = [&](int64_t t, Row<T> (&p)[3], bool with_c) {
        if constexpr (PK) {
            const T *src = C + 3 * (col + t * d);
            p[0] = ldg_row(src); p[1] = ldg_row(src + 8); p[2] = ldg_row(src + 16);
        } else {
            p[0] = ldg_row(x + col + t * d);
            p[1] = ldg_row(B + col + t * d);
            p[2] = with_c ? ldg_row(C + col + t * d) : zero_row<T>();
        }
    };
    Row<T> in[3];
    auto fetch = [&](int64_t s, Row<T> (&p)[3]) {
        const int64_t t = s * STEP + r;
        p[0] = zero_row<T>(); p[1] = zero_row<T>(); p[2] = zero_row<T>();
        if (cvalid && t < L) load_in(t, p, true);
    };
    fetch(s_lo, in);

    // A segment that starts inside the sequence first rebuilds the operands of the NK-1 steps
    // before it.  Their rows are requested together, so the replay costs one memory latency
    // instead of NK-1; step s_lo-i lands in ring slot NK-i, where phase 0 expects it.
    constexpr int NLEAD = NK > 1 ? NK - 1 : 1;
    Row<T> lead[NLEAD][3];
    if constexpr (NK > 1) {
        if (s_lo > 0) {
#pragma unroll
            for (int i = 1; i < NK; ++i) {
                const int64_t t = (s_lo - i) * STEP + r;
                lead[i - 1][0] = zero_row<T>(); lead[i - 1][1] = zero_row<T>(); lead[i - 1][2] = zero_row<T>();
                if (cvalid && t >= 0) load_in(t, lead[i - 1], false);
            }
        }
    }

    // While those rows are in flight: filter table of this wave's group,
    // htab[lag + 32] = h[hl-1-lag] for 0 <= lag < hl, else 0, and the Toeplitz operand tiles.
    {
        const int64_t cw = c0 + 16 * w;
        const int64_t grp = (cw < d) ? cw / dm.dg : 0;
        const hraw_t *hg = (const hraw_t *)h + grp * hl;
        for (int i = l; i < HTAB; i += 64) {
            const int lag = i - HPAD;
            htab[w][i] = (lag >= 0 && lag < hl) ? hg[hl - 1 - lag] : (hraw_t)0;
        }
    }
    __syncthreads();
    op_t W0[NK], W1[NK];   // output rows 0..15 / 16..31 of the step against input step s-i
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = M::toeplitz(htab[w], 32 * i, j, q);
        W1[i] = M::toeplitz(htab[w], 32 * i + 16, j, q);
    }

    if constexpr (NK > 1) {
        if (s_lo > 0) {
#pragma unroll
            for (int i = 1; i < NK; ++i) {
                float xf[8], Bf[8], Cf[8], uf[8];
                in_floats<T, PK>(lead[i - 1], xf, Bf, Cf);
#pragma unroll
                for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
                lds_store_row<T>(u_wr, pack8<T>(uf));
                __syncthreads();
                A[NK - i] = M::load_operand(u_rm, UROW, w, j, q, false);
                __syncthreads();
            }
        }
    }

    int64_t s = s_lo;
    while (s < s_hi) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < s_hi) {
                Row<T> nx[3] = {zero_row<T>(), zero_row<T>(), zero_row<T>()};
                if (s + 1 < s_hi) fetch(s + 1, nx);

                float xf[8], Bf[8], Cf[8], uf[8];
                in_floats<T, PK>(in, xf, Bf, Cf);
#pragma unroll
                for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
                const Row<T> up = pack8<T>(uf);
                lds_store_row<T>(u_wr, up);
                const int64_t t = s * STEP + r;
                const bool store_ok = cvalid && t < L;
                if (bxo && store_ok) stg_row(bxo + col + t * d, up);
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
                if (store_ok) {
                    const f32x4 p0 = *(const f32x4 *)y_rd;
                    const f32x4 p1 = *(const f32x4 *)(y_rd + 16);
                    float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                    float yf[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) yf[e] = Cf[e] * y2f[e];
                    stg_row(y + col + t * d, pack8<T>(yf));
                    if (y2o) stg_row(y2o + col + t * d, pack8<T>(y2f));
                }
                in[0] = nx[0]; in[1] = nx[1]; in[2] = nx[2];
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
// (one 32-deep product contracts 16 channels x 2 row halves), lag = 16*delta + i - j.  At the
// end the diagonals of the P tiles are summed in a fixed order into per-wave partials in
// the workspace, and a second kernel adds the partials in a fixed order.
//
// PK: x, B, C are interleaved in one tensor that starts at C, and dx, dB, dC in one that starts
// at dC (element stride 3).  C of step sigma+NK-1 then arrives together with x, B of that step,
// NK-1 iterations before they are used, and the outputs of a row leave as one interleaved row.
// The early x, B rows wait in LDS: each lane parks its own two row vectors in a ring of NK-1
// slots and reads them back itself, so the ring needs no barrier.
template <typename T, int NK, int NW, bool PK>
__global__ __launch_bounds__(64 * NW) void mfma_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                       const T *__restrict__ B, const T *__restrict__ C,
                                                       const T *__restrict__ h, T *__restrict__ dx,
                                                       T *__restrict__ dB, T *__restrict__ dC,
                                                       float *__restrict__ ws, Dims dm, MfmaPlan pl)
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
    constexpr int OFF_XB = (OFF_H + NW * HTAB * (int)sizeof(hraw_t) + 15) & ~15;   // PK: waiting x, B rows
    constexpr int XB_SLOTS = (PK && NK > 1) ? NK - 1 : 0;
    constexpr int XB_VEC = G::NT * 16 * M::RW;              // one row vector of every lane
    constexpr int LDS_MAIN = OFF_XB + XB_SLOTS * 2 * XB_VEC;
    constexpr int LDS_TAIL = NW * ND * 256 * 4;             // P tiles at the end
    constexpr int LDS_BYTES = LDS_MAIN > LDS_TAIL ? LDS_MAIN : LDS_TAIL;
    static_assert(LDS_BYTES <= 160 * 1024, "workgroup exceeds the 160 KB of LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_BYTES];
    unsigned char *u_rm = smem + OFF_U, *g_rm = smem + OFF_G, *y_st = smem + OFF_Y, *d_st = smem + OFF_D;
    hraw_t *htab = (hraw_t *)(smem + OFF_H);

    const int64_t wg_id = xcd_contiguous_id(blockIdx.x, gridDim.x);
    int64_t wg = wg_id;
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

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;

    const bool cvalid = c0 + 8 * a < d;
    const int64_t col = b * L * d + c0 + 8 * a;

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
    const int rm_off = r * UROW + 8 * ES * a;                                 // row layout, 8 channels
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    unsigned char *d_wr = d_st + (15 - j) * YROW + (16 * w + 4 * q) * 4;      // columns come out reversed
    const unsigned char *y_rd = y_st + r * YROW + 32 * a;
    const unsigned char *d_rd = d_st + r * YROW + 32 * a;
    unsigned char *xb_own = smem + OFF_XB + tid * 16 * M::RW;                 // PK: slot k at + k * 2 * XB_VEC

    // Rows of iteration sg.  Separate tensors: in[0], in[1] = x, B of step sg; in[2] = C and dyo = dy
    // of step sg+NK-1.  PK: in[] = the interleaved row and dyo = dy of step sg+NK-1.  Zero outside
    // the sequence.
    auto fetch = [&](int64_t sg, Row<T> (&in)[3], Row<T> &dyo) {
        in[0] = zero_row<T>(); in[1] = zero_row<T>(); in[2] = zero_row<T>(); dyo = zero_row<T>();
        if (cvalid) {
            const int64_t t = sg * STEP + r;
            const int64_t t2 = t + (NK - 1) * STEP;
            if constexpr (PK) {
                if (t2 >= 0 && t2 < L) {
                    const T *src = C + 3 * (col + t2 * d);
                    in[0] = ldg_row(src); in[1] = ldg_row(src + 8); in[2] = ldg_row(src + 16);
                    dyo = ldg_row(dy + col + t2 * d);
                }
            } else {
                if (t >= 0 && t < L) {
                    in[0] = ldg_row(x + col + t * d);
                    in[1] = ldg_row(B + col + t * d);
                }
                if (t2 >= 0 && t2 < L) {
                    dyo = ldg_row(dy + col + t2 * d);
                    in[2] = ldg_row(C + col + t2 * d);
                }
            }
        }
    };
    Row<T> in[3], dyr;
    fetch(s_lo, in, dyr);

    // Lead-in: u of the NK-1 steps before the segment and g2 of its first NK-1 steps, i.e. the
    // rows iterations s_lo-NK+1 .. s_lo-1 would have brought.  They are requested together,
    // so the lead-in costs one memory latency instead of NK-1.
    constexpr int NLEAD = NK > 1 ? NK - 1 : 1;
    Row<T> lead[NLEAD][3], wdy[NLEAD];
    Row<T> past[PK ? NLEAD : 1][3];            // PK: the interleaved rows of steps s_lo-1 .. s_lo-NK+1
    if constexpr (NK > 1) {
        if constexpr (PK) {
#pragma unroll
            for (int i = 1; i < NK; ++i) {
                const int64_t t = (s_lo - i) * STEP + r;
                past[i - 1][0] = zero_row<T>(); past[i - 1][1] = zero_row<T>(); past[i - 1][2] = zero_row<T>();
                if (cvalid && t >= 0) {
                    const T *src = C + 3 * (col + t * d);
                    past[i - 1][0] = ldg_row(src); past[i - 1][1] = ldg_row(src + 8); past[i - 1][2] = ldg_row(src + 16);
                }
            }
        }
#pragma unroll
        for (int i = 1; i < NK; ++i) fetch(s_lo - i, lead[i - 1], wdy[i - 1]);
    }

    // While those rows are in flight: the filter table of this wave's group and the Toeplitz tiles.
    {
        const int64_t grp = wave_valid ? (c0 + 16 * w) / dm.dg : 0;
        const hraw_t *hg = (const hraw_t *)h + grp * hl;
        for (int i = l; i < HTAB; i += 64) {
            const int lag = i - HPAD;
            htab[w * HTAB + i] = (lag >= 0 && lag < hl) ? hg[hl - 1 - lag] : (hraw_t)0;
        }
    }
    __syncthreads();
    op_t W0[NK], W1[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = M::toeplitz(htab + w * HTAB, 32 * i, j, q);
        W1[i] = M::toeplitz(htab + w * HTAB, 32 * i + 16, j, q);
    }

    if constexpr (NK > 1) {
#pragma unroll
        for (int i = 1; i < NK; ++i) {
            // iteration s_lo-i carries u of step s_lo-i and g2 / dy of step s_lo+NK-1-i
            float f0[8], f1[8], f2[8], tf[8], pf[8];
            if constexpr (PK) {
                in_floats<T, true>(past[i - 1], f0, f1, f2);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = f0[e] * f1[e];
                lds_store_row<T>(u_rm + rm_off, pack8<T>(pf));
                // x, B of step s_lo+NK-1-i wait in ring slot (NK-1-i) % (NK-1) for iteration s_lo+NK-1-i
                in_floats<T, true>(lead[i - 1], f0, f1, f2);
                unsigned char *slot = xb_own + ((NK - 1 - i) % (NK - 1)) * 2 * XB_VEC;
                lds_store_row<T>(slot, pack8<T>(f0));
                lds_store_row<T>(slot + XB_VEC, pack8<T>(f1));
            } else {
                unpack8<T>(lead[i - 1][0], f0);
                unpack8<T>(lead[i - 1][1], f1);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = f0[e] * f1[e];
                lds_store_row<T>(u_rm + rm_off, pack8<T>(pf));
                unpack8<T>(lead[i - 1][2], f2);
            }
            unpack8<T>(wdy[i - 1], tf);
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = tf[e] * f2[e];
            unsigned char *g_slot = g_rm + (NK - 1 - i) * STEP * UROW;
            lds_store_row<T>(g_slot + rm_off, pack8<T>(pf));
            dyq[NK - 1 - i] = wdy[i - 1];
            __syncthreads();
            Au[NK - i] = M::load_operand(u_rm, UROW, w, j, q, false);
            Ag[NK - 1 - i] = M::load_operand(g_slot, UROW, w, j, q, true);
            __syncthreads();
        }
    }

    int xb_slot = 0;      // PK: ring slot of step s (steps s_lo+k sit in slot k % (NK-1))
    int64_t s = s_lo;
    while (s < s_hi) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < s_hi) {
                const int slot_new = (ph + NK - 1) % NK;     // ring slot of step s+NK-1
                Row<T> nx[3] = {zero_row<T>(), zero_row<T>(), zero_row<T>()}, dyn = zero_row<T>();
                if (s + 1 < s_hi) fetch(s + 1, nx, dyn);

                float xf[8], Bf[8], tf[8], cf[8], pf[8];
                if constexpr (PK) {
                    float xa[8], Ba[8];
                    in_floats<T, true>(in, xa, Ba, cf);       // x, B, C of step s+NK-1
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
                } else {
                    unpack8<T>(in[0], xf);
                    unpack8<T>(in[1], Bf);
                    unpack8<T>(in[2], cf);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = xf[e] * Bf[e];
                lds_store_row<T>(u_rm + rm_off, pack8<T>(pf));
                unpack8<T>(dyr, tf);
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = tf[e] * cf[e];
                unsigned char *g_slot = g_rm + slot_new * STEP * UROW;
                lds_store_row<T>(g_slot + rm_off, pack8<T>(pf));
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
                    const op_t un = M::load_natural(u_rm + j * UROW, u_rm + (16 + j) * UROW, w, q);
#pragma unroll
                    for (int dl = 0; dl < ND; ++dl) {
                        int row0 = STEP * ph + 16 * dl + j;              // ring rows of the window's two halves
                        int row1 = row0 + 16;
                        row0 = (row0 >= RING_ROWS) ? row0 - RING_ROWS : row0;
                        row1 = (row1 >= RING_ROWS) ? row1 - RING_ROWS : row1;
                        const op_t gn = M::load_natural(g_rm + row0 * UROW, g_rm + row1 * UROW, w, q);
                        P[dl] = M::mfma(gn, un, P[dl]);
                    }
                }
                __syncthreads();
                const int64_t t = s * STEP + r;
                if (cvalid && t < L) {
                    const int64_t o = col + t * d;
                    const f32x4 p0 = *(const f32x4 *)y_rd;
                    const f32x4 p1 = *(const f32x4 *)(y_rd + 16);
                    const float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                    const f32x4 e0 = *(const f32x4 *)d_rd;
                    const f32x4 e1 = *(const f32x4 *)(d_rd + 16);
                    const float duf[8] = {e0[0], e0[1], e0[2], e0[3], e1[0], e1[1], e1[2], e1[3]};
                    float dyf[8], oC[8], ox[8], oB[8];
                    unpack8<T>(dyq[ph], dyf);
#pragma unroll
                    for (int e = 0; e < 8; ++e) oC[e] = dyf[e] * y2f[e];
                    if constexpr (!PK) stg_row(dC + o, pack8<T>(oC));
#pragma unroll
                    for (int e = 0; e < 8; ++e) ox[e] = duf[e] * Bf[e];
                    if constexpr (!PK) stg_row(dx + o, pack8<T>(ox));
#pragma unroll
                    for (int e = 0; e < 8; ++e) oB[e] = duf[e] * xf[e];
                    if constexpr (!PK) stg_row(dB + o, pack8<T>(oB));
                    if constexpr (PK) {
                        Row<T> po[3];
                        join_rows<T>(ox, oB, oC, po);
                        T *dst = dC + 3 * o;
                        stg_row(dst, po[0]); stg_row(dst + 8, po[1]); stg_row(dst + 16, po[2]);
                    }
                }
                in[0] = nx[0]; in[1] = nx[1]; in[2] = nx[2]; dyr = dyn;
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
        float *out = ws + ((size_t)wg_id * NW + w) * 128;
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
// fp32 doubles the register state per wave (operand tiles hold 8 floats), which caps the
// forward at 8 waves and the backward at 4.
int choose_nw(const Dims &dm, bool fp32)
{
    static const int forced = env_int("GCG_MFMA_NW", 0);   // tuning override: 4, 8 or 16
    if (forced == 4 || forced == 8 || (forced == 16 && !fp32)) return forced;
    if (dm.d >= 256 && !fp32) return 16;
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
    // 16-bit: ~112 registers, 4 waves per SIMD; fp32: ~200 registers, 2 waves per SIMD
    const MfmaPlan p = plan(dm, NW, 16, sizeof(T) == 4 ? 8 : 16);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (dm.es == 3)
        hipLaunchKernelGGL((mfma_fwd_kernel<T, NK, NW, true>), dim3((unsigned)p.nwg), dim3(64 * NW), 0, st,
                           (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    else
        hipLaunchKernelGGL((mfma_fwd_kernel<T, NK, NW, false>), dim3((unsigned)p.nwg), dim3(64 * NW), 0, st,
                           (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    return (int)hipGetLastError();
}

template <typename T, int NK>
int fwd_nk(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
           const Dims &dm, hipStream_t st)
{
    const int nw = choose_nw(dm, sizeof(T) == 4);
    if constexpr (sizeof(T) == 2) {
        if (nw == 16) return fwd_launch<T, NK, 16>(x, B, C, h, y, y2, bx, dm, st);
    }
    if (nw == 8) return fwd_launch<T, NK, 8>(x, B, C, h, y, y2, bx, dm, st);
    return fwd_launch<T, NK, 4>(x, B, C, h, y, y2, bx, dm, st);
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
    (void)dtype;   // bf16, f16 and fp32 all have a matrix-core form
    return dm.hl <= 128 && dm.dg % 16 == 0;
}

int mfma_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h, void *y,
                    void *y2, void *bx, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return fwd_t<bf16_t>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_F16) return fwd_t<f16_t>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_F32) return fwd_t<float>(x, B, C, h, y, y2, bx, dm, st);
    return (int)hipErrorInvalidValue;
}

bool mfma_bwd_available() { return true; }

namespace {

// The backward holds about twice the forward's register state per wave, so it runs two
// waves per SIMD and at most 8 waves (128 channels, 256-byte rows) per workgroup.
int choose_nw_bwd(const Dims &dm, bool fp32)
{
    static const int forced = env_int("GCG_MFMA_BWD_NW", 0);   // tuning override: 4 or 8
    if (forced == 4 || (forced == 8 && !fp32)) return forced;
    return (dm.d >= 128 && !fp32) ? 8 : 4;
}

// 16-bit: two waves per SIMD (8 per CU); fp32: one (4 per CU)
MfmaPlan plan_bwd(const Dims &dm, bool fp32) { return plan(dm, choose_nw_bwd(dm, fp32), 16, fp32 ? 4 : 8); }

template <typename T, int NK, int NW>
int bwd_launch(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
               void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    const MfmaPlan p = plan_bwd(dm, sizeof(T) == 4);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    if (dm.es == 3)
        hipLaunchKernelGGL((mfma_bwd_kernel<T, NK, NW, true>), dim3((unsigned)p.nwg), dim3(64 * NW), 0, st,
                           (const T *)dy, (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)dx, (T *)dB,
                           (T *)dC, (float *)ws, dm, p);
    else
        hipLaunchKernelGGL((mfma_bwd_kernel<T, NK, NW, false>), dim3((unsigned)p.nwg), dim3(64 * NW), 0, st,
                           (const T *)dy, (const T *)x, (const T *)B, (const T *)C, (const T *)h, (T *)dx, (T *)dB,
                           (T *)dC, (float *)ws, dm, p);
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
    if constexpr (sizeof(T) == 2) {
        if (choose_nw_bwd(dm, false) == 8) return bwd_launch<T, NK, 8>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    }
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

size_t mfma_bwd_workspace(int dtype, const Dims &dm)
{
    const MfmaPlan p = plan_bwd(dm, dtype == GCG_F32);
    return (size_t)p.nwg * p.nw * 128 * sizeof(float);
}

int mfma_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C, const void *h,
                    void *dx, void *dB, void *dC, void *dh, void *ws, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return bwd_t<bf16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dtype == GCG_F16) return bwd_t<f16_t>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    if (dtype == GCG_F32) return bwd_t<float>(dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st);
    return (int)hipErrorInvalidValue;
}

} // namespace gcg
