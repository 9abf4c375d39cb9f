// Shared pieces of the matrix-core kernels: element-type traits of the 32-deep banded-Toeplitz
// product, the row-vector helpers, streaming loads and stores, the filter-gradient reduction
// and the host-side launch plan.  Included by the separate-tensor kernels (gcg_mfma.hip) and
// the interleaved-features kernels (gcg_mfma_il.hip).
#pragma once
#include "gcg_common.h"

#include <atomic>
#include <cstdlib>
#include <mutex>
#include <type_traits>

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

// The transposed operand of the 32-deep product from a row-major LDS tile of 16-bit elements: time samples
// 8q .. 8q+7 of channel 16w+j from rows 0..31 (reversed: 31-k).
__device__ __forceinline__ uint4 tr_operand16(const unsigned char *tile, int urow, int w, int j, int q, bool reversed)
{
    const int col = (16 * w + 4 * (j & 3)) * 2;
    const int r0 = reversed ? 31 - 8 * q - (j >> 2) : 8 * q + (j >> 2);
    const int r1 = reversed ? r0 - 4 : r0 + 4;
    const s16x4 lo = lds_read_tr(tile + r0 * urow + col);
    const s16x4 hi = lds_read_tr(tile + r1 * urow + col);
    const short v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    uint4 r;
    __builtin_memcpy(&r, v, 16);
    return r;
}

template <typename OP> struct MT16 {
    static constexpr int ES = 2;                 // bytes per element in memory
    static constexpr int RW = 1;                 // 16-byte words per 8-channel row vector
    static constexpr int LES = 2;                // bytes per element of the operand tiles in LDS
    static constexpr bool SPLIT = false;         // operands are the tensors' own 16-bit values
    // bytes per LDS row of an operand tile of cb channels; the padding makes consecutive rows start 8 banks apart
    static constexpr int urow(int cb) { return cb * 2 + 32; }
    typedef OP op_t;                             // operand made of activations
    typedef OP wop_t;                            // operand made of filter taps
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
        const uint4 t4 = tr_operand16(tile, urow, w, j, q, reversed);
        op_t r;
        __builtin_memcpy(&r, &t4, 16);
        return r;
    }
    // natural-layout operand of the filter-gradient product: 8 channels of one of two rows;
    // lane quad q takes row half q>>1 and channels 8*(q&1)..+7 of the wave's 16
    static __device__ __forceinline__ op_t load_natural(const unsigned char *row_half0,
                                                        const unsigned char *row_half1, int urow, int w, int q)
    {
        (void)urow;
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
    typedef bf16_t filt_t;                       // element type of h and dh
    static __device__ __forceinline__ hraw_t to_hraw(float v) { return (hraw_t)float_to_bf16_bits(v); }
    static __device__ __forceinline__ float from_hraw(hraw_t v) { return bf16_bits_to_float(v); }
    static __device__ __forceinline__ f32x4 mfma(op_t a, op_t b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma_aa(op_t a, op_t b, f32x4 c) { return mfma(a, b, c); }
    static __device__ __forceinline__ void unpack2(uint32_t p, float &lo, float &hi)
    {
        lo = __uint_as_float(p << 16);
        hi = __uint_as_float(p & 0xffff0000u);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
};
template <> struct MT<f16_t> : MT16<f16x8> {
    typedef f16_t filt_t;
    static __device__ __forceinline__ hraw_t to_hraw(float v)
    {
        const _Float16 hv = (_Float16)v;
        hraw_t r;
        __builtin_memcpy(&r, &hv, 2);
        return r;
    }
    static __device__ __forceinline__ float from_hraw(hraw_t v)
    {
        _Float16 hv;
        __builtin_memcpy(&hv, &v, 2);
        return (float)hv;
    }
    static __device__ __forceinline__ f32x4 mfma(op_t a, op_t b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma_aa(op_t a, op_t b, f32x4 c) { return mfma(a, b, c); }
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

// fp32 arithmetic on the bf16 matrix cores.  An fp32 value is the exact sum of three bf16 values (8 significant
// bits each: v1 = bf16(v), v2 = bf16(v - v1), v3 = bf16(v - v1 - v2)), and the product of two bf16 values is
// exact in the fp32 accumulator, so  a * b  =  sum of a_m * b_n  over the planes; the terms with m + n <= 4 carry
// it to 2^-24 relative to |a b| (the ones left out are below that), i.e. to fp32 accuracy, at 6 matrix
// instructions of 16 cycles instead of the 8 fp32 ones of 32 cycles that the same 32-deep product costs on the
// fp32 matrix path.  Operand tiles in LDS hold the planes of a row side by side (plane m at byte offset
// m * plane(urow)), each laid out like a 16-bit tile, so operands come from the same transposing reads.
//
// NPA = planes of an activation operand.  fp32 tensors: 3.  bf16 tensors computed in fp32: 2, exactly (the pre-gate
// product of two bf16 values has 16 significant bits).  f16 tensors computed in fp32: 3 (22 significant bits).
// NPW = planes of a filter operand.  fp32 tensors: 3 (results to fp32 accuracy).  16-bit tensors with an fp32
// filter: 2 -- the taps enter the products rounded to 16 significant bits (2^-17 relative), 256 times below the
// resolution of the 16-bit outputs they are rounded to (over 99 % of the outputs still equal the exact result
// rounded once).
// SUM = the largest m + n of the plane products a_m b_n that are formed.  2 for fp32 and f16 tensors (6 and 5
// terms).  1 for bf16 tensors: the term left out, low plane times low plane, is at most 2^-18 of |a b|, which is
// 2^-9 of an output's last bit and, in the filter gradient, four orders of magnitude below what adding bs L dg
// products in fp32 leaves.  3 terms instead of 4: a single wave issues matrix and vector instructions strictly one
// after the other, so with one wave per SIMD every matrix instruction left out is time saved (7B layer shape, bf16
// tensors in fp32 arithmetic: forward 109 -> 99 -> 95.5 us, backward 282 -> 257 -> 232 us for 3 -> 2 filter
// planes -> 3 terms).
template <int NPA> struct SplitOp { bf16x8 p[NPA]; };
template <int NPA_, int NPW_, int SUM_> struct MTSplit {
    static constexpr int LES = 2;
    static constexpr bool SPLIT = true;
    static constexpr int NPA = NPA_, NPW = NPW_;
    static constexpr int SUM = SUM_;             // plane products a_m b_n with m + n <= SUM are formed
    static constexpr int RPAD = 32;              // with it consecutive rows start an odd multiple of 8 banks apart
    static constexpr int urow(int cb) { return NPA * cb * 2 + RPAD; }
    static __device__ __forceinline__ int plane(int urow) { return (urow - RPAD) / NPA; }   // bytes between planes
    typedef SplitOp<NPA> op_t;
    typedef SplitOp<NPW> wop_t;
    typedef float hraw_t;
    typedef float filt_t;
    static __device__ __forceinline__ hraw_t to_hraw(float v) { return v; }
    static __device__ __forceinline__ float from_hraw(hraw_t v) { return v; }
    static __device__ __forceinline__ int kmap(int q, int e) { return 8 * q + e; }
    template <int N> static __device__ __forceinline__ void split(float v, uint16_t (&o)[N])
    {
#pragma unroll
        for (int m = 0; m < N; ++m) {
            o[m] = (uint16_t)float_to_bf16_bits(v);
            if (m + 1 < N) v -= bf16_bits_to_float(o[m]);
        }
    }
    static __device__ __forceinline__ op_t zero_op()
    {
        op_t r;
        const uint4 z = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int m = 0; m < NPA; ++m) __builtin_memcpy(&r.p[m], &z, 16);
        return r;
    }
    static __device__ __forceinline__ op_t load_operand(const unsigned char *tile, int urow, int w, int j, int q,
                                                        bool reversed)
    {
        op_t r;
#pragma unroll
        for (int m = 0; m < NPA; ++m) {
            const uint4 t4 = tr_operand16(tile + m * plane(urow), urow, w, j, q, reversed);
            __builtin_memcpy(&r.p[m], &t4, 16);
        }
        return r;
    }
    static __device__ __forceinline__ op_t load_natural(const unsigned char *row_half0,
                                                        const unsigned char *row_half1, int urow, int w, int q)
    {
        const unsigned char *p = ((q >> 1) ? row_half1 : row_half0) + (16 * w + 8 * (q & 1)) * 2;
        op_t r;
#pragma unroll
        for (int m = 0; m < NPA; ++m) {
            const uint4 t4 = *(const uint4 *)(p + m * plane(urow));
            __builtin_memcpy(&r.p[m], &t4, 16);
        }
        return r;
    }
    static __device__ __forceinline__ wop_t toeplitz(const hraw_t *htab, int doff, int j, int q)
    {
        uint16_t v[NPW][8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            uint16_t o[NPW];
            split<NPW>(htab[doff + j - kmap(q, e) + HPAD], o);
#pragma unroll
            for (int m = 0; m < NPW; ++m) v[m][e] = o[m];
        }
        wop_t r;
#pragma unroll
        for (int m = 0; m < NPW; ++m) __builtin_memcpy(&r.p[m], v[m], 16);
        return r;
    }
    // smallest terms first
    template <int NA, int NB>
    static __device__ __forceinline__ f32x4 mfma_terms(const SplitOp<NA> &a, const SplitOp<NB> &b, f32x4 c)
    {
#pragma unroll
        for (int sum = SUM; sum >= 0; --sum)
#pragma unroll
            for (int m = 0; m <= sum; ++m)
                if (m < NA && sum - m < NB)
                    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.p[m], b.p[sum - m], c, 0, 0, 0);
        return c;
    }
    static __device__ __forceinline__ f32x4 mfma(const op_t &a, const wop_t &b, f32x4 c)
    {
        return mfma_terms<NPA, NPW>(a, b, c);
    }
    static __device__ __forceinline__ f32x4 mfma_aa(const op_t &a, const op_t &b, f32x4 c)
    {
        return mfma_terms<NPA, NPA>(a, b, c);
    }
    // a lane's 8 channels of one row into the planes of an operand tile
    static __device__ __forceinline__ void store_f8(unsigned char *p, int urow, const float (&f)[8])
    {
        uint16_t v[NPA][8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            uint16_t o[NPA];
            split<NPA>(f[e], o);
#pragma unroll
            for (int m = 0; m < NPA; ++m) v[m][e] = o[m];
        }
#pragma unroll
        for (int m = 0; m < NPA; ++m) {
            uint4 t4;
            __builtin_memcpy(&t4, v[m], 16);
            *(uint4 *)(p + m * plane(urow)) = t4;
        }
    }
};
template <> struct MT<float> : MTSplit<3, 3, 2> {
    static constexpr int ES = 4;                 // bytes per element in memory
    static constexpr int RW = 2;                 // 16-byte words per 8-channel row vector
};
// bf16 / f16 tensors, fp32 filter, fp32 arithmetic: what a 16-bit model gets from the operator run "in fp32"
// (every tensor cast up before it and the result cast down after), without the casts.
template <> struct MT<bf16w_t> : MTSplit<2, 2, 1> {
    static constexpr int ES = 2;
    static constexpr int RW = 1;
    static __device__ __forceinline__ void unpack2(uint32_t p, float &lo, float &hi) { MT<bf16_t>::unpack2(p, lo, hi); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
};
template <> struct MT<f16w_t> : MTSplit<3, 2, 2> {
    static constexpr int ES = 2;
    static constexpr int RW = 1;
    static __device__ __forceinline__ void unpack2(uint32_t p, float &lo, float &hi) { MT<f16_t>::unpack2(p, lo, hi); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_f16x2(lo, hi); }
};

// CYCLES idle cycles of the wave, and nothing scheduled across them
template <int CYCLES> __device__ __forceinline__ void idle_cycles()
{
#pragma unroll
    for (int i = 0; i < CYCLES / 16; ++i) asm volatile("s_nop 15");
    if constexpr (CYCLES % 16 != 0) asm volatile("s_nop %0" ::"n"(CYCLES % 16 - 1));
    __builtin_amdgcn_sched_barrier(0);
}

// A workgroup of NW waves owns CB = 16*NW adjacent channels; LDS rows are padded (see MT<T>::urow;
// the fp32 result tile: consecutive rows start 4 banks apart).
template <typename T, int NW> struct Geo {
    static constexpr int CB = 16 * NW;                          // channels per workgroup
    static constexpr int LPR = CB / 8;                          // lanes per row in the row layout (8 channels each)
    static constexpr int UROW = MT<T>::urow(CB);                // bytes per LDS row of u / g2
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

// a lane's 8 channels of one row into a matrix-operand tile (in the tile's own element format)
template <typename T> __device__ __forceinline__ void store_operand(unsigned char *p, int urow, const float (&f)[8])
{
    if constexpr (MT<T>::SPLIT) MT<T>::store_f8(p, urow, f);
    else *(uint4 *)p = pack8<T>(f).w[0];
}

template <typename T> __device__ __forceinline__ Row<T> lds_load_row(const unsigned char *p)
{
    Row<T> r;
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) r.w[i] = *(const uint4 *)(p + 16 * i);
    return r;
}

// 16-, 12- and 4-byte accesses of a tensor window (gcg_common.h)
__device__ __forceinline__ uint4 ldw16(win_t w, uint32_t off)
{
    const u32x4 v = win_load<u32x4>(w, off);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void stw16(win_t w, uint32_t off, const uint4 &v)
{
    win_store(w, off, u32x4{v.x, v.y, v.z, v.w});
}
__device__ __forceinline__ u32x3 ldw12(win_t w, uint32_t off) { return win_load<u32x3>(w, off); }
__device__ __forceinline__ void stw12(win_t w, uint32_t off, const u32x3 &v) { win_store(w, off, v); }
__device__ __forceinline__ uint32_t ldw4(win_t w, uint32_t off) { return win_load<uint32_t>(w, off); }
__device__ __forceinline__ void stw4(win_t w, uint32_t off, uint32_t v) { win_store(w, off, v); }
template <typename T> __device__ __forceinline__ Row<T> ldw_row(win_t w, uint32_t off)
{
    Row<T> r;
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) r.w[i] = ldw16(w, off + 16 * i);
    return r;
}
template <typename T> __device__ __forceinline__ void stw_row(win_t w, uint32_t off, const Row<T> &r)
{
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) stw16(w, off + 16 * i, r.w[i]);
}
template <typename T, int AUX> __device__ __forceinline__ Row<T> ldw_row_policy(win_t w, uint32_t off)
{
    Row<T> r;
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i) {
        const u32x4 v = win_load_policy<AUX>(w, off + 16 * i);
        r.w[i] = make_uint4(v[0], v[1], v[2], v[3]);
    }
    return r;
}
// the same with the store's cache-policy bits given (gcg_common.h: win_store_policy)
template <typename T, int AUX> __device__ __forceinline__ void stw_row_policy(win_t w, uint32_t off, const Row<T> &r)
{
#pragma unroll
    for (int i = 0; i < MT<T>::RW; ++i)
        win_store_policy<AUX>(w, off + 16 * i, u32x4{r.w[i].x, r.w[i].y, r.w[i].z, r.w[i].w});
}

// The filter table of a wave's group: tab[lag + HPAD] = h[hl-1-lag] for 0 <= lag < hl, else 0; lane l
// holds entries l, l + 64, l + 128 between load_taps and store_taps.  The taps come from h, or -- decayed
// explicit filter -- are formed here as F(fw * fdecay).  Both sources are read through windows, the one not
// in use empty (its loads return zero and touch no memory), so there is no branch around a load: the taps
// are requested before the first tensor rows, and a branch would make their use wait for those rows too.
template <typename T>
__device__ __forceinline__ void load_taps(const Dims &dm, const void *h, int64_t grp, int l,
                                          typename MT<T>::hraw_t (&hv)[HTAB / 64])
{
    typedef MT<T> M;
    typedef typename M::hraw_t hraw_t;
    const bool dec = dm.fw != nullptr;
    const int hl = dm.hl;
    const win_t wh = make_window(h, dec ? 0 : (int64_t)dm.g * hl * (int64_t)sizeof(hraw_t));
    const win_t ww = make_window(dm.fw, dec ? (int64_t)dm.g * dm.lc * 4 : 0);
    const win_t wd = make_window(dm.fdecay, dec ? (int64_t)dm.g * dm.lc * 4 : 0);
#pragma unroll
    for (int k = 0; k < HTAB / 64; ++k) {
        const int lag = l + 64 * k - HPAD;
        const bool in = lag >= 0 && lag < hl;
        const int tap = in ? hl - 1 - lag : 0;
        const uint32_t oh = (uint32_t)((grp * hl + tap) * (int64_t)sizeof(hraw_t));
        const uint32_t od = (uint32_t)((grp * dm.lc + tap) * 4);
        hraw_t plain;
        if constexpr (sizeof(hraw_t) == 2) plain = (hraw_t)win_load_u16(wh, oh);
        else plain = win_load_f32_cached(wh, oh);
        const hraw_t made = M::to_hraw(win_load_f32_cached(ww, od) * win_load_f32_cached(wd, od));
        const hraw_t v = dec ? made : plain;
        hv[k] = in ? v : (hraw_t)0;
    }
}
template <typename H> __device__ __forceinline__ void store_taps(H *tab, int l, const H (&hv)[HTAB / 64])
{
#pragma unroll
    for (int k = 0; k < HTAB / 64; ++k) tab[l + 64 * k] = hv[k];
}
// one value of the filter gradient: dh[grp, k] in the filter's element type, or -- decayed filter -- the
// gradient of fw, dw[grp, k] = float(F(dh[grp, k])) * fdecay[grp, k]
template <typename T> __device__ __forceinline__ void store_dh(void *dh, const Dims &dm, int64_t grp, int k, float sum)
{
    typedef MT<T> M;
    typedef typename M::filt_t F;
    if (dm.fw) ((float *)dh)[grp * dm.lc + k] = M::from_hraw(M::to_hraw(sum)) * dm.fdecay[grp * dm.lc + k];
    else Elem<F>::store((F *)dh + grp * dm.hl + k, sum);
}

// Exact division of a number below 2^31 by a launch constant d: n / d = (n * mul) >> sh, with
// sh = 31 + ceil(log2 d) and mul = ceil(2^sh / d) < 2^32 (the error n * (mul * d - 2^sh) / (d * 2^sh) stays
// below 1 / d because n * d <= 2^sh).  A workgroup finds its place in the launch with two of these instead of
// 64-bit divisions: with sixteen waves per CU sharing one scalar unit those took over a microsecond before
// the first load went out.
struct FastDiv { uint32_t mul, sh; };
inline FastDiv make_fastdiv(uint32_t d)
{
    int l = 0;
    while ((1ull << l) < d) ++l;
    FastDiv f;
    f.sh = 31u + (uint32_t)l;
    f.mul = (uint32_t)(((1ull << f.sh) + d - 1) / d);
    return f;
}
__device__ __forceinline__ uint32_t fdiv(uint32_t n, FastDiv f) { return (uint32_t)(((uint64_t)n * f.mul) >> f.sh); }

struct MfmaPlan {
    int ncb, nseg, steps_per_seg, nw, xcd;
    int64_t nsteps, nwg;
    int fuse_dh, slot;
    FastDiv q_ncb, q_nseg, q_dg16;      // divisions by ncb, nseg and dg / 16
};

// (channel block, segment, batch row) of a workgroup from its index in the launch (below 2^31)
__device__ __forceinline__ void wg_place(uint32_t id, const MfmaPlan &pl, int &cb, int &seg, int &b)
{
    const uint32_t t = fdiv(id, pl.q_ncb);
    cb = (int)(id - t * (uint32_t)pl.ncb);
    const uint32_t bq = fdiv(t, pl.q_nseg);
    seg = (int)(t - bq * (uint32_t)pl.nseg);
    b = (int)bq;
}

// Operand tile of the banded Toeplitz matrix at row offset doff = (out time) - (in time) of the
// tile origins: element e of lane (j, q) is the tap for lag doff + j - kmap(q, e)  (MT<T>::toeplitz).


// dh[grp][k] = sum of the per-wave partials of the 16-channel blocks of the group
template <typename T>
__global__ __launch_bounds__(256) void mfma_dh_reduce_kernel(const float *__restrict__ ws, T *__restrict__ dh,
                                                             Dims dm, MfmaPlan pl)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int row = dm.fw ? dm.lc : dm.hl;                // taps per group in the output
    if (i >= (int64_t)dm.g * row) return;
    const int64_t grp = i / row;
    const int k = (int)(i % row);
    if (k >= dm.hl) {                                    // the parameter's taps beyond the filter in use
        ((float *)dh)[i] = 0.f;
        return;
    }
    const int lag = dm.hl - 1 - k;
    const int bpg = dm.dg / 16;                          // 16-channel blocks per group
    const int64_t slots = (int64_t)pl.ncb * pl.nw;       // block slots per (batch, segment)
    float sum = 0.f;
    for (int64_t p = 0; p < dm.bs * pl.nseg; ++p)
        for (int kk = 0; kk < bpg; ++kk)
            sum += ws[(p * slots + grp * bpg + kk) * 128 + lag];
    store_dh<T>(dh, dm, grp, k, sum);
}

// ---- filter-gradient reduction at the end of the backward kernel itself ----------------------
// The workgroups that share a channel block -- one per (batch row, segment) -- each leave a partial
// sum per wave in the workspace.  Instead of a second launch, the last of them to finish adds the
// partials of its channel block, in the same fixed order whoever that is, so dh stays
// bit-reproducible.  "Last" is decided by a ticket per channel block.  The tickets live in the
// library image (zero when the code is loaded; the last arrival puts its ticket back to zero), in
// DH_SLOTS sets.  A set belongs to a stream (dh_slot_for_stream): launches on one stream run one
// after the other, so two launches that may run at the same time never count on the same tickets.
//
// Ordering, in the terms of the AMDGPU memory model for gfx942 / gfx950 (several XCDs, each with an L2 of its own):
//  * partials are written with device-scope atomic stores (sc1): they are written through the XCD's L2, and the
//    store's vmcnt slot is released only when that write has been acknowledged;
//  * every wave then waits for vmcnt(0) -- all of its stores, the partials among them, have completed -- and the
//    workgroup meets at a barrier: only after that does thread 0 take the ticket with a device-scope atomic add
//    (performed where all XCDs see it).  So a workgroup that reads `arrivals` from the ticket knows that every
//    partial of its channel block is in memory;
//  * that workgroup invalidates what its own caches may hold (acquire fence at device scope) and reads the
//    partials with device-scope atomic loads, which are served from beyond the XCD's L2.
// A device-scope release fence instead (the textbook form) writes back the XCD's whole L2, dirty output rows
// included: one per workgroup cost 45 us at the end of a 175 us kernel.
constexpr int DH_SLOTS = 64, DH_UNITS = 1024;
static __device__ unsigned int dh_tickets[DH_SLOTS * DH_UNITS];

// The ticket set of a stream, or -1 when DH_SLOTS other streams already hold one each (the caller then adds the
// partials with a second launch), or when the stream is being captured into a graph (a replayed launch keeps the
// set it was recorded with and would count on it whatever stream it is replayed on).
int dh_slot_for_stream(hipStream_t st)
{
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return -1;
    static std::mutex mu;
    static hipStream_t owner[DH_SLOTS];
    static int used = 0;
    std::lock_guard<std::mutex> lk(mu);
    for (int i = 0; i < used; ++i)
        if (owner[i] == st) return i;
    if (used == DH_SLOTS) return -1;
    owner[used] = st;
    return used++;
}

// Arrival of a workgroup at the ticket of its channel block, after every wave has issued its partial stores.
// Returns true in the one workgroup that arrives last (uniformly over its threads).
__device__ __forceinline__ bool dh_arrive_last(const MfmaPlan &pl, int cb, unsigned int arrivals)
{
    __shared__ unsigned int is_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // this wave's stores have been acknowledged ...
    __syncthreads();                                         // ... and so have the other waves', before the ticket is taken
    if (threadIdx.x == 0) {
        unsigned int *tk = dh_tickets + pl.slot * DH_UNITS + cb;
        const unsigned int mine = __hip_atomic_fetch_add(tk, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
        is_last = (mine == arrivals);
        if (mine == arrivals) __hip_atomic_store(tk, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last) return false;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return true;
}

// Sums of n partials `stride` floats apart, in index order, for two outputs at once; sixteen reads are in flight
// together, so that the sums cost one memory latency per eight terms rather than one per term.
__device__ __forceinline__ void dh_sum_partials2(const float *pa, const float *pb, int64_t stride, int64_t n, float &sa,
                                                 float &sb)
{
    sa = sb = 0.f;
    for (int64_t i0 = 0; i0 < n; i0 += 8) {
        float va[8], vb[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const bool in = i0 + u < n;
            va[u] = __hip_atomic_load(pa + (in ? (i0 + u) * stride : 0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            vb[u] = __hip_atomic_load(pb + (in ? (i0 + u) * stride : 0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            va[u] = in ? va[u] : 0.f;
            vb[u] = in ? vb[u] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            sa += va[u];
            sb += vb[u];
        }
    }
}

// Tail of both backward kernels.  P: the wave's ND accumulator tiles, P[dl][v] = element
// (row 4q+v, column j) of tile dl; smem: at least NW*(16*ND+16)*17*4 bytes of LDS that is no longer in use.
// NT: threads of the workgroup.  holds_tiles: whether this wave holds accumulator tiles (its channel block is w);
// workgroups with more waves than channel blocks pass false in the others, which then only help with the sums.
template <typename T, int NW, int ND, int NT = 64 * NW>
__device__ __forceinline__ void dh_finish(const f32x4 (&P)[ND], unsigned char *smem, float *__restrict__ ws,
                                          T *__restrict__ dh, const Dims &dm, const MfmaPlan &pl, int64_t wg_id,
                                          int cb, bool wave_valid, bool holds_tiles = true, int w = (int)(threadIdx.x >> 6))
{
    const int tid = threadIdx.x, l = tid & 63, j = l & 15, q = l >> 4;
    // The tiles go to LDS one below the other, as one matrix of 16*ND rows (17 floats apart: the diagonal walks
    // below then touch every bank once) followed by 16 rows of zeros.  lag = (row of the matrix) - column, so the
    // partial for a lag is the sum over columns c of element (lag + c, c).
    constexpr int RS = 17, ROWS = 16 * ND + 16;
    __syncthreads();
    float *pt = (float *)smem + w * ROWS * RS;
    if (holds_tiles) {
#pragma unroll
        for (int dl = 0; dl < ND; ++dl)
#pragma unroll
            for (int v = 0; v < 4; ++v) pt[(16 * dl + 4 * q + v) * RS + j] = P[dl][v];
#pragma unroll
        for (int v = 0; v < 4; ++v) pt[(16 * ND + 4 * q + v) * RS + j] = 0.f;
    }
    __syncthreads();
    if (holds_tiles && wave_valid) {
        float *out = ws + ((size_t)wg_id * NW + w) * 128;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int lag = l + 64 * half;
            const float *d = pt + (lag < 16 * ND ? lag : 16 * ND) * RS;   // lags beyond the tiles: the rows of zeros
            float sum = 0.f;
#pragma unroll
            for (int c = 0; c < 16; ++c) sum += d[c * (RS + 1)];
            __hip_atomic_store(out + lag, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (!pl.fuse_dh) return;       // a second launch adds the partials

    const int64_t np = dm.bs * pl.nseg;
    if (!dh_arrive_last(pl, cb, (unsigned int)np)) return;
    constexpr int CB = 16 * NW;
    const int gpc = CB / dm.dg, bpg = dm.dg / 16;      // filter groups per channel block, 16-channel blocks per group
    const int row = dm.fw ? dm.lc : dm.hl;              // taps per group in the output
    // a thread takes outputs idx and idx + NT of the block's gpc * row together (one memory latency for both)
    for (int idx0 = tid; idx0 < gpc * row; idx0 += 2 * NT) {
        int gl[2], k[2];
        bool live[2], tap[2];
        const float *src[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int idx = idx0 + e * NT;
            gl[e] = 0;
            while (gl[e] + 1 < gpc && idx >= (gl[e] + 1) * row) ++gl[e];
            k[e] = idx - gl[e] * row;
            live[e] = idx < gpc * row && (int64_t)cb * gpc + gl[e] < dm.g;
            tap[e] = live[e] && k[e] < dm.hl;             // else: the parameter's taps beyond the filter in use
            // partial (p, kk) lies at ((p * ncb + cb) * NW + gl * bpg + kk) * 128 + lag
            src[e] = ws + ((int64_t)cb * NW + (tap[e] ? gl[e] * bpg : 0)) * 128 + (tap[e] ? dm.hl - 1 - k[e] : 0);
        }
        float sum[2] = {0.f, 0.f};
        if (bpg == 1) {
            dh_sum_partials2(src[0], src[1], (int64_t)pl.ncb * NW * 128, np, sum[0], sum[1]);
        } else {                                          // p-major, as the second launch adds them
            for (int64_t p = 0; p < np; ++p)
                for (int kk = 0; kk < bpg; ++kk)
#pragma unroll
                    for (int e = 0; e < 2; ++e)
                        sum[e] += __hip_atomic_load(src[e] + (p * pl.ncb * NW + kk) * 128, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int64_t grp = (int64_t)cb * gpc + gl[e];
            if (tap[e]) store_dh<T>(dh, dm, grp, k[e], sum[e]);
            else if (live[e]) ((float *)dh)[grp * row + k[e]] = 0.f;
        }
    }
}

// ---- backward kernels with product waves and row waves (gcg_mfma.hip, gcg_mfma_il.hip) ---------------------------
// LDS of such a workgroup: five-slice filters, four channel blocks of 16, 512 threads.  Every tile of a step
// but g2 exists twice (even and odd steps); g2 is kept in a ring of NK+1 steps, read by the product waves (the
// newest step) and by the filter-gradient products (NK steps) while the row waves write the one after.
template <typename T> struct DuoGeo {
    typedef MT<T> M;
    typedef Geo<T, 4> G;
    static constexpr int NK = 5, NW = 4, ND = 2 * NK - 1, RSLOTS = NK + 1;
    static constexpr int UROW = G::UROW, YROW = G::YROW;
    static constexpr int USZ = STEP * UROW, YSZ = STEP * YROW, RING_ROWS = STEP * RSLOTS;
    static constexpr int OFF_U = 0;                         // u of a step: even steps, odd steps
    static constexpr int OFF_R = OFF_U + 2 * USZ;           // g2 ring of NK+1 steps: slot (step - s_lo) % (NK+1)
    static constexpr int OFF_Y = OFF_R + RSLOTS * USZ;      // y2 tiles, fp32
    static constexpr int OFF_D = OFF_Y + 2 * YSZ;           // du tiles, fp32
    static constexpr int OFF_H = OFF_D + 2 * YSZ;           // filter tables (dead after the barrier that follows the Toeplitz tiles)
    static constexpr int H_BYTES = NW * HTAB * (int)sizeof(typename M::hraw_t);
    static constexpr int LDS_TAIL = NW * (16 * ND + 16) * 17 * 4;   // P tiles at the end (dh_finish)
};

// The product waves' whole run: Toeplitz operands from the filter, the operand rings of the lead-in, then per step
// the operands of step s from the tiles of its parity, the y2 / du products and their tiles.  Barriers: (A) taps in
// LDS, (A2) Toeplitz tiles built, NK-1 pairs (B_i), (C_i) for the lead-in tiles, (D) step s_lo prepared, then one per
// step; the row waves make the same calls.
template <typename T>
__device__ __forceinline__ void duo_product_waves(unsigned char *smem, const T *__restrict__ h, const Dims &dm,
                                                  const MfmaPlan &pl, int cb, int w, int l, bool wave_valid, int64_t s_lo,
                                                  int64_t s_hi)
{
    typedef DuoGeo<T> D;
    typedef typename D::M M;
    typedef typename M::op_t op_t;
    typedef typename M::hraw_t hraw_t;
    constexpr int NK = D::NK, NW = D::NW, UROW = D::UROW, YROW = D::YROW, USZ = D::USZ, YSZ = D::YSZ;
    const int j = l & 15, q = l >> 4;
    hraw_t *htab = (hraw_t *)(smem + D::OFF_H);
    hraw_t hv[HTAB / 64];
    load_taps<T>(dm, h, wave_valid ? fdiv((uint32_t)(cb * NW + w), pl.q_dg16) : 0, l, hv);
    op_t Au[NK], Ag[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        Au[i] = M::zero_op();
        Ag[i] = M::zero_op();
    }
    const int y_wr = j * YROW + (16 * w + 4 * q) * 4;
    const int d_wr = (15 - j) * YROW + (16 * w + 4 * q) * 4;      // columns come out reversed
    store_taps(htab + w * HTAB, l, hv);
    __syncthreads();                                              // (A)
    typename M::wop_t W0[NK], W1[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = M::toeplitz(htab + w * HTAB, 32 * i, j, q);
        W1[i] = M::toeplitz(htab + w * HTAB, 32 * i + 16, j, q);
    }
    __syncthreads();                                              // (A2)
#pragma unroll
    for (int i = 1; i < NK; ++i) {
        __syncthreads();                                          // (B_i) lead-in tiles written
        Au[NK - i] = M::load_operand(smem + D::OFF_U, UROW, w, j, q, false);
        Ag[NK - 1 - i] = M::load_operand(smem + D::OFF_R + (NK - 1 - i) * USZ, UROW, w, j, q, true);
        __syncthreads();                                          // (C_i) and read
    }
    __syncthreads();                                              // (D) step s_lo prepared
    int64_t s = s_lo;
    int gnew = NK - 1;                    // ring slot of step s+NK-1, the newest g2 (the ring's period is not the operand rings')
    auto product_step = [&](int pu) __attribute__((always_inline)) {
        const int ph = pu % NK, par = pu & 1;
        const int slot_new = (ph + NK - 1) % NK;
        Au[ph] = M::load_operand(smem + D::OFF_U + par * USZ, UROW, w, j, q, false);
        Ag[slot_new] = M::load_operand(smem + D::OFF_R + gnew * USZ, UROW, w, j, q, true);
        gnew = (gnew + 1 == D::RSLOTS) ? 0 : gnew + 1;
        f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
        f32x4 dac0 = {0.f, 0.f, 0.f, 0.f}, dac1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            acc0 = M::mfma(Au[(ph - i + NK) % NK], W0[i], acc0);
            acc1 = M::mfma(Au[(ph - i + NK) % NK], W1[i], acc1);
            dac0 = M::mfma(Ag[(ph + i) % NK], W1[i], dac0);   // output rows 0..15
            dac1 = M::mfma(Ag[(ph + i) % NK], W0[i], dac1);   // output rows 16..31
        }
        unsigned char *const y_cur = smem + D::OFF_Y + par * YSZ, *const d_cur = smem + D::OFF_D + par * YSZ;
        *(f32x4 *)(y_cur + y_wr) = acc0;
        *(f32x4 *)(y_cur + y_wr + 16 * YROW) = acc1;
        *(f32x4 *)(d_cur + d_wr) = dac0;
        *(f32x4 *)(d_cur + d_wr + 16 * YROW) = dac1;
        __syncthreads();
        ++s;
    };
    while (s < s_hi) {
#pragma unroll
        for (int pu = 0; pu < 2 * NK; ++pu)
            if (s < s_hi) product_step(pu);
    }
}

// The row waves' filter-gradient products of the step in ring phase pu (step - s_lo modulo NK+1): u of the step
// against the 2 NK - 1 windows of 32 rows of g2 that start 16 rows apart at the step's first row; natural-layout
// operands (rows j and 16+j of a window), wave w's 16 channels.
template <typename T>
__device__ __forceinline__ void duo_filter_gradient(f32x4 (&P)[DuoGeo<T>::ND], const unsigned char *u_cur,
                                                    const unsigned char *ring, int pu, int w, int l)
{
    typedef DuoGeo<T> D;
    typedef typename D::M M;
    typedef typename M::op_t op_t;
    constexpr int UROW = D::UROW;
    const int j = l & 15, q = l >> 4;
    const op_t un = M::load_natural(u_cur + j * UROW, u_cur + (16 + j) * UROW, UROW, w, q);
#pragma unroll
    for (int dl = 0; dl < D::ND; ++dl) {
        int row0 = STEP * pu + 16 * dl + j;              // ring rows of the window's two halves
        int row1 = row0 + 16;
        row0 = (row0 >= D::RING_ROWS) ? row0 - D::RING_ROWS : row0;
        row1 = (row1 >= D::RING_ROWS) ? row1 - D::RING_ROWS : row1;
        const op_t gn = M::load_natural(ring + row0 * UROW, ring + row1 * UROW, UROW, w, q);
        P[dl] = M::mfma_aa(gn, un, P[dl]);
    }
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

// tuning overrides from the environment (tuning builds only, gcg_common.h): unset or empty -> dflt; any integer,
// 0 included, is taken
int env_int(const char *name, int dflt)
{
    const char *v = tuning_env(name);
    if (!v || !*v) return dflt;
    char *end = nullptr;
    const long n = strtol(v, &end, 10);
    return (end == v) ? dflt : (int)n;
}

// Waves per workgroup: wider workgroups read wider rows (16*NW channels, 32*NW bytes), which
// the memory system rewards; narrow tensors fall back to what their width fills.
// fp32 doubles the register state per wave (operand tiles hold 8 floats), which caps the
// forward at 8 waves and the backward at 4.
int choose_nw(const Dims &dm, bool fp32)
{
    static const int forced = env_int("GCG_MFMA_NW", 0);   // tuning override: 4, 8 or 16
    if (forced == 4 || forced == 8 || (forced == 16 && !fp32)) return forced;
    if (dm.d >= 256 && !fp32) {
        // A tensor so small that 16-wave workgroups, one per CU, would get runs of fewer than 16 steps is better
        // served by twice as many 8-wave workgroups (two per CU): (1, 8192, 1024) 16.9 against 22.2 us,
        // (1, 8192, 2048) 28.6 against 34.8, (1, 4096, 4096) 28.9 against 31.9; from runs of 16 steps on the wide
        // workgroups win again ((4, 8192, 1024) 50.4 against 52.3, (1, 8192, 4096) 51.2 against 52.7).
        const int64_t col_steps = dm.bs * ((dm.d + 255) / 256) * ((dm.L + STEP - 1) / STEP);
        return col_steps < 16 * (int64_t)cu_count() ? 8 : 16;
    }
    if (dm.d >= 128) return 8;
    return 4;
}

// elem_bytes: size of one element; segments are kept short enough for the widest window (an
// interleaved tensor, 3 * d elements per row) to stay below WIN_MAX_BYTES.
MfmaPlan plan(const Dims &dm, int nw, int min_steps, int waves_per_cu, int elem_bytes)
{
    MfmaPlan p;
    const int cb = 16 * nw;
    p.nw = nw;
    p.ncb = (int)((dm.d + cb - 1) / cb);
    p.nsteps = (dm.L + STEP - 1) / STEP;
    const int wg_per_cu = waves_per_cu / nw > 0 ? waves_per_cu / nw : 1;
    // Segments per (batch row, channel block): the count that needs the fewest step times.  With
    // `slots` workgroups running at once the launch takes ceil(workgroups / slots) rounds of a run's
    // steps plus its lead-in; e.g. 192 columns on 256 slots are better cut in 4 (3 rounds of 68
    // steps) than in 2 (2 rounds of 132), and 128 columns in 2 (one round of 132).
    const int64_t cols = dm.bs * p.ncb, slots = (int64_t)cu_count() * wg_per_cu;
    static const int min_forced = env_int("GCG_MFMA_MIN_STEPS", 0);         // tuning override: shortest run considered
    if (min_forced > 0) min_steps = min_forced;
    int64_t max_seg = p.nsteps / min_steps;
    if (max_seg < 1) max_seg = 1;
    const int64_t lead = (dm.hl + 30) / 32 < 4 ? (dm.hl + 30) / 32 : 4;     // NK - 1 steps replayed by a later segment
    int64_t cap = WIN_MAX_BYTES / (STEP * 3 * dm.d * elem_bytes) - 2 * 5;   // a run, with NK-1 steps either side, fits a window
    if (cap < 1) cap = 1;
    const int64_t n_min = (p.nsteps + cap - 1) / cap;                       // fewest segments the windows allow
    int64_t want = n_min, best = -1;
    for (int64_t n = n_min; (n <= max_seg || n == n_min) && n <= n_min + 4 * (slots / cols + 1); ++n) {
        const int64_t rounds = (cols * n + slots - 1) / slots;
        const int64_t cost = rounds * ((p.nsteps + n - 1) / n + (n > 1 ? lead : 0));
        if (best < 0 || cost < best) { best = cost; want = n; }
    }
    static const int forced = env_int("GCG_MFMA_STEPS_PER_SEG", 0);        // tuning override
    int64_t sps = (p.nsteps + want - 1) / want;
    if (forced > 0) sps = forced;
    if (sps > cap) sps = cap;
    p.steps_per_seg = (int)sps;
    p.nseg = (int)((p.nsteps + sps - 1) / sps);
    p.nwg = dm.bs * p.nseg * p.ncb;
    p.xcd = 1;
    p.fuse_dh = 0;
    p.slot = 0;
    p.q_ncb = make_fastdiv((uint32_t)p.ncb);
    p.q_nseg = make_fastdiv((uint32_t)p.nseg);
    p.q_dg16 = make_fastdiv((uint32_t)(dm.dg >= 16 ? dm.dg / 16 : 1));
    return p;
}

// input steps an output step reaches back over: lags up to hl-1 from rows 0..31 of the step
int nk_for(int hl) { const int n = (hl + 30) / 32 + 1; return n > 5 ? 5 : n; }

// The backward holds about twice the forward's register state per wave (two waves per SIMD at
// most), and one wave per SIMD measured best: 4-wave workgroups, one per CU, with runs twice as
// long (half the lead-in) take 176 us where 8-wave workgroups took 201 at (2, 8192, 4096) and 660
// against 749 at (1, 32768, 8192); on interleaved operands 173 against 196 and 641 against 754.
// Two 4-wave workgroups sharing a CU are slower than either (237 us), so the kernels' LDS
// request keeps a CU to one.  The 8-wave form is no longer instantiated.
constexpr int BWD_NW = 4;

// one workgroup per CU in either geometry (fp32: one wave per SIMD by its registers alone)
MfmaPlan plan_bwd_nw(const Dims &dm, int nw, int elem_bytes);
MfmaPlan plan_bwd(const Dims &dm, bool split, int elem_bytes)
{
    (void)split;
    return plan_bwd_nw(dm, BWD_NW, elem_bytes);
}
// The backward that recomputes the featurizer spends twice the vector instructions per row: with two waves per
// SIMD they hide behind each other (8-wave workgroups: 220 us at the 7B shape against 263 with 4 waves).
int choose_nw_bwd_feat(bool split)
{
    static const int forced = env_int("GCG_MFMA_FEAT_BWD_NW", 0);   // tuning override: 4 or 8
    if (forced == 4 || (forced == 8 && !split)) return forced;
    return split ? 4 : 8;
}
MfmaPlan plan_bwd_nw(const Dims &dm, int nw, int elem_bytes)
{
    MfmaPlan p = plan(dm, nw, 16, nw, elem_bytes);
    // the kernel adds the partials itself when a filter group lies within one channel block (and the launch gets a
    // ticket set, dh_slot_for_stream); otherwise a second launch does
    p.fuse_dh = (16 * nw) % dm.dg == 0 && p.ncb <= DH_UNITS;
    return p;
}

} // namespace
} // namespace gcg
