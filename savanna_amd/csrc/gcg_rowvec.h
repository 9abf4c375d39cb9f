// Row vectors of the register-window kernels: a lane's few adjacent channels of one time row
// as raw 32-bit words, and their conversion to and from fp32.
#pragma once
#include "gcg_common.h"

namespace gcg {
namespace {

// A lane's row vector: VV channels as raw 32-bit words (fp32: one channel per word;
// bf16 / f16: two).  VV = 4 everywhere, or 8 for the 16-bit types (16-byte accesses).
template <typename T, int VV> struct Vec;
template <> struct Vec<float, 4> { typedef u32x4 raw; static constexpr int W = 4; };
template <> struct Vec<bf16_t, 4> { typedef u32x2 raw; static constexpr int W = 2; };
template <> struct Vec<f16_t, 4> { typedef u32x2 raw; static constexpr int W = 2; };
template <> struct Vec<bf16_t, 8> { typedef u32x4 raw; static constexpr int W = 4; };
template <> struct Vec<f16_t, 8> { typedef u32x4 raw; static constexpr int W = 4; };
// one 32-bit word per row: the lane width of the interleaved kernels, whose row piece
// (C, B, x per channel) is then 12 contiguous bytes
template <> struct Vec<float, 1> { typedef u32x1 raw; static constexpr int W = 1; };
template <> struct Vec<bf16_t, 2> { typedef u32x1 raw; static constexpr int W = 1; };
template <> struct Vec<f16_t, 2> { typedef u32x1 raw; static constexpr int W = 1; };
// 16-bit tensors with an fp32 filter: the row vectors of the plain 16-bit types
template <int VV> struct Vec<bf16w_t, VV> : Vec<bf16_t, VV> {};
template <int VV> struct Vec<f16w_t, VV> : Vec<f16_t, VV> {};
// the three words of an interleaved row piece in one 12-byte access
__device__ __forceinline__ void load_piece(win_t w, uint32_t off, u32x1 (&p)[3])
{
    const u32x3 v = win_load<u32x3>(w, off);
    p[0][0] = v[0]; p[1][0] = v[1]; p[2][0] = v[2];
}
__device__ __forceinline__ void store_piece(win_t w, uint32_t off, const u32x1 (&p)[3])
{
    win_store(w, off, u32x3{p[0][0], p[1][0], p[2][0]});
}
// (with the choice of cache policy; the interleaved kernels' lanes are one word wide)
template <bool KEEP> __device__ __forceinline__ void store_piece_as(win_t w, uint32_t off, const u32x1 (&p)[3])
{
    win_store_as<KEEP>(w, off, u32x3{p[0][0], p[1][0], p[2][0]});
}
template <typename R> __device__ __forceinline__ void load_piece(win_t w, uint32_t off, R (&p)[3])
{
    constexpr int NB = sizeof(R);
    p[0] = win_load<R>(w, off); p[1] = win_load<R>(w, off + NB); p[2] = win_load<R>(w, off + 2 * NB);
}
template <typename R> __device__ __forceinline__ void store_piece(win_t w, uint32_t off, const R (&p)[3])
{
    constexpr int NB = sizeof(R);
    win_store(w, off, p[0]); win_store(w, off + NB, p[1]); win_store(w, off + 2 * NB, p[2]);
}
template <typename T> struct Word;   // conversions of one 32-bit word
template <> struct Word<float> {
    static constexpr int N = 1;
    static __device__ __forceinline__ void unpack(uint32_t w, float *f) { f[0] = __uint_as_float(w); }
    static __device__ __forceinline__ uint32_t pack(const float *f) { return __float_as_uint(f[0]); }
};
template <> struct Word<bf16_t> {
    static constexpr int N = 2;
    static __device__ __forceinline__ void unpack(uint32_t w, float *f)
    {
        f[0] = __uint_as_float(w << 16);
        f[1] = __uint_as_float(w & 0xffff0000u);
    }
    static __device__ __forceinline__ uint32_t pack(const float *f) { return pack_bf16x2(f[0], f[1]); }
};
template <> struct Word<f16_t> {
    static constexpr int N = 2;
    static __device__ __forceinline__ void unpack(uint32_t w, float *f)
    {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 a;
        __builtin_memcpy(&a, &w, 4);
        f[0] = (float)a[0];
        f[1] = (float)a[1];
    }
    static __device__ __forceinline__ uint32_t pack(const float *f) { return pack_f16x2(f[0], f[1]); }
};

template <> struct Word<bf16w_t> : Word<bf16_t> {};
template <> struct Word<f16w_t> : Word<f16_t> {};

template <typename T, int VV>
__device__ __forceinline__ void unpackv(const typename Vec<T, VV>::raw &r, float (&f)[VV])
{
#pragma unroll
    for (int i = 0; i < Vec<T, VV>::W; ++i) Word<T>::unpack(r[i], &f[i * Word<T>::N]);
}
template <typename T, int VV>
__device__ __forceinline__ typename Vec<T, VV>::raw packv(const float (&f)[VV])
{
    typename Vec<T, VV>::raw r;
#pragma unroll
    for (int i = 0; i < Vec<T, VV>::W; ++i) r[i] = Word<T>::pack(&f[i * Word<T>::N]);
    return r;
}
template <typename T, int VV> __device__ __forceinline__ typename Vec<T, VV>::raw zero_raw()
{
    typename Vec<T, VV>::raw r;
#pragma unroll
    for (int i = 0; i < Vec<T, VV>::W; ++i) r[i] = 0u;
    return r;
}


// Filter-gradient reduction shared by the register-window kernels.  The walk kernels leave
// partials ws[tap][row][col]: one row per (batch, run), one column per lane (or per channel);
// filter f owns the lpg adjacent columns [f * lpg, (f+1) * lpg).  out[f * ntap + tap] is their
// sum over all rows.  A workgroup takes a tile of whole filters at most 64 columns wide (one
// filter if it is wider) and 4 row slices: its 64-lane rows read contiguous runs of a partial
// row, every thread adds its terms in a fixed order, and the slices and columns of a filter are
// then combined in a fixed order -- the result is bit-reproducible.
struct ColsumJob { const float *ws; void *out; int64_t nrow, ncol; int lpg, nfilt, ntap; };

template <typename T> __device__ __forceinline__ void colsum_reduce_block(const ColsumJob &jb, int bx, int tap)
{
    __shared__ float red[4][64];
    const float *__restrict__ ws = jb.ws;
    T *__restrict__ out = (T *)jb.out;
    const int64_t nrow = jb.nrow, ncol = jb.ncol;
    const int lpg = jb.lpg, nfilt = jb.nfilt, ntap = jb.ntap;
    const int fpb = lpg >= 64 ? 1 : 64 / lpg;                 // filters per workgroup
    const int64_t f0 = (int64_t)bx * fpb;
    const int nf = (int)((f0 + fpb <= nfilt) ? fpb : nfilt - f0);
    const int width = nf * lpg;                                // columns of the tile
    const int c = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const float *src = ws + (size_t)tap * nrow * ncol + f0 * lpg;
    float s = 0.f;
    for (int cc = c; cc < width; cc += 64) {                   // more than one column only for one wide filter
        int64_t r = slice;
        for (; r + 28 < nrow; r += 32) {                       // eight loads in flight, added in row order
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = src[(r + 4 * i) * ncol + cc];
#pragma unroll
            for (int i = 0; i < 8; ++i) s += v[i];
        }
        for (; r < nrow; r += 4) s += src[r * ncol + cc];
    }
    red[slice][c] = s;
    __syncthreads();
    if ((int)threadIdx.x < nf) {
        const int lo = lpg >= 64 ? 0 : (int)threadIdx.x * lpg, n = lpg >= 64 ? 64 : lpg;
        float t = 0.f;
        for (int q = 0; q < n; ++q)
            for (int sl = 0; sl < 4; ++sl) t += red[sl][lo + q];
        Elem<T>::store(out + (f0 + threadIdx.x) * ntap + tap, t);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void colsum_reduce_kernel(ColsumJob jb)
{
    colsum_reduce_block<T>(jb, blockIdx.x, blockIdx.y);
}

// two reductions in one launch (the filter gradients of two filters from one walk): the first
// nb0 workgroups of a grid row belong to the first; grid rows beyond a job's tap count idle
// (T0, T1: element types of the two results)
template <typename T0, typename T1>
__global__ __launch_bounds__(256) void colsum_reduce2_kernel(ColsumJob j0, ColsumJob j1, int nb0)
{
    const bool second = (int)blockIdx.x >= nb0;
    if ((int)blockIdx.y >= (second ? j1.ntap : j0.ntap)) return;
    if (second) colsum_reduce_block<T1>(j1, (int)blockIdx.x - nb0, blockIdx.y);
    else colsum_reduce_block<T0>(j0, (int)blockIdx.x, blockIdx.y);
}

inline unsigned colsum_blocks(int lpg, int nfilt)
{
    const int fpb = lpg >= 64 ? 1 : 64 / lpg;
    return (unsigned)((nfilt + fpb - 1) / fpb);
}

template <typename T>
inline int launch_colsum_reduce(const float *ws, T *out, int64_t nrow, int64_t ncol, int lpg, int nfilt, int ntap,
                                hipStream_t st)
{
    int e = 0;
    const ColsumJob jb{ws, out, nrow, ncol, lpg, nfilt, ntap};
    e = launch_plain(colsum_reduce_kernel<T>, dim3(colsum_blocks(lpg, nfilt), (unsigned)ntap), dim3(256), st, jb);
    return e;
}

template <typename T0, typename T1 = T0>
inline int launch_colsum_reduce2(const ColsumJob &j0, const ColsumJob &j1, hipStream_t st)
{
    int e = 0;
    const unsigned nb0 = colsum_blocks(j0.lpg, j0.nfilt), nb1 = colsum_blocks(j1.lpg, j1.nfilt);
    const unsigned ny = (unsigned)(j0.ntap > j1.ntap ? j0.ntap : j1.ntap);
    e = launch_plain((colsum_reduce2_kernel<T0, T1>), dim3(nb0 + nb1, ny), dim3(256), st, j0, j1, (int)nb0);
    return e;
}

} // namespace
} // namespace gcg
