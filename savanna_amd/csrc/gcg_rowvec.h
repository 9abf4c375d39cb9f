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

} // namespace
} // namespace gcg
