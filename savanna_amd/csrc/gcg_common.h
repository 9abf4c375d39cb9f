// Shared device helpers for the gated chunked causal convolution kernels (gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/gcg.h"

namespace gcg {

// ---- element types -------------------------------------------------------------------
// bf16 and f16 travel as raw 16-bit patterns; arithmetic is always fp32.
struct bf16_t { uint16_t v; };
struct f16_t  { uint16_t v; };

__device__ __forceinline__ float bf16_bits_to_float(uint32_t lo16)
{
    return __uint_as_float(lo16 << 16);
}

// fp32 -> bf16, round to nearest even; gfx950 has a packed hardware conversion
// (v_cvt_pk_bf16_f32) that the compiler selects for these casts.
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f)
{
    const __bf16 b = (__bf16)f;
    uint16_t u;
    __builtin_memcpy(&u, &b, 2);
    return u;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 r;
    r[0] = (__bf16)lo;
    r[1] = (__bf16)hi;
    uint32_t u;
    __builtin_memcpy(&u, &r, 4);
    return u;
}

__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi)
{
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 r = {(_Float16)lo, (_Float16)hi};
    uint32_t u;
    __builtin_memcpy(&u, &r, 4);
    return u;
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
    static __device__ __forceinline__ float load(const bf16_t *p) { return bf16_bits_to_float(p->v); }
    static __device__ __forceinline__ void store(bf16_t *p, float v) { p->v = (uint16_t)float_to_bf16_bits(v); }
};
template <> struct Elem<f16_t> {
    static __device__ __forceinline__ float load(const f16_t *p)
    {
        _Float16 hv;
        __builtin_memcpy(&hv, &p->v, 2);
        return (float)hv;
    }
    static __device__ __forceinline__ void store(f16_t *p, float v)
    {
        _Float16 hv = (_Float16)v;
        __builtin_memcpy(&p->v, &hv, 2);
    }
};

// ---- launch descriptors shared by host dispatch and kernels --------------------------
struct Dims {
    int64_t bs, L;
    int32_t g, dg, hl;
    int64_t d; // g * dg
    // Element stride of the x, B, C operands and of dx, dB, dC.  1: three separate contiguous
    // tensors.  3: one interleaved tensor (bs, L, g, dg, 3) with [..., 0] = C, [..., 1] = B,
    // [..., 2] = x; the launchers then receive C = base, B = base + 1, x = base + 2 elements
    // (and dC, dB, dx likewise).  y, y2, bx and dy are always plain.
    int32_t es;
};

constexpr int kWave = 64;


// interleaved operands: feat / dfeat are (bs, L, g, dg, 3) with [..., 0] = C, [..., 1] = B, [..., 2] = x
int mfma_il_fwd_launch(int dtype, const void *feat, const void *h, void *y, const Dims &dm, hipStream_t st);
int mfma_il_bwd_launch(int dtype, const void *dy, const void *feat, const void *h, void *dfeat, void *dh,
                       void *ws, const Dims &dm, hipStream_t st);

} // namespace gcg

// Host-side launchers, one translation unit per kernel family.  Each returns a
// hipError_t as int; none of them allocates or synchronises.
namespace gcg {

int direct_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h,
                      void *y, void *y2, void *bx, const Dims &dm, hipStream_t st);
size_t direct_bwd_workspace(const Dims &dm);
int direct_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C,
                      const void *h, void *dx, void *dB, void *dC, void *dh, void *ws,
                      const Dims &dm, hipStream_t st);

bool window_supported(const Dims &dm);
int window_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h,
                      void *y, void *y2, void *bx, const Dims &dm, hipStream_t st);
size_t window_bwd_workspace(const Dims &dm);
int window_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C,
                      const void *h, void *dx, void *dB, void *dC, void *dh, void *ws,
                      const Dims &dm, hipStream_t st);

bool mfma_supported(int dtype, const Dims &dm);
bool mfma_bwd_available();
int mfma_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h,
                    void *y, void *y2, void *bx, const Dims &dm, hipStream_t st);
size_t mfma_bwd_workspace(int dtype, const Dims &dm);
int mfma_bwd_launch(int dtype, const void *dy, const void *x, const void *B, const void *C,
                    const void *h, void *dx, void *dB, void *dC, void *dh, void *ws,
                    const Dims &dm, hipStream_t st);


// interleaved operands: feat / dfeat are (bs, L, g, dg, 3) with [..., 0] = C, [..., 1] = B, [..., 2] = x
int mfma_il_fwd_launch(int dtype, const void *feat, const void *h, void *y, const Dims &dm, hipStream_t st);
int mfma_il_bwd_launch(int dtype, const void *dy, const void *feat, const void *h, void *dfeat, void *dh,
                       void *ws, const Dims &dm, hipStream_t st);

// interleaved operands: feat / dfeat are (bs, L, g, dg, 3) with [..., 0] = C, [..., 1] = B, [..., 2] = x
int mfma_il_fwd_launch(int dtype, const void *feat, const void *h, void *y, const Dims &dm, hipStream_t st);
int mfma_il_bwd_launch(int dtype, const void *dy, const void *feat, const void *h, void *dfeat, void *dh,
                       void *ws, const Dims &dm, hipStream_t st);

} // namespace gcg
