// Explicit decayed filter of Hyena-MR, generated for the convolution kernels in one launch:
//   h[g, 0, k] = T(w[g, k] * decay[g, k])            for k < hl       (parameters in fp32, (g, L_cache))
// and its backward in one launch:
//   dw[g, k]   = float(dh[g, 0, k]) * decay[g, k]    for k < hl,  0 for hl <= k < L_cache.
// This is the slice, product and cast (and, backwards, cast, product and zero padding) that the
// reference spreads over several elementwise launches around the operator.
#include "gcg_common.h"

namespace gcg {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void filter_fwd_kernel(const float *__restrict__ w, const float *__restrict__ decay,
                                                         T *__restrict__ h, int g, int l_cache, int hl)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)g * hl) return;
    const int64_t grp = i / hl, k = i % hl;
    Elem<T>::store(h + i, w[grp * l_cache + k] * decay[grp * l_cache + k]);
}

template <typename T>
__global__ __launch_bounds__(256) void filter_bwd_kernel(const T *__restrict__ dh, const float *__restrict__ decay,
                                                         float *__restrict__ dw, int g, int l_cache, int hl)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)g * l_cache) return;
    const int64_t grp = i / l_cache, k = i % l_cache;
    dw[i] = k < hl ? Elem<T>::load(dh + grp * hl + k) * decay[i] : 0.f;
}

} // namespace

int filter_fwd_launch(int dtype, const float *w, const float *decay, void *h, int g, int l_cache, int hl,
                      hipStream_t st)
{
    int e = 0;
    const unsigned nb = (unsigned)(((int64_t)g * hl + 255) / 256);
    switch (dtype) {
    case GCG_F32:  e = launch_plain(filter_fwd_kernel<float>, dim3(nb), dim3(256), st, w, decay, (float *)h, g, l_cache, hl); break;
    case GCG_BF16: e = launch_plain(filter_fwd_kernel<bf16_t>, dim3(nb), dim3(256), st, w, decay, (bf16_t *)h, g, l_cache, hl); break;
    case GCG_F16:  e = launch_plain(filter_fwd_kernel<f16_t>, dim3(nb), dim3(256), st, w, decay, (f16_t *)h, g, l_cache, hl); break;
    default: return (int)hipErrorInvalidValue;
    }
    return e;
}

int filter_bwd_launch(int dtype, const void *dh, const float *decay, float *dw, int g, int l_cache, int hl,
                      hipStream_t st)
{
    int e = 0;
    const unsigned nb = (unsigned)(((int64_t)g * l_cache + 255) / 256);
    switch (dtype) {
    case GCG_F32:  e = launch_plain(filter_bwd_kernel<float>, dim3(nb), dim3(256), st, (const float *)dh, decay, dw, g, l_cache, hl); break;
    case GCG_BF16: e = launch_plain(filter_bwd_kernel<bf16_t>, dim3(nb), dim3(256), st, (const bf16_t *)dh, decay, dw, g, l_cache, hl); break;
    case GCG_F16:  e = launch_plain(filter_bwd_kernel<f16_t>, dim3(nb), dim3(256), st, (const f16_t *)dh, decay, dw, g, l_cache, hl); break;
    default: return (int)hipErrorInvalidValue;
    }
    return e;
}

} // namespace gcg
