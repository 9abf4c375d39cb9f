// Shared device helpers for the gated chunked causal convolution kernels (gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <tuple>
#include <utility>

#include "../../include/gcg.h"

namespace gcg {

// ---- element types -------------------------------------------------------------------
// bf16 and f16 travel as raw 16-bit patterns; arithmetic is always fp32.
struct bf16_t { uint16_t v; };
struct f16_t  { uint16_t v; };
// GCG_BF16_F32 / GCG_F16_F32: 16-bit tensors with an fp32 filter, fp32 filter gradient and nothing rounded to
// 16 bits between load and store -- the operator "run in fp32" on a 16-bit model without the casts around it.
struct bf16w_t { uint16_t v; };
struct f16w_t  { uint16_t v; };
// element type of h and dh for tensors of type T
template <typename T> struct Filt { typedef T type; };
template <> struct Filt<bf16w_t> { typedef float type; };
template <> struct Filt<f16w_t> { typedef float type; };

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
template <> struct Elem<bf16w_t> {
    static __device__ __forceinline__ float load(const bf16w_t *p) { return bf16_bits_to_float(p->v); }
    static __device__ __forceinline__ void store(bf16w_t *p, float v) { p->v = (uint16_t)float_to_bf16_bits(v); }
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

template <> struct Elem<f16w_t> {
    static __device__ __forceinline__ float load(const f16w_t *p) { return Elem<f16_t>::load((const f16_t *)p); }
    static __device__ __forceinline__ void store(f16w_t *p, float v) { Elem<f16_t>::store((f16_t *)p, v); }
};

// ---- tensor windows --------------------------------------------------------------------
// A kernel addresses each tensor through a buffer descriptor that covers the rows it touches:
// byte offsets are 32-bit, a load outside the window returns zero and a store outside it is
// dropped.  Rows before the sequence start (negative offsets, which wrap past the window) and
// after its end thus need no test, and a lane whose channels lie beyond the tensor adds WIN_OFF
// to its offsets.  With no branch around any load or store the instruction stream is
// straight-line, and the compiler's wait-count insertion can tell exactly how many accesses are
// in flight; across a branch it cannot, and it then waits for every outstanding access.
// Every element is touched once, so accesses carry the nontemporal hint.
typedef uint32_t u32x1 __attribute__((ext_vector_type(1)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t win_t;
constexpr uint32_t WIN_OFF = 0x80000000u;           // offsets at or above this are outside every window
constexpr int64_t WIN_MAX_BYTES = (1ll << 31) - (1ll << 27);
#ifndef GCG_NT
#define GCG_NT 3                                    // bit 0: loads, bit 1: stores
#endif
#if defined(GCG_LD_AUX) && defined(GCG_ST_AUX)      // tuning builds: the cache-policy bits spelled out (1 sc0, 2 nt, 16 sc1)
constexpr int WIN_NT = GCG_LD_AUX, WIN_NT_ST = GCG_ST_AUX;
#else
constexpr int WIN_NT = (GCG_NT & 1) ? 2 : 0, WIN_NT_ST = (GCG_NT & 2) ? 2 : 0;   // cache policy "nt"
#endif

__device__ __forceinline__ win_t make_window(const void *base, int64_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(bytes > 0 ? bytes : 0), 0x00020000);
}
template <typename R> __device__ __forceinline__ R win_load(win_t w, uint32_t off);
template <> __device__ __forceinline__ uint32_t win_load<uint32_t>(win_t w, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b32(w, (int)off, 0, WIN_NT);
}
// a 16-bit element (zero-extended)
__device__ __forceinline__ uint32_t win_load_u16(win_t w, uint32_t off)
{
    return (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(w, (int)off, 0, 0);
}
__device__ __forceinline__ float win_load_f32_cached(win_t w, uint32_t off)
{
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(w, (int)off, 0, 0));
}
template <> __device__ __forceinline__ u32x1 win_load<u32x1>(win_t w, uint32_t off)
{
    u32x1 r;
    r[0] = __builtin_amdgcn_raw_buffer_load_b32(w, (int)off, 0, WIN_NT);
    return r;
}
template <> __device__ __forceinline__ u32x2 win_load<u32x2>(win_t w, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b64(w, (int)off, 0, WIN_NT);
}
template <> __device__ __forceinline__ u32x3 win_load<u32x3>(win_t w, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b96(w, (int)off, 0, WIN_NT);
}
template <> __device__ __forceinline__ u32x4 win_load<u32x4>(win_t w, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b128(w, (int)off, 0, WIN_NT);
}
__device__ __forceinline__ void win_store(win_t w, uint32_t off, uint32_t v)
{
    __builtin_amdgcn_raw_buffer_store_b32(v, w, (int)off, 0, WIN_NT_ST);
}
__device__ __forceinline__ void win_store(win_t w, uint32_t off, const u32x1 &v)
{
    __builtin_amdgcn_raw_buffer_store_b32(v[0], w, (int)off, 0, WIN_NT_ST);
}
__device__ __forceinline__ void win_store(win_t w, uint32_t off, const u32x2 &v)
{
    __builtin_amdgcn_raw_buffer_store_b64(v, w, (int)off, 0, WIN_NT_ST);
}
__device__ __forceinline__ void win_store(win_t w, uint32_t off, const u32x3 &v)
{
    __builtin_amdgcn_raw_buffer_store_b96(v, w, (int)off, 0, WIN_NT_ST);
}
__device__ __forceinline__ void win_store(win_t w, uint32_t off, const u32x4 &v)
{
    __builtin_amdgcn_raw_buffer_store_b128(v, w, (int)off, 0, WIN_NT_ST);
}
// a 16-byte store with the cache-policy bits spelled out (1 sc0, 2 nt, 16 sc1), for the kernels that measured
// a better one than the default
template <int AUX> __device__ __forceinline__ void win_store_policy(win_t w, uint32_t off, const u32x4 &v)
{
    __builtin_amdgcn_raw_buffer_store_b128(v, w, (int)off, 0, AUX);
}
template <int AUX> __device__ __forceinline__ u32x4 win_load_policy(win_t w, uint32_t off)
{
    return __builtin_amdgcn_raw_buffer_load_b128(w, (int)off, 0, AUX);
}
// The same without the nontemporal hint, for an output the next kernel of a chain reads back at once
// (the featurized tensor, the gradient of the features): stored through the cache it is still
// partly there when that kernel starts.  A kernel timed alone loses a few percent this way, which
// is why it is the caller's choice (GCG_KEEP_OUTPUT).
template <bool KEEP> __device__ __forceinline__ void win_store_as(win_t w, uint32_t off, const u32x2 &v)
{
    __builtin_amdgcn_raw_buffer_store_b64(v, w, (int)off, 0, KEEP ? 0 : WIN_NT_ST);
}
template <bool KEEP> __device__ __forceinline__ void win_store_as(win_t w, uint32_t off, const u32x3 &v)
{
    __builtin_amdgcn_raw_buffer_store_b96(v, w, (int)off, 0, KEEP ? 0 : WIN_NT_ST);
}
template <bool KEEP> __device__ __forceinline__ void win_store_as(win_t w, uint32_t off, const u32x4 &v)
{
    __builtin_amdgcn_raw_buffer_store_b128(v, w, (int)off, 0, KEEP ? 0 : WIN_NT_ST);
}

#ifndef GCG_XCD_SWIZZLE
#define GCG_XCD_SWIZZLE 1
#endif
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
// the same on 32-bit indices (launches of fewer than 2^31 workgroups)
__device__ __forceinline__ uint32_t xcd_contiguous_u32(uint32_t id, uint32_t n)
{
#if GCG_XCD_SWIZZLE
    if ((n & 7u) == 0) return (id & 7u) * (n >> 3) + (id >> 3);
#endif
    return id;
}

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
    int32_t keep_out;   // GCG_KEEP_OUTPUT: store the main output through the cache (kernels that have the variant)
    // Decayed explicit filter built inside the matrix-core kernels (the *_decay entry points): when fw is set
    // the filter is h[g, k] = F(fw[g * lc + k] * fdecay[g * lc + k]) for k < hl (F = element type of the filter),
    // the kernels' h argument is unused, and their dh argument is the (g, lc) fp32 gradient of fw.
    const float *fw, *fdecay;
    int32_t lc;
    // Time-major operands (register-window kernels, separate tensors): x, B, C and dx, dB, dC are laid out
    // (L, bs, g, dg) -- the rows of one batch entry lie bs * d elements apart -- while y and dy stay (bs, L, g, dg).
    int32_t tmajor;
    // Planar features (the split without interleaving, block.py:881-884): x, B, C are the thirds of the rows of one
    // (bs, L, 3 * d) tensor -- C = base, B = base + d, x = base + 2 d elements, rows 3 * d elements apart -- and
    // dC, dB, dx the thirds of its gradient; y and dy stay (bs, L, g, dg).  Separate-tensor kernels only (es = 1).
    int32_t planar;
};

constexpr int kWave = 64;

} // namespace gcg

#include <cstdlib>
namespace gcg {
// Tuning overrides from the environment exist in builds with -DGCG_TUNING only (A/B builds of a variant
// against the library); the library as built by the Makefile reads no environment variable.
inline const char *tuning_env(const char *name)
{
#ifdef GCG_TUNING
    return getenv(name);
#else
    (void)name;
    return nullptr;
#endif
}
} // namespace gcg

// Host-side launchers, one translation unit per kernel family.  Each returns a
// hipError_t as int; none of them allocates or synchronises.
namespace gcg {

// gcg_time_next_kernel: a pair of events the caller armed on this thread.  The launcher of an entry
// point's main kernel takes them (once) and has the runtime stamp them at that kernel's own start
// and end, so the elapsed time is the kernel's duration without the launches around it.
struct KernelTimer { hipEvent_t start, stop; };
KernelTimer take_kernel_timer();

// Every launch returns the runtime's own code for that launch (hipLaunchKernel / hipExtLaunchKernel)
// rather than the thread's sticky last error, so an error left behind by other code on the thread is
// neither reported as this library's nor cleared from under its owner.
template <typename... KArgs, size_t... I>
inline int launch_packed(const void *fn, dim3 grid, dim3 block, hipStream_t st, const KernelTimer &t,
                         std::tuple<KArgs...> &vals, std::index_sequence<I...>)
{
    void *ptrs[] = {(void *)&std::get<I>(vals)...};
    if (t.start && t.stop)
        return (int)hipExtLaunchKernel(fn, grid, block, ptrs, 0, st, t.start, t.stop, 0);
    return (int)hipLaunchKernel(fn, grid, block, ptrs, 0, st);
}

// a small kernel beside the main one (reductions, filter generation): never timed
template <typename... KArgs, typename... Args>
inline int launch_plain(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t st, Args... args)
{
    std::tuple<KArgs...> vals{static_cast<KArgs>(args)...};
    return launch_packed((const void *)kernel, grid, block, st, KernelTimer{nullptr, nullptr}, vals,
                         std::index_sequence_for<KArgs...>{});
}

// an entry point's main kernel: carries the caller's event pair when one is armed
template <typename... KArgs, typename... Args>
inline int launch_main(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t st, Args... args)
{
    std::tuple<KArgs...> vals{static_cast<KArgs>(args)...};
    return launch_packed((const void *)kernel, grid, block, st, take_kernel_timer(), vals,
                         std::index_sequence_for<KArgs...>{});
}

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

// the same forward with the featurizer in front: raw is the projection output, wfeat (3 * d, 1, kf)
bool mfma_feat_supported(int dtype, const Dims &dm, int kf);
size_t mfma_feat_bwd_workspace(int dtype, const Dims &dm);
int mfma_il_fwd_feat_launch(int dtype, const void *raw, const void *wfeat, int kf, const void *h, void *y,
                            const Dims &dm, hipStream_t st);
int mfma_il_bwd_feat_launch(int dtype, const void *dy, const void *raw, const void *wfeat, int kf, const void *h,
                            void *dfeat, void *dh, void *ws, const Dims &dm, hipStream_t st);

// the whole backward of featurizer -> Hyena-MR operator in one kernel (no gradient of the features in memory)
bool mixer_mr_fused_supported(int dtype, const Dims &dm, int kf);
size_t mixer_mr_fused_workspace(const Dims &dm, int kf);
int mixer_mr_fused_fwd_launch(int dtype, const void *raw, const void *wfeat, int kf, const void *h, void *y,
                              const Dims &dm, hipStream_t st);
int mixer_mr_fused_bwd_launch(int dtype, const void *dy, const void *raw, const void *wfeat, int kf, const void *h,
                              void *draw, void *dwf, void *dh, void *ws, const Dims &dm, hipStream_t st);

// ungated short causal depthwise convolution (the featurizer), (bs, L, g, dg) channel-fastest
bool dwconv_supported(const Dims &dm);
int dwconv_fwd_launch(int dtype, const void *x, const void *w, void *y, const Dims &dm, hipStream_t st);
size_t dwconv_bwd_workspace(const Dims &dm);
int dwconv_bwd_launch(int dtype, const void *dy, const void *x, const void *w, void *dx, void *dw, void *ws,
                      const Dims &dm, hipStream_t st);

// featurizer and Hyena-SE operator in one pass: raw / draw are (bs, L, g, dg, 3), wf (3 * g * dg, 1, kf)
bool mixer_se_supported(const Dims &dm, int kf);
int mixer_se_fwd_launch(int dtype, const void *raw, const void *wf, const void *h, void *y, const Dims &dm, int kf,
                        hipStream_t st);
size_t mixer_se_bwd_workspace(int dtype, const Dims &dm, int kf);
int mixer_se_bwd_launch(int dtype, const void *dy, const void *raw, const void *wf, const void *h, void *draw,
                        void *dwf, void *dh, void *ws, const Dims &dm, int kf, hipStream_t st);

// explicit decayed filter: h = T(w * decay) cut to hl taps, and its backward
int filter_fwd_launch(int dtype, const float *w, const float *decay, void *h, int g, int l_cache, int hl,
                      hipStream_t st);
int filter_bwd_launch(int dtype, const void *dh, const float *decay, float *dw, int g, int l_cache, int hl,
                      hipStream_t st);

} // namespace gcg
