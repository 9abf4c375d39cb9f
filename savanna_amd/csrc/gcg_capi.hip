// C ABI (include/gcg.h): argument checks, kernel-family selection, launch.
#include "gcg_common.h"

#include <initializer_list>
#include <mutex>

namespace {

thread_local int tls_hip_error = 0;
thread_local gcg::KernelTimer tls_timer = {nullptr, nullptr};

// an armed kernel timer lasts for one launching entry point, however that call ends
struct TimerScope { ~TimerScope() { tls_timer = {nullptr, nullptr}; } };

// gfx950 check, cached per device ordinal.
int check_device()
{
    static std::mutex mu;
    static int ok[64];  // 0 unknown, 1 yes, -1 no
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { tls_hip_error = (int)e; return GCG_ERR_LAUNCH; }
    if (dev < 0 || dev >= 64) return GCG_OK;
    std::lock_guard<std::mutex> lk(mu);
    if (ok[dev] == 0) {
        hipDeviceProp_t p;
        e = hipGetDeviceProperties(&p, dev);
        if (e != hipSuccess) { tls_hip_error = (int)e; return GCG_ERR_LAUNCH; }
        ok[dev] = (__builtin_strncmp(p.gcnArchName, "gfx950", 6) == 0) ? 1 : -1;
    }
    return ok[dev] == 1 ? GCG_OK : GCG_ERR_DEVICE;
}

// mixed_ok: the entry point takes GCG_BF16_F32 / GCG_F16_F32 (the gated operator does, the featurizer does not)
int make_dims(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, gcg::Dims *dm,
              bool mixed_ok = false)
{
    if (bs <= 0 || L <= 0 || g <= 0 || dg <= 0 || hl <= 0) return GCG_ERR_BAD_ARG;
    const bool plain = dtype == GCG_F32 || dtype == GCG_BF16 || dtype == GCG_F16;
    const bool mixed = dtype == GCG_BF16_F32 || dtype == GCG_F16_F32;
    if (!plain && !(mixed && mixed_ok)) return GCG_ERR_BAD_ARG;
    dm->bs = bs; dm->L = L; dm->g = g; dm->dg = dg; dm->hl = hl; dm->d = (int64_t)g * dg; dm->es = 1; dm->keep_out = 0;
    dm->fw = dm->fdecay = nullptr; dm->lc = 0; dm->tmajor = 0; dm->planar = 0;
    return GCG_OK;
}

// The window and MFMA kernels move 8- and 16-byte vectors and need 16-byte aligned
// tensors; the direct kernels load element by element and take any alignment.
int resolve_algo(int algo, int dtype, const gcg::Dims &dm, bool backward, bool aligned16 = true)
{
    const bool mfma_ok = aligned16 && gcg::mfma_supported(dtype, dm) && (!backward || gcg::mfma_bwd_available());
    switch (algo) {
    case GCG_ALGO_AUTO:
        if (aligned16 && gcg::window_supported(dm)) return GCG_ALGO_WINDOW;
        if (mfma_ok) return GCG_ALGO_MFMA;
        return GCG_ALGO_DIRECT;
    case GCG_ALGO_DIRECT: return GCG_ALGO_DIRECT;
    case GCG_ALGO_WINDOW:
        return (aligned16 && gcg::window_supported(dm)) ? GCG_ALGO_WINDOW : GCG_ERR_UNSUPPORTED;
    case GCG_ALGO_MFMA:
        return mfma_ok ? GCG_ALGO_MFMA : GCG_ERR_UNSUPPORTED;
    }
    return GCG_ERR_BAD_ARG;
}

bool all_aligned16(std::initializer_list<const void *> ps)
{
    for (const void *p : ps)
        if (p && ((uintptr_t)p & 15)) return false;
    return true;
}

int finish(int hip_rc)
{
    if (hip_rc == 0) return GCG_OK;
    tls_hip_error = hip_rc;
    return GCG_ERR_LAUNCH;
}

size_t elem_bytes(int dtype) { return dtype == GCG_F32 ? 4 : 2; }

// Scratch of gcg_bwd_static: the filter-gradient partials live in this file-scope device array
// instead of a caller's workspace.  Every GPU the library runs on holds its own copy from the
// first use until the process ends.  `scratch` itself is only the host-side handle of the
// symbol; the device address is looked up once per device and kernels are given that address.
static __device__ __align__(256) unsigned char scratch[GCG_BWD_STATIC_SCRATCH_BYTES];

int static_scratch(void **out)
{
    static std::mutex mu;
    static void *ptr[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { tls_hip_error = (int)e; return GCG_ERR_LAUNCH; }
    if (dev < 0 || dev >= 64) return GCG_ERR_DEVICE;
    std::lock_guard<std::mutex> lk(mu);
    if (!ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) { tls_hip_error = (int)e; return GCG_ERR_LAUNCH; }
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return GCG_OK;
}

// pointer `elems` elements of `dtype` past p
template <typename P> P *at(P *p, size_t elems, int dtype)
{
    return (P *)((uintptr_t)p + elems * elem_bytes(dtype));
}

} // namespace

namespace gcg {
KernelTimer take_kernel_timer()
{
    const KernelTimer t = tls_timer;
    tls_timer = {nullptr, nullptr};
    return t;
}
} // namespace gcg

extern "C" {

GCG_API const char *gcg_strerror(int code)
{
    switch (code) {
    case GCG_OK:              return "ok";
    case GCG_ERR_BAD_ARG:     return "bad argument (null pointer, non-positive size, unknown dtype or algo)";
    case GCG_ERR_UNSUPPORTED: return "shape not supported by the requested kernel family";
    case GCG_ERR_WORKSPACE:   return "workspace missing, misaligned or too small";
    case GCG_ERR_LAUNCH:      return "HIP launch failed (see gcg_last_hip_error)";
    case GCG_ERR_DEVICE:      return "current device is not gfx950";
    case GCG_ERR_STATIC_SCRATCH:
        return "sizes need more filter-gradient scratch than gcg_bwd_static holds (GCG_BWD_STATIC_SCRATCH_BYTES); "
               "use gcg_bwd with a workspace";
    }
    return "unknown error";
}

GCG_API int gcg_last_hip_error(void) { return tls_hip_error; }

GCG_API int gcg_time_next_kernel(void *start_event, void *stop_event)
{
    if ((start_event == nullptr) != (stop_event == nullptr)) return GCG_ERR_BAD_ARG;
    tls_timer = {(hipEvent_t)start_event, (hipEvent_t)stop_event};
    return GCG_OK;
}

GCG_API int gcg_version(void) { return 106; }

GCG_API int gcg_select_algo(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, int32_t backward)
{
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    return resolve_algo(GCG_ALGO_AUTO, dtype, dm, backward != 0);
}

namespace {
// the tensors' own type code of a mixed code (16-bit tensors, fp32 arithmetic)
int plain_tensor_code(int dtype) { return dtype == GCG_BF16_F32 ? GCG_BF16 : dtype == GCG_F16_F32 ? GCG_F16 : dtype; }
} // namespace

GCG_API int gcg_route_supported(int32_t route, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
                                int32_t dtype)
{
    gcg::Dims dm;
    const bool mixer = route == GCG_ROUTE_MIXER_SE || route == GCG_ROUTE_MIXER_MR || route == GCG_ROUTE_MIXER_MR_PLANAR;
    if (make_dims(bs, L, g, dg, hl, dtype, &dm, true) || (mixer && kf <= 0)) return GCG_ERR_BAD_ARG;
    switch (route) {
    case GCG_ROUTE_DECAY:               // the filter is formed in the matrix-core kernels only
        return gcg::mfma_supported(dtype, dm) ? 1 : 0;
    case GCG_ROUTE_TIME_MAJOR:          // register-window kernels, whose windows span bs rows of memory per time row
        dm.tmajor = 1;
        return gcg::window_supported(dm) ? 1 : 0;
    case GCG_ROUTE_MIXER_SE:
        dm.es = 3;
        return gcg::mixer_se_supported(dm, kf) ? 1 : 0;
    case GCG_ROUTE_MIXER_MR: {          // one kernel each way, or the 8-wave kernels with the featurizer in front
        dm.es = 3;
        if (!gcg::mfma_feat_supported(dtype, dm, kf)) return 0;
        if (gcg::mixer_mr_fused_supported(dtype, dm, kf)) return 1;
        gcg::Dims df;                   // the two-kernel backward ends in the featurizer's own backward
        if (make_dims(bs, L, 3 * g * dg, 1, kf, plain_tensor_code(dtype), &df)) return 0;
        return gcg::dwconv_supported(df) ? 1 : 0;
    }
    case GCG_ROUTE_MIXER_MR_PLANAR:
        dm.planar = 1;
        dm.es = 1;
        return gcg::mfma_feat_supported(dtype, dm, kf) && gcg::mixer_mr_fused_supported(dtype, dm, kf) ? 1 : 0;
    }
    return GCG_ERR_BAD_ARG;
}

GCG_API int gcg_fwd(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, int32_t algo,
            void *stream)
{
    TimerScope timer_scope;
    if (!x || !B || !C || !h || !y) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    const int a = resolve_algo(algo, dtype, dm, false, all_aligned16({x, B, C, y, y2, bx}));
    if (a < 0) return a;
    rc = check_device();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (a) {
    case GCG_ALGO_DIRECT: return finish(gcg::direct_fwd_launch(dtype, x, B, C, h, y, y2, bx, dm, st));
    case GCG_ALGO_WINDOW: return finish(gcg::window_fwd_launch(dtype, x, B, C, h, y, y2, bx, dm, st));
    case GCG_ALGO_MFMA:   return finish(gcg::mfma_fwd_launch(dtype, x, B, C, h, y, y2, bx, dm, st));
    }
    return GCG_ERR_BAD_ARG;
}

GCG_API size_t gcg_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype,
                               int32_t algo)
{
    gcg::Dims dm;
    if (make_dims(bs, L, g, dg, hl, dtype, &dm, true)) return 0;
    const int a = resolve_algo(algo, dtype, dm, true);
    size_t n = 0;
    switch (a) {
    case GCG_ALGO_DIRECT: n = gcg::direct_bwd_workspace(dm); break;
    case GCG_ALGO_WINDOW: n = gcg::window_bwd_workspace(dm); break;
    case GCG_ALGO_MFMA:   n = gcg::mfma_bwd_workspace(dtype, dm); break;
    default: return 0;
    }
    // under AUTO a misaligned tensor reroutes to the direct kernels: size for both
    if (algo == GCG_ALGO_AUTO && gcg::direct_bwd_workspace(dm) > n) n = gcg::direct_bwd_workspace(dm);
    return (n + 255) & ~(size_t)255;
}

GCG_API int gcg_bwd(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx, void *dB,
            void *dC, void *dh, void *workspace, size_t workspace_bytes, int64_t bs, int64_t L, int32_t g,
            int32_t dg, int32_t hl, int32_t dtype, int32_t algo, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !x || !B || !C || !h || !dx || !dB || !dC || !dh) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    const int a = resolve_algo(algo, dtype, dm, true, all_aligned16({dy, x, B, C, dx, dB, dC}));
    if (a < 0) return a;
    const size_t need = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, dtype, a);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (a) {
    case GCG_ALGO_DIRECT:
        return finish(gcg::direct_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    case GCG_ALGO_WINDOW:
        return finish(gcg::window_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    case GCG_ALGO_MFMA:
        return finish(gcg::mfma_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    }
    return GCG_ERR_BAD_ARG;
}

GCG_API int gcg_bwd_static(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx,
                           void *dB, void *dC, void *dh, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                           int32_t dtype, int32_t algo, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !x || !B || !C || !h || !dx || !dB || !dC || !dh) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    const int a = resolve_algo(algo, dtype, dm, true, all_aligned16({dy, x, B, C, dx, dB, dC}));
    if (a < 0) return a;
    const size_t need = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, dtype, a);
    if (need == 0) return GCG_ERR_BAD_ARG;
    if (need > (size_t)GCG_BWD_STATIC_SCRATCH_BYTES) return GCG_ERR_STATIC_SCRATCH;
    rc = check_device();
    if (rc) return rc;
    void *ws = nullptr;
    rc = static_scratch(&ws);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (a) {
    case GCG_ALGO_DIRECT:
        return finish(gcg::direct_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st));
    case GCG_ALGO_WINDOW:
        return finish(gcg::window_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st));
    case GCG_ALGO_MFMA:
        return finish(gcg::mfma_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, ws, dm, st));
    }
    return GCG_ERR_BAD_ARG;
}

// ---- interleaved operands: one (bs, L, g, dg, 3) tensor instead of three (bs, L, g, dg) ones

GCG_API int gcg_fwd_interleaved(const void *feat, const void *h, void *y, int64_t bs, int64_t L, int32_t g, int32_t dg,
                                int32_t hl, int32_t dtype, int32_t algo, void *stream)
{
    TimerScope timer_scope;
    if (!feat || !h || !y) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.es = 3;
    const int a = resolve_algo(algo, dtype, dm, false, all_aligned16({feat, y}));
    if (a < 0) return a;
    rc = check_device();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const void *C = feat, *B = at(feat, 1, dtype), *x = at(feat, 2, dtype);
    switch (a) {
    case GCG_ALGO_DIRECT: return finish(gcg::direct_fwd_launch(dtype, x, B, C, h, y, nullptr, nullptr, dm, st));
    case GCG_ALGO_WINDOW: return finish(gcg::window_fwd_launch(dtype, x, B, C, h, y, nullptr, nullptr, dm, st));
    case GCG_ALGO_MFMA:   return finish(gcg::mfma_il_fwd_launch(dtype, feat, h, y, dm, st));
    }
    return GCG_ERR_BAD_ARG;
}

GCG_API int gcg_bwd_interleaved(const void *dy, const void *feat, const void *h, void *dfeat, void *dh, void *workspace,
                                size_t workspace_bytes, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                                int32_t dtype, int32_t algo, int32_t flags, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !feat || !h || !dfeat || !dh || (flags & ~GCG_KEEP_OUTPUT)) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.es = 3;
    dm.keep_out = flags & GCG_KEEP_OUTPUT;
    const int a = resolve_algo(algo, dtype, dm, true, all_aligned16({dy, feat, dfeat}));
    if (a < 0) return a;
    const size_t need = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, dtype, a);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const void *C = feat, *B = at(feat, 1, dtype), *x = at(feat, 2, dtype);
    void *dC = dfeat, *dB = at(dfeat, 1, dtype), *dx = at(dfeat, 2, dtype);
    switch (a) {
    case GCG_ALGO_DIRECT:
        return finish(gcg::direct_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    case GCG_ALGO_WINDOW:
        return finish(gcg::window_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    case GCG_ALGO_MFMA:
        return finish(gcg::mfma_il_bwd_launch(dtype, dy, feat, h, dfeat, dh, workspace, dm, st));
    }
    return GCG_ERR_BAD_ARG;
}

// ---- planar operands: the thirds (C | B | x) of the rows of one (bs, L, 3 * g * dg) tensor, read in place

namespace {
const void *plane(const void *base, int k, int64_t d, int dtype)
{
    return (const char *)base + (size_t)k * d * (dtype == GCG_F32 ? 4 : 2);
}
void *plane_out(void *base, int k, int64_t d, int dtype) { return (char *)base + (size_t)k * d * (dtype == GCG_F32 ? 4 : 2); }
} // namespace

GCG_API int gcg_fwd_planar(const void *feat, const void *h, void *y, int64_t bs, int64_t L, int32_t g, int32_t dg,
                           int32_t hl, int32_t dtype, int32_t algo, void *stream)
{
    TimerScope timer_scope;
    if (!feat || !h || !y) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.planar = 1;
    const void *C = feat, *B = plane(feat, 1, dm.d, dtype), *x = plane(feat, 2, dm.d, dtype);
    // (the planes themselves lie d elements apart: a multiple of the kernels' vector width wherever a family takes the shape)
    const int a = resolve_algo(algo, dtype, dm, false, all_aligned16({feat, y}));
    if (a < 0) return a;
    rc = check_device();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (a) {
    case GCG_ALGO_DIRECT: return finish(gcg::direct_fwd_launch(dtype, x, B, C, h, y, nullptr, nullptr, dm, st));
    case GCG_ALGO_WINDOW: return finish(gcg::window_fwd_launch(dtype, x, B, C, h, y, nullptr, nullptr, dm, st));
    case GCG_ALGO_MFMA:   return finish(gcg::mfma_fwd_launch(dtype, x, B, C, h, y, nullptr, nullptr, dm, st));
    }
    return GCG_ERR_BAD_ARG;
}

GCG_API int gcg_bwd_planar(const void *dy, const void *feat, const void *h, void *dfeat, void *dh, void *workspace,
                           size_t workspace_bytes, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                           int32_t dtype, int32_t algo, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !feat || !h || !dfeat || !dh) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.planar = 1;
    const void *C = feat, *B = plane(feat, 1, dm.d, dtype), *x = plane(feat, 2, dm.d, dtype);
    void *dC = dfeat, *dB = plane_out(dfeat, 1, dm.d, dtype), *dx = plane_out(dfeat, 2, dm.d, dtype);
    const int a = resolve_algo(algo, dtype, dm, true, all_aligned16({dy, feat, dfeat}));
    if (a < 0) return a;
    const size_t need = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, dtype, a);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (a) {
    case GCG_ALGO_DIRECT:
        return finish(gcg::direct_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    case GCG_ALGO_WINDOW:
        return finish(gcg::window_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    case GCG_ALGO_MFMA:
        return finish(gcg::mfma_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, st));
    }
    return GCG_ERR_BAD_ARG;
}

// ---- the gated convolution with the decayed explicit filter built inside the kernels ---------------
// Matrix-core kernels only (hl <= 128, dg % 16 == 0, 16-byte aligned tensors); other shapes are refused and
// the caller makes the filter with gcg_filter_decay_fwd.

namespace {
int decay_dims(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, const float *w,
               const float *decay, int32_t l_cache, gcg::Dims *dm)
{
    if (!w || !decay || l_cache < hl) return GCG_ERR_BAD_ARG;
    const int rc = make_dims(bs, L, g, dg, hl, dtype, dm, true);
    if (rc) return rc;
    dm->fw = w; dm->fdecay = decay; dm->lc = l_cache;
    return GCG_OK;
}
} // namespace

GCG_API int gcg_fwd_decay(const void *x, const void *B, const void *C, const float *w, const float *decay,
                          int32_t l_cache, void *y, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                          int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!x || !B || !C || !y) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    const int a = resolve_algo(GCG_ALGO_MFMA, dtype, dm, false, all_aligned16({x, B, C, y}));
    if (a < 0) return a;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::mfma_fwd_launch(dtype, x, B, C, nullptr, y, nullptr, nullptr, dm, (hipStream_t)stream));
}

GCG_API int gcg_bwd_decay(const void *dy, const void *x, const void *B, const void *C, const float *w,
                          const float *decay, int32_t l_cache, void *dx, void *dB, void *dC, float *dw,
                          void *workspace, size_t workspace_bytes, int64_t bs, int64_t L, int32_t g, int32_t dg,
                          int32_t hl, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !x || !B || !C || !dx || !dB || !dC || !dw) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    const int a = resolve_algo(GCG_ALGO_MFMA, dtype, dm, true, all_aligned16({dy, x, B, C, dx, dB, dC}));
    if (a < 0) return a;
    const size_t need = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, dtype, a);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::mfma_bwd_launch(dtype, dy, x, B, C, nullptr, dx, dB, dC, dw, workspace, dm, (hipStream_t)stream));
}

GCG_API int gcg_fwd_interleaved_decay(const void *feat, const float *w, const float *decay, int32_t l_cache, void *y,
                                      int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype,
                                      void *stream)
{
    TimerScope timer_scope;
    if (!feat || !y) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    dm.es = 3;
    const int a = resolve_algo(GCG_ALGO_MFMA, dtype, dm, false, all_aligned16({feat, y}));
    if (a < 0) return a;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::mfma_il_fwd_launch(dtype, feat, nullptr, y, dm, (hipStream_t)stream));
}

GCG_API int gcg_bwd_interleaved_decay(const void *dy, const void *feat, const float *w, const float *decay,
                                      int32_t l_cache, void *dfeat, float *dw, void *workspace, size_t workspace_bytes,
                                      int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype,
                                      int32_t flags, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !feat || !dfeat || !dw || (flags & ~GCG_KEEP_OUTPUT)) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    dm.es = 3;
    dm.keep_out = flags & GCG_KEEP_OUTPUT;
    const int a = resolve_algo(GCG_ALGO_MFMA, dtype, dm, true, all_aligned16({dy, feat, dfeat}));
    if (a < 0) return a;
    const size_t need = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, dtype, a);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::mfma_il_bwd_launch(dtype, dy, feat, nullptr, dfeat, dw, workspace, dm, (hipStream_t)stream));
}

// ---- the short-filter operator on time-major operands (the layout of run_short_hyena) ------------
// Register-window kernels only (hl <= 8, dg % 4 == 0, 16-byte aligned tensors).

GCG_API int gcg_fwd_time_major(const void *x, const void *B, const void *C, const void *h, void *y, int64_t bs,
                               int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!x || !B || !C || !h || !y) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.tmajor = 1;
    const int a = resolve_algo(GCG_ALGO_WINDOW, dtype, dm, false, all_aligned16({x, B, C, y}));
    if (a < 0) return a;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::window_fwd_launch(dtype, x, B, C, h, y, nullptr, nullptr, dm, (hipStream_t)stream));
}

GCG_API size_t gcg_bwd_time_major_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                                                  int32_t dtype)
{
    gcg::Dims dm;
    if (make_dims(bs, L, g, dg, hl, dtype, &dm, true)) return 0;
    dm.tmajor = 1;
    if (!gcg::window_supported(dm)) return 0;
    return (gcg::window_bwd_workspace(dm) + 255) & ~(size_t)255;
}

GCG_API int gcg_bwd_time_major(const void *dy, const void *x, const void *B, const void *C, const void *h, void *dx,
                               void *dB, void *dC, void *dh, void *workspace, size_t workspace_bytes, int64_t bs,
                               int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !x || !B || !C || !h || !dx || !dB || !dC || !dh) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.tmajor = 1;
    const int a = resolve_algo(GCG_ALGO_WINDOW, dtype, dm, true, all_aligned16({dy, x, B, C, dx, dB, dC}));
    if (a < 0) return a;
    const size_t need = gcg_bwd_time_major_workspace_bytes(bs, L, g, dg, hl, dtype);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::window_bwd_launch(dtype, dy, x, B, C, h, dx, dB, dC, dh, workspace, dm, (hipStream_t)stream));
}

// ---- ungated short causal depthwise convolution (featurizer)

GCG_API int gcg_dwconv_fwd(const void *x, const void *w, void *y, int64_t bs, int64_t L, int32_t g, int32_t dg,
                           int32_t hl, int32_t dtype, int32_t flags, void *stream)
{
    TimerScope timer_scope;
    if (!x || !w || !y || (flags & ~GCG_KEEP_OUTPUT)) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm);
    if (rc) return rc;
    dm.keep_out = flags & GCG_KEEP_OUTPUT;
    if (!gcg::dwconv_supported(dm) || !all_aligned16({x, y})) return GCG_ERR_UNSUPPORTED;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::dwconv_fwd_launch(dtype, x, w, y, dm, (hipStream_t)stream));
}

GCG_API size_t gcg_dwconv_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype)
{
    gcg::Dims dm;
    if (make_dims(bs, L, g, dg, hl, dtype, &dm) || !gcg::dwconv_supported(dm)) return 0;
    return (gcg::dwconv_bwd_workspace(dm) + 255) & ~(size_t)255;
}

GCG_API int gcg_dwconv_bwd(const void *dy, const void *x, const void *w, void *dx, void *dw, void *workspace,
                           size_t workspace_bytes, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                           int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !x || !w || !dx || !dw) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm);
    if (rc) return rc;
    if (!gcg::dwconv_supported(dm) || !all_aligned16({dy, x, dx})) return GCG_ERR_UNSUPPORTED;
    const size_t need = gcg_dwconv_bwd_workspace_bytes(bs, L, g, dg, hl, dtype);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::dwconv_bwd_launch(dtype, dy, x, w, dx, dw, workspace, dm, (hipStream_t)stream));
}

// ---- featurizer + Hyena-SE operator in one pass

namespace {
int mixer_se_fwd_any(const void *raw, const void *wf, const void *h, void *y, int64_t bs, int64_t L, int32_t g,
                     int32_t dg, int32_t hl, int32_t kf, int32_t dtype, int planar, void *stream)
{
    if (!raw || !wf || !h || !y) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    if (kf <= 0) return GCG_ERR_BAD_ARG;
    dm.planar = planar;
    if (!gcg::mixer_se_supported(dm, kf) || !all_aligned16({raw, y})) return GCG_ERR_UNSUPPORTED;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::mixer_se_fwd_launch(dtype, raw, wf, h, y, dm, kf, (hipStream_t)stream));
}
int mixer_se_bwd_any(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh,
                     void *workspace, size_t workspace_bytes, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                     int32_t kf, int32_t dtype, int planar, void *stream)
{
    if (!dy || !raw || !wf || !h || !draw || !dwf || !dh) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    if (kf <= 0) return GCG_ERR_BAD_ARG;
    dm.planar = planar;
    if (!gcg::mixer_se_supported(dm, kf) || !all_aligned16({dy, raw, draw})) return GCG_ERR_UNSUPPORTED;
    const size_t need = gcg_mixer_se_bwd_workspace_bytes(bs, L, g, dg, hl, kf, dtype);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    return finish(gcg::mixer_se_bwd_launch(dtype, dy, raw, wf, h, draw, dwf, dh, workspace, dm, kf, (hipStream_t)stream));
}
} // namespace

GCG_API int gcg_mixer_se_fwd(const void *raw, const void *wf, const void *h, void *y, int64_t bs, int64_t L, int32_t g,
                             int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    return mixer_se_fwd_any(raw, wf, h, y, bs, L, g, dg, hl, kf, dtype, 0, stream);
}

GCG_API int gcg_mixer_se_fwd_planar(const void *raw, const void *wf, const void *h, void *y, int64_t bs, int64_t L,
                                    int32_t g, int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    return mixer_se_fwd_any(raw, wf, h, y, bs, L, g, dg, hl, kf, dtype, 1, stream);
}

GCG_API size_t gcg_mixer_se_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
                                                int32_t dtype)
{
    gcg::Dims dm;
    if (make_dims(bs, L, g, dg, hl, dtype, &dm, true) || kf <= 0 || !gcg::mixer_se_supported(dm, kf)) return 0;
    return (gcg::mixer_se_bwd_workspace(dtype, dm, kf) + 255) & ~(size_t)255;
}

GCG_API int gcg_mixer_se_bwd(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf,
                             void *dh, void *workspace, size_t workspace_bytes, int64_t bs, int64_t L, int32_t g,
                             int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    return mixer_se_bwd_any(dy, raw, wf, h, draw, dwf, dh, workspace, workspace_bytes, bs, L, g, dg, hl, kf, dtype, 0,
                            stream);
}

GCG_API int gcg_mixer_se_bwd_planar(const void *dy, const void *raw, const void *wf, const void *h, void *draw,
                                    void *dwf, void *dh, void *workspace, size_t workspace_bytes, int64_t bs, int64_t L,
                                    int32_t g, int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    return mixer_se_bwd_any(dy, raw, wf, h, draw, dwf, dh, workspace, workspace_bytes, bs, L, g, dg, hl, kf, dtype, 1,
                            stream);
}

// ---- featurizer and Hyena-MR operator: the forward in one pass

namespace {
int mixer_mr_fwd_dims(const void *raw, const void *wf, const void *h, void *y, gcg::Dims &dm, int kf, int dtype,
                      void *stream);
}

GCG_API int gcg_mixer_mr_fwd(const void *raw, const void *wf, const void *h, void *y, int64_t bs, int64_t L, int32_t g,
                             int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!raw || !wf || !h || !y || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    return mixer_mr_fwd_dims(raw, wf, h, y, dm, kf, dtype, stream);
}

GCG_API int gcg_mixer_mr_fwd_planar(const void *raw, const void *wf, const void *h, void *y, int64_t bs, int64_t L,
                                    int32_t g, int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!raw || !wf || !h || !y || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.planar = 1;
    return mixer_mr_fwd_dims(raw, wf, h, y, dm, kf, dtype, stream);
}

GCG_API int gcg_mixer_mr_fwd_decay(const void *raw, const void *wf, const float *w, const float *decay, int32_t l_cache,
                                   void *y, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
                                   int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!raw || !wf || !y || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    return mixer_mr_fwd_dims(raw, wf, nullptr, y, dm, kf, dtype, stream);
}

GCG_API int gcg_mixer_mr_fwd_planar_decay(const void *raw, const void *wf, const float *w, const float *decay,
                                          int32_t l_cache, void *y, int64_t bs, int64_t L, int32_t g, int32_t dg,
                                          int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!raw || !wf || !y || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    dm.planar = 1;
    return mixer_mr_fwd_dims(raw, wf, nullptr, y, dm, kf, dtype, stream);
}

namespace {
int mixer_mr_fwd_dims(const void *raw, const void *wf, const void *h, void *y, gcg::Dims &dm, int kf, int dtype,
                      void *stream)
{
    int rc = 0;
    dm.es = dm.planar ? 1 : 3;
    if (!all_aligned16({raw, y}) || !gcg::mfma_feat_supported(dtype, dm, kf)) return GCG_ERR_UNSUPPORTED;
    if (dm.planar && !gcg::mixer_mr_fused_supported(dtype, dm, kf)) return GCG_ERR_UNSUPPORTED;   // one-kernel path only
    rc = check_device();
    if (rc) return rc;
    if (gcg::mixer_mr_fused_supported(dtype, dm, kf))
        return finish(gcg::mixer_mr_fused_fwd_launch(dtype, raw, wf, kf, h, y, dm, (hipStream_t)stream));
    return finish(gcg::mfma_il_fwd_feat_launch(dtype, raw, wf, kf, h, y, dm, (hipStream_t)stream));
}
} // namespace

namespace {
size_t up256(size_t n) { return (n + 255) & ~(size_t)255; }
} // namespace

GCG_API size_t gcg_mixer_mr_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
                                                int32_t dtype)
{
    gcg::Dims dm, df;
    if (kf <= 0 || make_dims(bs, L, g, dg, hl, dtype, &dm, true)) return 0;
    if (!gcg::mfma_feat_supported(dtype, dm, kf)) return 0;
    if (make_dims(bs, L, 3 * g * dg, 1, kf, plain_tensor_code(dtype), &df) || !gcg::dwconv_supported(df)) return 0;
    const size_t chain = up256(gcg::mfma_feat_bwd_workspace(dtype, dm)) + up256(gcg::dwconv_bwd_workspace(df));
    const size_t fused = gcg::mixer_mr_fused_supported(dtype, dm, kf) ? up256(gcg::mixer_mr_fused_workspace(dm, kf)) : 0;
    return chain > fused ? chain : fused;
}

GCG_API size_t gcg_mixer_mr_bwd_scratch_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
                                              int32_t dtype)
{
    gcg::Dims dm;
    if (kf <= 0 || make_dims(bs, L, g, dg, hl, dtype, &dm, true)) return 0;
    if (gcg::mixer_mr_fused_supported(dtype, dm, kf)) return 0;
    return (size_t)(3 * bs * L * dm.d) * (dtype == GCG_F32 ? 4 : 2);
}

namespace {
int mixer_mr_bwd_dims(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh,
                      void *dfeat_scratch, void *workspace, size_t workspace_bytes, gcg::Dims &dm, int kf, int dtype,
                      void *stream);
}

GCG_API int gcg_mixer_mr_bwd(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf,
                             void *dh, void *dfeat_scratch, void *workspace, size_t workspace_bytes, int64_t bs,
                             int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !raw || !wf || !h || !draw || !dwf || !dh || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    return mixer_mr_bwd_dims(dy, raw, wf, h, draw, dwf, dh, dfeat_scratch, workspace, workspace_bytes, dm, kf, dtype, stream);
}

GCG_API int gcg_mixer_mr_bwd_planar(const void *dy, const void *raw, const void *wf, const void *h, void *draw,
                                    void *dwf, void *dh, void *workspace, size_t workspace_bytes, int64_t bs, int64_t L,
                                    int32_t g, int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !raw || !wf || !h || !draw || !dwf || !dh || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = make_dims(bs, L, g, dg, hl, dtype, &dm, true);
    if (rc) return rc;
    dm.planar = 1;
    return mixer_mr_bwd_dims(dy, raw, wf, h, draw, dwf, dh, nullptr, workspace, workspace_bytes, dm, kf, dtype, stream);
}

GCG_API int gcg_mixer_mr_bwd_decay(const void *dy, const void *raw, const void *wf, const float *w, const float *decay,
                                   int32_t l_cache, void *draw, void *dwf, float *dw, void *dfeat_scratch,
                                   void *workspace, size_t workspace_bytes, int64_t bs, int64_t L, int32_t g, int32_t dg,
                                   int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !raw || !wf || !draw || !dwf || !dw || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    return mixer_mr_bwd_dims(dy, raw, wf, nullptr, draw, dwf, dw, dfeat_scratch, workspace, workspace_bytes, dm, kf, dtype,
                             stream);
}

GCG_API int gcg_mixer_mr_bwd_planar_decay(const void *dy, const void *raw, const void *wf, const float *w,
                                          const float *decay, int32_t l_cache, void *draw, void *dwf, float *dw,
                                          void *workspace, size_t workspace_bytes, int64_t bs, int64_t L, int32_t g,
                                          int32_t dg, int32_t hl, int32_t kf, int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dy || !raw || !wf || !draw || !dwf || !dw || kf <= 0) return GCG_ERR_BAD_ARG;
    gcg::Dims dm;
    const int rc = decay_dims(bs, L, g, dg, hl, dtype, w, decay, l_cache, &dm);
    if (rc) return rc;
    dm.planar = 1;
    return mixer_mr_bwd_dims(dy, raw, wf, nullptr, draw, dwf, dw, nullptr, workspace, workspace_bytes, dm, kf, dtype, stream);
}

namespace {
int mixer_mr_bwd_dims(const void *dy, const void *raw, const void *wf, const void *h, void *draw, void *dwf, void *dh,
                      void *dfeat_scratch, void *workspace, size_t workspace_bytes, gcg::Dims &dm, int kf, int dtype,
                      void *stream)
{
    gcg::Dims df;
    const int64_t bs = dm.bs, L = dm.L;
    const int32_t g = dm.g, dg = dm.dg, hl = dm.hl;
    int rc = 0;
    dm.es = dm.planar ? 1 : 3;
    dm.keep_out = 1;
    const bool fused = gcg::mixer_mr_fused_supported(dtype, dm, kf);
    if (dm.planar && !fused) return GCG_ERR_UNSUPPORTED;          // one-kernel path only
    if (!fused && !dfeat_scratch) return GCG_ERR_BAD_ARG;
    if (!all_aligned16({dy, raw, draw}) || (!fused && !all_aligned16({dfeat_scratch})) ||
        !gcg::mfma_feat_supported(dtype, dm, kf))
        return GCG_ERR_UNSUPPORTED;
    rc = make_dims(bs, L, 3 * g * dg, 1, kf, plain_tensor_code(dtype), &df);
    if (rc) return rc;
    if (!gcg::dwconv_supported(df)) return GCG_ERR_UNSUPPORTED;
    const size_t need = gcg_mixer_mr_bwd_workspace_bytes(bs, L, g, dg, hl, kf, dtype);
    if (!need || !workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return GCG_ERR_WORKSPACE;
    rc = check_device();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (fused)
        return finish(gcg::mixer_mr_fused_bwd_launch(dtype, dy, raw, wf, kf, h, draw, dwf, dh, workspace, dm, st));
    void *ws2 = (char *)workspace + up256(gcg::mfma_feat_bwd_workspace(dtype, dm));
    int e = gcg::mfma_il_bwd_feat_launch(dtype, dy, raw, wf, kf, h, dfeat_scratch, dh, workspace, dm, st);
    if (e) return finish(e);
    return finish(gcg::dwconv_bwd_launch(plain_tensor_code(dtype), dfeat_scratch, raw, wf, draw, dwf, ws2, df, st));
}
} // namespace

// ---- explicit decayed filter (Hyena-MR parametrization)

GCG_API int gcg_filter_decay_fwd(const float *w, const float *decay, void *h, int32_t g, int32_t l_cache, int32_t hl,
                                 int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!w || !decay || !h || g <= 0 || hl <= 0 || l_cache < hl) return GCG_ERR_BAD_ARG;
    if (dtype != GCG_F32 && dtype != GCG_BF16 && dtype != GCG_F16) return GCG_ERR_BAD_ARG;
    const int rc = check_device();
    if (rc) return rc;
    return finish(gcg::filter_fwd_launch(dtype, w, decay, h, g, l_cache, hl, (hipStream_t)stream));
}

GCG_API int gcg_filter_decay_bwd(const void *dh, const float *decay, float *dw, int32_t g, int32_t l_cache, int32_t hl,
                                 int32_t dtype, void *stream)
{
    TimerScope timer_scope;
    if (!dh || !decay || !dw || g <= 0 || hl <= 0 || l_cache < hl) return GCG_ERR_BAD_ARG;
    if (dtype != GCG_F32 && dtype != GCG_BF16 && dtype != GCG_F16) return GCG_ERR_BAD_ARG;
    const int rc = check_device();
    if (rc) return rc;
    return finish(gcg::filter_bwd_launch(dtype, dh, decay, dw, g, l_cache, hl, (hipStream_t)stream));
}

} // extern "C"
