// PyTorch binding of the C ABI (include/gcg.h): the operators are registered in the `gcg`
// namespace of torch.ops with device and meta (shape-only) implementations, so that they can be
// called from eager code, traced by torch.compile and captured into graphs.  Each device
// implementation checks its arguments, allocates the outputs with torch's allocator, and
// enqueues the C-ABI entry point on torch's current stream under a device guard; error codes
// become exceptions.  The backward formulas of the forward operators are registered on the Python side
// (savanna_amd/_ops.py: torch.library.register_autograd), each in terms of the backward operator defined here.
//
// This is the counterpart of the Triton launch wrappers two_pass_fwd_grouped /
// two_pass_bwd_refactor (savanna/kernels/triton_src/cgcg/src/fwd.py:13-233, src/bwd.py:347-474)
// as TwoPassChunkedGateConvGate calls them (cgcg/interface.py:27-127).
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>
#include <torch/types.h>

#include <tuple>

#include "../../include/gcg.h"

namespace {

using at::Tensor;
using DeviceGuard = at::hip::OptionalHIPGuardMasqueradingAsCUDA;

int dtype_code(at::ScalarType t)
{
    switch (t) {
    case at::kFloat: return GCG_F32;
    case at::kBFloat16: return GCG_BF16;
    case at::kHalf: return GCG_F16;
    default: TORCH_CHECK(false, "gcg: unsupported dtype ", t, "; expected float32, bfloat16 or float16");
    }
}

// dtype code of the gated operator: the tensors' dtype, or 16-bit tensors with an fp32 filter
int gated_code(const Tensor &x, const Tensor &h)
{
    const at::ScalarType t = x.scalar_type(), f = h.scalar_type();
    if (f == t) return dtype_code(t);
    TORCH_CHECK(f == at::kFloat && (t == at::kBFloat16 || t == at::kHalf),
                "gcg: the filter must have the tensors' dtype, or be float32 with bfloat16 / float16 tensors; got ", t,
                " tensors and a ", f, " filter");
    return t == at::kBFloat16 ? GCG_BF16_F32 : GCG_F16_F32;
}

void *stream_of(const Tensor &t)
{
    return (void *)at::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

void check_rc(int rc, const char *what)
{
    TORCH_CHECK(rc == 0, what, ": ", gcg_strerror(rc), " (code ", rc, ", hipError ", gcg_last_hip_error(), ")");
}

void require_gpu(const Tensor &t, const char *name)
{
    TORCH_CHECK(t.is_cuda(), "gcg: ", name, " is on ", t.device(),
                "; the kernels run on an MI355X (gfx950) device only and there is no CPU path");
}

// x, B, C (and dy): contiguous (bs, L, g, dg) of one dtype on one device; h: contiguous (g, 1, hl)
void check_gated(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h)
{
    TORCH_CHECK(x.dim() == 4, "gcg: x must be (bs, L, g, dg)");
    TORCH_CHECK(B.sizes() == x.sizes() && C.sizes() == x.sizes(), "gcg: x, B and C must have one shape");
    TORCH_CHECK(h.dim() == 3 && h.size(0) == x.size(2) && h.size(1) == 1, "gcg: h must be (g, 1, hl)");
    TORCH_CHECK(B.scalar_type() == x.scalar_type() && C.scalar_type() == x.scalar_type(),
                "gcg: x, B and C must share one dtype");
    (void)gated_code(x, h);
    TORCH_CHECK(B.device() == x.device() && C.device() == x.device() && h.device() == x.device(),
                "gcg: x, B, C and h must be on one device");
    TORCH_CHECK(x.is_contiguous() && B.is_contiguous() && C.is_contiguous() && h.is_contiguous(),
                "gcg: x, B, C and h must be contiguous");
}

void check_like(const Tensor &t, const Tensor &ref, const char *name)
{
    TORCH_CHECK(t.sizes() == ref.sizes() && t.scalar_type() == ref.scalar_type() && t.device() == ref.device() &&
                    t.is_contiguous(),
                "gcg: ", name, " must be a contiguous tensor with the shape, dtype and device of its counterpart");
}

void check_feat(const Tensor &feat, const Tensor &h)
{
    TORCH_CHECK(feat.dim() == 5 && feat.size(4) == 3 && feat.is_contiguous(),
                "gcg: feat must be a contiguous (bs, L, g, dg, 3) tensor");
    TORCH_CHECK(h.dim() == 3 && h.size(0) == feat.size(2) && h.size(1) == 1 && h.is_contiguous(),
                "gcg: h must be a contiguous (g, 1, hl) tensor");
    TORCH_CHECK(h.device() == feat.device(), "gcg: feat and h must be on one device");
    (void)gated_code(feat, h);
}

Tensor workspace(size_t bytes, const Tensor &like, const char *what)
{
    TORCH_CHECK(bytes > 0, what, ": arguments rejected (shape not supported by the requested kernel family)");
    return at::empty({(int64_t)bytes}, like.options().dtype(at::kByte));
}

// ---- gated convolution on separate tensors ----------------------------------------------------

// (bx, y2, y); bx / y2 are empty (0-element) tensors unless asked for
std::tuple<Tensor, Tensor, Tensor> fwd_full(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h,
                                            bool return_bx, bool return_y2, int64_t algo)
{
    require_gpu(x, "x");
    check_gated(x, B, C, h);
    DeviceGuard guard(x.device());
    Tensor y = at::empty_like(x);
    Tensor y2 = return_y2 ? at::empty_like(x) : at::empty({0}, x.options());
    Tensor bx = return_bx ? at::empty_like(x) : at::empty({0}, x.options());
    if (x.numel() == 0) return {bx, y2, y};
    check_rc(gcg_fwd(x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), y.data_ptr(),
                     return_y2 ? y2.data_ptr() : nullptr, return_bx ? bx.data_ptr() : nullptr, x.size(0), x.size(1),
                     (int32_t)x.size(2), (int32_t)x.size(3), (int32_t)h.size(2), gated_code(x, h),
                     (int32_t)algo, stream_of(x)),
             "gcg_fwd");
    return {bx, y2, y};
}

Tensor fwd(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h, int64_t algo)
{
    return std::get<2>(fwd_full(x, B, C, h, false, false, algo));
}

// y into a tensor the caller owns
void fwd_out(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h, Tensor &y, int64_t algo)
{
    require_gpu(x, "x");
    check_gated(x, B, C, h);
    check_like(y, x, "out");
    if (x.numel() == 0) return;
    DeviceGuard guard(x.device());
    check_rc(gcg_fwd(x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), y.data_ptr(), nullptr, nullptr, x.size(0),
                     x.size(1), (int32_t)x.size(2), (int32_t)x.size(3), (int32_t)h.size(2),
                     gated_code(x, h), (int32_t)algo, stream_of(x)),
             "gcg_fwd");
}

std::tuple<Tensor, Tensor, Tensor, Tensor> bwd(const Tensor &dy, const Tensor &x, const Tensor &B, const Tensor &C,
                                               const Tensor &h, int64_t algo)
{
    require_gpu(x, "x");
    check_gated(x, B, C, h);
    check_like(dy, x, "dy");
    DeviceGuard guard(x.device());
    Tensor dx = at::empty_like(x), dB = at::empty_like(x), dC = at::empty_like(x), dh = at::empty_like(h);
    if (x.numel() == 0) return {dx, dB, dC, dh.zero_()};
    const int64_t bs = x.size(0), L = x.size(1);
    const int32_t g = (int32_t)x.size(2), dg = (int32_t)x.size(3), hl = (int32_t)h.size(2);
    const int code = gated_code(x, h);
    const size_t nbytes = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, (int32_t)algo);
    Tensor ws = workspace(nbytes, x, "gcg_bwd_workspace_bytes");
    check_rc(gcg_bwd(dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), dx.data_ptr(),
                     dB.data_ptr(), dC.data_ptr(), dh.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl, code,
                     (int32_t)algo, stream_of(x)),
             "gcg_bwd");
    return {dx, dB, dC, dh};
}

// ---- gated convolution on the interleaved features tensor ------------------------------------

Tensor fwd_interleaved(const Tensor &feat, const Tensor &h, int64_t algo)
{
    require_gpu(feat, "feat");
    check_feat(feat, h);
    DeviceGuard guard(feat.device());
    Tensor y = at::empty({feat.size(0), feat.size(1), feat.size(2), feat.size(3)}, feat.options());
    if (y.numel() == 0) return y;
    check_rc(gcg_fwd_interleaved(feat.data_ptr(), h.data_ptr(), y.data_ptr(), feat.size(0), feat.size(1),
                                 (int32_t)feat.size(2), (int32_t)feat.size(3), (int32_t)h.size(2),
                                 gated_code(feat, h), (int32_t)algo, stream_of(feat)),
             "gcg_fwd_interleaved");
    return y;
}

std::tuple<Tensor, Tensor> bwd_interleaved(const Tensor &dy, const Tensor &feat, const Tensor &h, int64_t algo,
                                           bool keep_output)
{
    require_gpu(feat, "feat");
    check_feat(feat, h);
    TORCH_CHECK(dy.dim() == 4 && dy.sizes() == feat.sizes().slice(0, 4) && dy.scalar_type() == feat.scalar_type() &&
                    dy.device() == feat.device() && dy.is_contiguous(),
                "gcg: dy must be a contiguous (bs, L, g, dg) tensor of feat's dtype and device");
    DeviceGuard guard(feat.device());
    Tensor dfeat = at::empty_like(feat), dh = at::empty_like(h);
    if (dy.numel() == 0) return {dfeat, dh.zero_()};
    const int64_t bs = feat.size(0), L = feat.size(1);
    const int32_t g = (int32_t)feat.size(2), dg = (int32_t)feat.size(3), hl = (int32_t)h.size(2);
    const int code = gated_code(feat, h);
    const size_t nbytes = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, (int32_t)algo);
    Tensor ws = workspace(nbytes, feat, "gcg_bwd_workspace_bytes");
    check_rc(gcg_bwd_interleaved(dy.data_ptr(), feat.data_ptr(), h.data_ptr(), dfeat.data_ptr(), dh.data_ptr(),
                                 ws.data_ptr(), nbytes, bs, L, g, dg, hl, code, (int32_t)algo,
                                 keep_output ? GCG_KEEP_OUTPUT : 0, stream_of(feat)),
             "gcg_bwd_interleaved");
    return {dfeat, dh};
}

// ---- gated convolution on the planar features tensor (bs, L, 3, g, dg) ---------------------------

void check_planar(const Tensor &feat, const Tensor &h)
{
    TORCH_CHECK(feat.dim() == 5 && feat.size(2) == 3 && feat.is_contiguous(),
                "gcg: feat must be a contiguous (bs, L, 3, g, dg) tensor");
    TORCH_CHECK(h.dim() == 3 && h.size(0) == feat.size(3) && h.size(1) == 1 && h.is_contiguous(),
                "gcg: h must be a contiguous (g, 1, hl) tensor");
    TORCH_CHECK(h.device() == feat.device(), "gcg: feat and h must be on one device");
    (void)gated_code(feat, h);
}

Tensor fwd_planar(const Tensor &feat, const Tensor &h, int64_t algo)
{
    require_gpu(feat, "feat");
    check_planar(feat, h);
    DeviceGuard guard(feat.device());
    Tensor y = at::empty({feat.size(0), feat.size(1), feat.size(3), feat.size(4)}, feat.options());
    if (y.numel() == 0) return y;
    check_rc(gcg_fwd_planar(feat.data_ptr(), h.data_ptr(), y.data_ptr(), feat.size(0), feat.size(1),
                            (int32_t)feat.size(3), (int32_t)feat.size(4), (int32_t)h.size(2), gated_code(feat, h),
                            (int32_t)algo, stream_of(feat)),
             "gcg_fwd_planar");
    return y;
}

std::tuple<Tensor, Tensor> bwd_planar(const Tensor &dy, const Tensor &feat, const Tensor &h, int64_t algo)
{
    require_gpu(feat, "feat");
    check_planar(feat, h);
    TORCH_CHECK(dy.dim() == 4 && dy.size(0) == feat.size(0) && dy.size(1) == feat.size(1) && dy.size(2) == feat.size(3) &&
                    dy.size(3) == feat.size(4) && dy.scalar_type() == feat.scalar_type() && dy.device() == feat.device() &&
                    dy.is_contiguous(),
                "gcg: dy must be a contiguous (bs, L, g, dg) tensor of feat's dtype and device");
    DeviceGuard guard(feat.device());
    Tensor dfeat = at::empty_like(feat), dh = at::empty_like(h);
    if (dy.numel() == 0) return {dfeat, dh.zero_()};
    const int64_t bs = feat.size(0), L = feat.size(1);
    const int32_t g = (int32_t)feat.size(3), dg = (int32_t)feat.size(4), hl = (int32_t)h.size(2);
    const int code = gated_code(feat, h);
    const size_t nbytes = gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, (int32_t)algo);
    Tensor ws = workspace(nbytes, feat, "gcg_bwd_workspace_bytes");
    check_rc(gcg_bwd_planar(dy.data_ptr(), feat.data_ptr(), h.data_ptr(), dfeat.data_ptr(), dh.data_ptr(), ws.data_ptr(),
                            nbytes, bs, L, g, dg, hl, code, (int32_t)algo, stream_of(feat)),
             "gcg_bwd_planar");
    return {dfeat, dh};
}

// ---- featurizer convolution -------------------------------------------------------------------

void check_dwconv(const Tensor &x, const Tensor &w)
{
    TORCH_CHECK(x.dim() == 4 && x.is_contiguous(), "gcg: x must be a contiguous (bs, L, g, dg) tensor");
    TORCH_CHECK(w.dim() == 3 && w.size(0) == x.size(2) && w.size(1) == 1 && w.is_contiguous(),
                "gcg: w must be a contiguous (g, 1, hl) tensor");
    TORCH_CHECK(w.scalar_type() == x.scalar_type() && w.device() == x.device(),
                "gcg: x and w must share dtype and device");
}

Tensor dwconv_fwd(const Tensor &x, const Tensor &w, bool keep_output)
{
    require_gpu(x, "x");
    check_dwconv(x, w);
    DeviceGuard guard(x.device());
    Tensor y = at::empty_like(x);
    if (x.numel() == 0) return y;
    check_rc(gcg_dwconv_fwd(x.data_ptr(), w.data_ptr(), y.data_ptr(), x.size(0), x.size(1), (int32_t)x.size(2),
                            (int32_t)x.size(3), (int32_t)w.size(2), dtype_code(x.scalar_type()),
                            keep_output ? GCG_KEEP_OUTPUT : 0, stream_of(x)),
             "gcg_dwconv_fwd");
    return y;
}

std::tuple<Tensor, Tensor> dwconv_bwd(const Tensor &dy, const Tensor &x, const Tensor &w)
{
    require_gpu(x, "x");
    check_dwconv(x, w);
    check_like(dy, x, "dy");
    DeviceGuard guard(x.device());
    Tensor dx = at::empty_like(x), dw = at::empty_like(w);
    if (x.numel() == 0) return {dx, dw.zero_()};
    const int64_t bs = x.size(0), L = x.size(1);
    const int32_t g = (int32_t)x.size(2), dg = (int32_t)x.size(3), hl = (int32_t)w.size(2);
    const int code = dtype_code(x.scalar_type());
    const size_t nbytes = gcg_dwconv_bwd_workspace_bytes(bs, L, g, dg, hl, code);
    if (nbytes == 0) check_rc(GCG_ERR_UNSUPPORTED, "gcg_dwconv_bwd_workspace_bytes");
    Tensor ws = workspace(nbytes, x, "gcg_dwconv_bwd_workspace_bytes");
    check_rc(gcg_dwconv_bwd(dy.data_ptr(), x.data_ptr(), w.data_ptr(), dx.data_ptr(), dw.data_ptr(), ws.data_ptr(),
                            nbytes, bs, L, g, dg, hl, code, stream_of(x)),
             "gcg_dwconv_bwd");
    return {dx, dw};
}

// ---- featurizer + Hyena-SE operator in one pass ------------------------------------------------

// planar: raw is (bs, L, 3, g, dg) -- the planes C | B | x of each row one after the other -- instead of (bs, L, g, dg, 3)
void check_mixer_se(const Tensor &raw, const Tensor &wf, const Tensor &h, bool planar = false)
{
    TORCH_CHECK(raw.dim() == 5 && raw.size(planar ? 2 : 4) == 3 && raw.is_contiguous(),
                planar ? "gcg: raw must be a contiguous (bs, L, 3, g, dg) tensor"
                       : "gcg: raw must be a contiguous (bs, L, g, dg, 3) tensor");
    const int64_t g = raw.size(planar ? 3 : 2), dg = raw.size(planar ? 4 : 3);
    TORCH_CHECK(wf.dim() == 3 && wf.size(0) == 3 * g * dg && wf.size(1) == 1 && wf.is_contiguous(),
                "gcg: wf must be a contiguous (3 * g * dg, 1, kf) tensor");
    TORCH_CHECK(h.dim() == 3 && h.size(0) == g && h.size(1) == 1 && h.is_contiguous(),
                "gcg: h must be a contiguous (g, 1, hl) tensor");
    TORCH_CHECK(wf.scalar_type() == raw.scalar_type() && wf.device() == raw.device() && h.device() == raw.device(),
                "gcg: raw and wf must share dtype, and raw, wf and h their device");
    (void)gated_code(raw, h);       // h of raw's dtype, or fp32 with 16-bit raw (fp32 arithmetic)
}

Tensor mixer_se_fwd(const Tensor &raw, const Tensor &wf, const Tensor &h, bool planar)
{
    require_gpu(raw, "raw");
    check_mixer_se(raw, wf, h, planar);
    DeviceGuard guard(raw.device());
    const int64_t g = raw.size(planar ? 3 : 2), dg = raw.size(planar ? 4 : 3);
    Tensor y = at::empty({raw.size(0), raw.size(1), g, dg}, raw.options());
    if (y.numel() == 0) return y;
    check_rc((planar ? gcg_mixer_se_fwd_planar : gcg_mixer_se_fwd)(
                 raw.data_ptr(), wf.data_ptr(), h.data_ptr(), y.data_ptr(), raw.size(0), raw.size(1), (int32_t)g,
                 (int32_t)dg, (int32_t)h.size(2), (int32_t)wf.size(2), gated_code(raw, h), stream_of(raw)),
             planar ? "gcg_mixer_se_fwd_planar" : "gcg_mixer_se_fwd");
    return y;
}

std::tuple<Tensor, Tensor, Tensor> mixer_se_bwd(const Tensor &dy, const Tensor &raw, const Tensor &wf, const Tensor &h,
                                                bool planar)
{
    require_gpu(raw, "raw");
    check_mixer_se(raw, wf, h, planar);
    const int32_t g = (int32_t)raw.size(planar ? 3 : 2), dg = (int32_t)raw.size(planar ? 4 : 3);
    TORCH_CHECK(dy.dim() == 4 && dy.size(0) == raw.size(0) && dy.size(1) == raw.size(1) && dy.size(2) == g &&
                    dy.size(3) == dg && dy.scalar_type() == raw.scalar_type() && dy.device() == raw.device() &&
                    dy.is_contiguous(),
                "gcg: dy must be a contiguous (bs, L, g, dg) tensor of raw's dtype and device");
    DeviceGuard guard(raw.device());
    Tensor draw = at::empty_like(raw), dwf = at::empty_like(wf), dh = at::empty_like(h);
    if (raw.numel() == 0) return {draw, dwf.zero_(), dh.zero_()};
    const int64_t bs = raw.size(0), L = raw.size(1);
    const int32_t hl = (int32_t)h.size(2), kf = (int32_t)wf.size(2);
    const int code = gated_code(raw, h);
    const size_t nbytes = gcg_mixer_se_bwd_workspace_bytes(bs, L, g, dg, hl, kf, code);
    if (nbytes == 0) check_rc(GCG_ERR_UNSUPPORTED, "gcg_mixer_se_bwd_workspace_bytes");
    Tensor ws = workspace(nbytes, raw, "gcg_mixer_se_bwd_workspace_bytes");
    check_rc((planar ? gcg_mixer_se_bwd_planar : gcg_mixer_se_bwd)(
                 dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), h.data_ptr(), draw.data_ptr(), dwf.data_ptr(),
                 dh.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl, kf, code, stream_of(raw)),
             planar ? "gcg_mixer_se_bwd_planar" : "gcg_mixer_se_bwd");
    return {draw, dwf, dh};
}

// ---- explicit decayed filter ---------------------------------------------------------------------

void check_filter_params(const Tensor &w, const Tensor &decay)
{
    TORCH_CHECK(w.dim() == 2 && decay.dim() == 2 && w.scalar_type() == at::kFloat && decay.scalar_type() == at::kFloat &&
                    w.is_contiguous() && decay.is_contiguous(),
                "gcg: w and decay must be contiguous fp32 (g, L_cache) tensors");
    TORCH_CHECK(w.sizes() == decay.sizes() && w.device() == decay.device(), "gcg: w and decay must share shape and device");
}

Tensor filter_decay_fwd(const Tensor &w, const Tensor &decay, int64_t hl, at::ScalarType dtype)
{
    require_gpu(w, "w");
    check_filter_params(w, decay);
    TORCH_CHECK(hl > 0 && hl <= w.size(1), "gcg: hl must be in 1..L_cache");
    DeviceGuard guard(w.device());
    Tensor h = at::empty({w.size(0), 1, hl}, w.options().dtype(dtype));
    check_rc(gcg_filter_decay_fwd((const float *)w.data_ptr(), (const float *)decay.data_ptr(), h.data_ptr(),
                                  (int32_t)w.size(0), (int32_t)w.size(1), (int32_t)hl, dtype_code(dtype), stream_of(w)),
             "gcg_filter_decay_fwd");
    return h;
}

Tensor filter_decay_bwd(const Tensor &dh, const Tensor &decay)
{
    require_gpu(dh, "dh");
    check_filter_params(decay, decay);
    TORCH_CHECK(dh.dim() == 3 && dh.size(0) == decay.size(0) && dh.size(1) == 1 && dh.size(2) <= decay.size(1) &&
                    dh.is_contiguous() && dh.device() == decay.device(),
                "gcg: dh must be a contiguous (g, 1, hl) tensor with hl <= L_cache on decay's device");
    DeviceGuard guard(dh.device());
    Tensor dw = at::empty_like(decay);
    check_rc(gcg_filter_decay_bwd(dh.data_ptr(), (const float *)decay.data_ptr(), (float *)dw.data_ptr(),
                                  (int32_t)decay.size(0), (int32_t)decay.size(1), (int32_t)dh.size(2),
                                  dtype_code(dh.scalar_type()), stream_of(dh)),
             "gcg_filter_decay_bwd");
    return dw;
}

// ---- gated convolution with the decayed explicit filter built inside the kernels ---------------

// dtype code for tensors of type t with a filter of element type filt
int gated_code_for(at::ScalarType t, at::ScalarType filt)
{
    if (filt == t) return dtype_code(t);
    TORCH_CHECK(filt == at::kFloat && (t == at::kBFloat16 || t == at::kHalf),
                "gcg: the filter must have the tensors' dtype, or be float32 with bfloat16 / float16 tensors; got ", t,
                " tensors and a ", filt, " filter");
    return t == at::kBFloat16 ? GCG_BF16_F32 : GCG_F16_F32;
}

void check_decay(const Tensor &w, const Tensor &decay, int64_t hl, int64_t g, const Tensor &on)
{
    check_filter_params(w, decay);
    TORCH_CHECK(w.size(0) == g && hl > 0 && hl <= w.size(1) && w.device() == on.device(),
                "gcg: w and decay must be (g, L_cache) on the tensors' device with 0 < hl <= L_cache");
}

void check_xbc(const Tensor &x, const Tensor &B, const Tensor &C)
{
    TORCH_CHECK(x.dim() == 4 && B.sizes() == x.sizes() && C.sizes() == x.sizes(), "gcg: x, B and C must be (bs, L, g, dg) of one shape");
    TORCH_CHECK(B.scalar_type() == x.scalar_type() && C.scalar_type() == x.scalar_type() && B.device() == x.device() &&
                    C.device() == x.device() && x.is_contiguous() && B.is_contiguous() && C.is_contiguous(),
                "gcg: x, B and C must be contiguous and share one dtype and device");
}

Tensor fwd_decay(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &w, const Tensor &decay, int64_t hl,
                 at::ScalarType filt)
{
    require_gpu(x, "x");
    check_xbc(x, B, C);
    check_decay(w, decay, hl, x.size(2), x);
    const int code = gated_code_for(x.scalar_type(), filt);
    DeviceGuard guard(x.device());
    Tensor y = at::empty_like(x);
    if (x.numel() == 0) return y;
    check_rc(gcg_fwd_decay(x.data_ptr(), B.data_ptr(), C.data_ptr(), (const float *)w.data_ptr(),
                           (const float *)decay.data_ptr(), (int32_t)w.size(1), y.data_ptr(), x.size(0), x.size(1),
                           (int32_t)x.size(2), (int32_t)x.size(3), (int32_t)hl, code, stream_of(x)),
             "gcg_fwd_decay");
    return y;
}

std::tuple<Tensor, Tensor, Tensor, Tensor> bwd_decay(const Tensor &dy, const Tensor &x, const Tensor &B, const Tensor &C,
                                                     const Tensor &w, const Tensor &decay, int64_t hl,
                                                     at::ScalarType filt)
{
    require_gpu(x, "x");
    check_xbc(x, B, C);
    check_like(dy, x, "dy");
    check_decay(w, decay, hl, x.size(2), x);
    const int code = gated_code_for(x.scalar_type(), filt);
    DeviceGuard guard(x.device());
    Tensor dx = at::empty_like(x), dB = at::empty_like(x), dC = at::empty_like(x), dw = at::empty_like(w);
    if (x.numel() == 0) return {dx, dB, dC, dw.zero_()};
    const int64_t bs = x.size(0), L = x.size(1);
    const int32_t g = (int32_t)x.size(2), dg = (int32_t)x.size(3);
    const size_t nbytes = gcg_bwd_workspace_bytes(bs, L, g, dg, (int32_t)hl, code, GCG_ALGO_MFMA);
    Tensor ws = workspace(nbytes, x, "gcg_bwd_workspace_bytes");
    check_rc(gcg_bwd_decay(dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), (const float *)w.data_ptr(),
                           (const float *)decay.data_ptr(), (int32_t)w.size(1), dx.data_ptr(), dB.data_ptr(),
                           dC.data_ptr(), (float *)dw.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, (int32_t)hl,
                           code, stream_of(x)),
             "gcg_bwd_decay");
    return {dx, dB, dC, dw};
}

void check_feat_only(const Tensor &feat)
{
    TORCH_CHECK(feat.dim() == 5 && feat.size(4) == 3 && feat.is_contiguous(),
                "gcg: feat must be a contiguous (bs, L, g, dg, 3) tensor");
}

Tensor fwd_interleaved_decay(const Tensor &feat, const Tensor &w, const Tensor &decay, int64_t hl, at::ScalarType filt)
{
    require_gpu(feat, "feat");
    check_feat_only(feat);
    check_decay(w, decay, hl, feat.size(2), feat);
    const int code = gated_code_for(feat.scalar_type(), filt);
    DeviceGuard guard(feat.device());
    Tensor y = at::empty({feat.size(0), feat.size(1), feat.size(2), feat.size(3)}, feat.options());
    if (y.numel() == 0) return y;
    check_rc(gcg_fwd_interleaved_decay(feat.data_ptr(), (const float *)w.data_ptr(), (const float *)decay.data_ptr(),
                                       (int32_t)w.size(1), y.data_ptr(), feat.size(0), feat.size(1),
                                       (int32_t)feat.size(2), (int32_t)feat.size(3), (int32_t)hl, code,
                                       stream_of(feat)),
             "gcg_fwd_interleaved_decay");
    return y;
}

std::tuple<Tensor, Tensor> bwd_interleaved_decay(const Tensor &dy, const Tensor &feat, const Tensor &w,
                                                 const Tensor &decay, int64_t hl, at::ScalarType filt, bool keep_output)
{
    require_gpu(feat, "feat");
    check_feat_only(feat);
    check_decay(w, decay, hl, feat.size(2), feat);
    TORCH_CHECK(dy.dim() == 4 && dy.sizes() == feat.sizes().slice(0, 4) && dy.scalar_type() == feat.scalar_type() &&
                    dy.device() == feat.device() && dy.is_contiguous(),
                "gcg: dy must be a contiguous (bs, L, g, dg) tensor of feat's dtype and device");
    const int code = gated_code_for(feat.scalar_type(), filt);
    DeviceGuard guard(feat.device());
    Tensor dfeat = at::empty_like(feat), dw = at::empty_like(w);
    if (dy.numel() == 0) return {dfeat, dw.zero_()};
    const int64_t bs = feat.size(0), L = feat.size(1);
    const int32_t g = (int32_t)feat.size(2), dg = (int32_t)feat.size(3);
    const size_t nbytes = gcg_bwd_workspace_bytes(bs, L, g, dg, (int32_t)hl, code, GCG_ALGO_MFMA);
    Tensor ws = workspace(nbytes, feat, "gcg_bwd_workspace_bytes");
    check_rc(gcg_bwd_interleaved_decay(dy.data_ptr(), feat.data_ptr(), (const float *)w.data_ptr(),
                                       (const float *)decay.data_ptr(), (int32_t)w.size(1), dfeat.data_ptr(),
                                       (float *)dw.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, (int32_t)hl, code,
                                       keep_output ? GCG_KEEP_OUTPUT : 0, stream_of(feat)),
             "gcg_bwd_interleaved_decay");
    return {dfeat, dw};
}

// ---- short-filter operator on time-major operands (seqlen, bs, g, dg) --------------------------

void check_time_major(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h)
{
    TORCH_CHECK(x.dim() == 4 && B.sizes() == x.sizes() && C.sizes() == x.sizes(),
                "gcg: x, B and C must be (seqlen, bs, g, dg) of one shape");
    TORCH_CHECK(h.dim() == 3 && h.size(0) == x.size(2) && h.size(1) == 1 && h.is_contiguous(), "gcg: h must be a contiguous (g, 1, hl) tensor");
    TORCH_CHECK(B.scalar_type() == x.scalar_type() && C.scalar_type() == x.scalar_type() && B.device() == x.device() &&
                    C.device() == x.device() && h.device() == x.device() && x.is_contiguous() && B.is_contiguous() &&
                    C.is_contiguous(),
                "gcg: x, B and C must be contiguous and share one dtype and device");
}

Tensor fwd_time_major(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h)
{
    require_gpu(x, "x");
    check_time_major(x, B, C, h);
    const int code = gated_code(x, h);
    DeviceGuard guard(x.device());
    Tensor y = at::empty({x.size(1), x.size(0), x.size(2), x.size(3)}, x.options());
    if (x.numel() == 0) return y;
    check_rc(gcg_fwd_time_major(x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), y.data_ptr(), x.size(1),
                                x.size(0), (int32_t)x.size(2), (int32_t)x.size(3), (int32_t)h.size(2), code,
                                stream_of(x)),
             "gcg_fwd_time_major");
    return y;
}

std::tuple<Tensor, Tensor, Tensor, Tensor> bwd_time_major(const Tensor &dy, const Tensor &x, const Tensor &B,
                                                          const Tensor &C, const Tensor &h)
{
    require_gpu(x, "x");
    check_time_major(x, B, C, h);
    TORCH_CHECK(dy.dim() == 4 && dy.size(0) == x.size(1) && dy.size(1) == x.size(0) && dy.size(2) == x.size(2) &&
                    dy.size(3) == x.size(3) && dy.scalar_type() == x.scalar_type() && dy.device() == x.device() &&
                    dy.is_contiguous(),
                "gcg: dy must be a contiguous (bs, seqlen, g, dg) tensor of x's dtype and device");
    const int code = gated_code(x, h);
    DeviceGuard guard(x.device());
    Tensor dx = at::empty_like(x), dB = at::empty_like(x), dC = at::empty_like(x), dh = at::empty_like(h);
    if (x.numel() == 0) return {dx, dB, dC, dh.zero_()};
    const int64_t L = x.size(0), bs = x.size(1);
    const int32_t g = (int32_t)x.size(2), dg = (int32_t)x.size(3), hl = (int32_t)h.size(2);
    const size_t nbytes = gcg_bwd_time_major_workspace_bytes(bs, L, g, dg, hl, code);
    Tensor ws = workspace(nbytes, x, "gcg_bwd_time_major_workspace_bytes");
    check_rc(gcg_bwd_time_major(dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), dx.data_ptr(),
                                dB.data_ptr(), dC.data_ptr(), dh.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl,
                                code, stream_of(x)),
             "gcg_bwd_time_major");
    return {dx, dB, dC, dh};
}

// ---- featurizer and Hyena-MR operator without the featurized tensor ----------------------------

// planar: raw is (bs, L, 3, g, dg) -- the planes C | B | x of each row one after the other -- instead of (bs, L, g, dg, 3)
void check_mixer_mr(const Tensor &raw, const Tensor &wf, const Tensor &h, bool planar = false)
{
    TORCH_CHECK(raw.dim() == 5 && raw.size(planar ? 2 : 4) == 3 && raw.is_contiguous(),
                planar ? "gcg: raw must be a contiguous (bs, L, 3, g, dg) tensor"
                       : "gcg: raw must be a contiguous (bs, L, g, dg, 3) tensor");
    const int64_t g = raw.size(planar ? 3 : 2), dg = raw.size(planar ? 4 : 3);
    TORCH_CHECK(wf.dim() == 3 && wf.size(0) == 3 * g * dg && wf.size(1) == 1 && wf.is_contiguous() &&
                    wf.scalar_type() == raw.scalar_type(),
                "gcg: wf must be a contiguous (3 * g * dg, 1, kf) tensor of raw's dtype");
    TORCH_CHECK(h.dim() == 3 && h.size(0) == g && h.size(1) == 1 && h.is_contiguous(),
                "gcg: h must be a contiguous (g, 1, hl) tensor");
    TORCH_CHECK(wf.device() == raw.device() && h.device() == raw.device(), "gcg: raw, wf and h must be on one device");
    (void)gated_code(raw, h);
}

void check_mixer_mr_decay(const Tensor &raw, const Tensor &wf, const Tensor &w, const Tensor &decay, int64_t hl,
                          bool planar = false)
{
    TORCH_CHECK(raw.dim() == 5 && raw.size(planar ? 2 : 4) == 3 && raw.is_contiguous(),
                planar ? "gcg: raw must be a contiguous (bs, L, 3, g, dg) tensor"
                       : "gcg: raw must be a contiguous (bs, L, g, dg, 3) tensor");
    const int64_t g = raw.size(planar ? 3 : 2), dg = raw.size(planar ? 4 : 3);
    TORCH_CHECK(wf.dim() == 3 && wf.size(0) == 3 * g * dg && wf.size(1) == 1 && wf.is_contiguous() &&
                    wf.scalar_type() == raw.scalar_type() && wf.device() == raw.device(),
                "gcg: wf must be a contiguous (3 * g * dg, 1, kf) tensor of raw's dtype and device");
    check_decay(w, decay, hl, g, raw);
}

Tensor mixer_mr_fwd_decay(const Tensor &raw, const Tensor &wf, const Tensor &w, const Tensor &decay, int64_t hl,
                          at::ScalarType filt, bool planar)
{
    require_gpu(raw, "raw");
    check_mixer_mr_decay(raw, wf, w, decay, hl, planar);
    const int code = gated_code_for(raw.scalar_type(), filt);
    DeviceGuard guard(raw.device());
    const int64_t g = raw.size(planar ? 3 : 2), dg = raw.size(planar ? 4 : 3);
    Tensor y = at::empty({raw.size(0), raw.size(1), g, dg}, raw.options());
    if (y.numel() == 0) return y;
    check_rc((planar ? gcg_mixer_mr_fwd_planar_decay : gcg_mixer_mr_fwd_decay)(
                 raw.data_ptr(), wf.data_ptr(), (const float *)w.data_ptr(), (const float *)decay.data_ptr(),
                 (int32_t)w.size(1), y.data_ptr(), raw.size(0), raw.size(1), (int32_t)g, (int32_t)dg, (int32_t)hl,
                 (int32_t)wf.size(2), code, stream_of(raw)),
             planar ? "gcg_mixer_mr_fwd_planar_decay" : "gcg_mixer_mr_fwd_decay");
    return y;
}

std::tuple<Tensor, Tensor, Tensor> mixer_mr_bwd_decay(const Tensor &dy, const Tensor &raw, const Tensor &wf,
                                                      const Tensor &w, const Tensor &decay, int64_t hl,
                                                      at::ScalarType filt, bool planar)
{
    require_gpu(raw, "raw");
    check_mixer_mr_decay(raw, wf, w, decay, hl, planar);
    const int32_t g = (int32_t)raw.size(planar ? 3 : 2), dg = (int32_t)raw.size(planar ? 4 : 3), kf = (int32_t)wf.size(2);
    TORCH_CHECK(dy.dim() == 4 && dy.size(0) == raw.size(0) && dy.size(1) == raw.size(1) && dy.size(2) == g &&
                    dy.size(3) == dg && dy.scalar_type() == raw.scalar_type() && dy.device() == raw.device() &&
                    dy.is_contiguous(),
                "gcg: dy must be a contiguous (bs, L, g, dg) tensor of raw's dtype and device");
    const int code = gated_code_for(raw.scalar_type(), filt);
    DeviceGuard guard(raw.device());
    Tensor draw = at::empty_like(raw), dwf = at::empty_like(wf), dw = at::empty_like(w);
    if (dy.numel() == 0) return {draw, dwf.zero_(), dw.zero_()};
    const int64_t bs = raw.size(0), L = raw.size(1);
    const size_t nbytes = gcg_mixer_mr_bwd_workspace_bytes(bs, L, g, dg, (int32_t)hl, kf, code);
    Tensor ws = workspace(nbytes, raw, "gcg_mixer_mr_bwd_workspace_bytes");
    if (planar) {
        check_rc(gcg_mixer_mr_bwd_planar_decay(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), (const float *)w.data_ptr(),
                                               (const float *)decay.data_ptr(), (int32_t)w.size(1), draw.data_ptr(),
                                               dwf.data_ptr(), (float *)dw.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg,
                                               (int32_t)hl, kf, code, stream_of(raw)),
                 "gcg_mixer_mr_bwd_planar_decay");
        return {draw, dwf, dw};
    }
    const size_t sbytes = gcg_mixer_mr_bwd_scratch_bytes(bs, L, g, dg, (int32_t)hl, kf, code);
    Tensor scratch = at::empty({(int64_t)sbytes}, raw.options().dtype(at::kByte));
    check_rc(gcg_mixer_mr_bwd_decay(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), (const float *)w.data_ptr(),
                                    (const float *)decay.data_ptr(), (int32_t)w.size(1), draw.data_ptr(), dwf.data_ptr(),
                                    (float *)dw.data_ptr(), scratch.numel() ? scratch.data_ptr() : nullptr, ws.data_ptr(),
                                    nbytes, bs, L, g, dg, (int32_t)hl, kf, code, stream_of(raw)),
             "gcg_mixer_mr_bwd_decay");
    return {draw, dwf, dw};
}

Tensor mixer_mr_fwd(const Tensor &raw, const Tensor &wf, const Tensor &h, bool planar)
{
    require_gpu(raw, "raw");
    check_mixer_mr(raw, wf, h, planar);
    DeviceGuard guard(raw.device());
    const int64_t g = raw.size(planar ? 3 : 2), dg = raw.size(planar ? 4 : 3);
    Tensor y = at::empty({raw.size(0), raw.size(1), g, dg}, raw.options());
    if (y.numel() == 0) return y;
    check_rc((planar ? gcg_mixer_mr_fwd_planar : gcg_mixer_mr_fwd)(
                 raw.data_ptr(), wf.data_ptr(), h.data_ptr(), y.data_ptr(), raw.size(0), raw.size(1), (int32_t)g,
                 (int32_t)dg, (int32_t)h.size(2), (int32_t)wf.size(2), gated_code(raw, h), stream_of(raw)),
             planar ? "gcg_mixer_mr_fwd_planar" : "gcg_mixer_mr_fwd");
    return y;
}

std::tuple<Tensor, Tensor, Tensor> mixer_mr_bwd(const Tensor &dy, const Tensor &raw, const Tensor &wf, const Tensor &h,
                                                bool planar)
{
    require_gpu(raw, "raw");
    check_mixer_mr(raw, wf, h, planar);
    const int32_t g = (int32_t)raw.size(planar ? 3 : 2), dg = (int32_t)raw.size(planar ? 4 : 3);
    TORCH_CHECK(dy.dim() == 4 && dy.size(0) == raw.size(0) && dy.size(1) == raw.size(1) && dy.size(2) == g &&
                    dy.size(3) == dg && dy.scalar_type() == raw.scalar_type() && dy.device() == raw.device() &&
                    dy.is_contiguous(),
                "gcg: dy must be a contiguous (bs, L, g, dg) tensor of raw's dtype and device");
    DeviceGuard guard(raw.device());
    Tensor draw = at::empty_like(raw), dwf = at::empty_like(wf), dh = at::empty_like(h);
    if (dy.numel() == 0) return {draw, dwf.zero_(), dh.zero_()};
    const int64_t bs = raw.size(0), L = raw.size(1);
    const int32_t hl = (int32_t)h.size(2), kf = (int32_t)wf.size(2);
    const int code = gated_code(raw, h);
    const size_t nbytes = gcg_mixer_mr_bwd_workspace_bytes(bs, L, g, dg, hl, kf, code);
    Tensor ws = workspace(nbytes, raw, "gcg_mixer_mr_bwd_workspace_bytes");
    if (planar) {
        check_rc(gcg_mixer_mr_bwd_planar(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), h.data_ptr(), draw.data_ptr(),
                                         dwf.data_ptr(), dh.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl, kf, code,
                                         stream_of(raw)),
                 "gcg_mixer_mr_bwd_planar");
        return {draw, dwf, dh};
    }
    // gradient of the featurized features, for the duration of the call (not needed where one kernel does it all)
    const size_t sbytes = gcg_mixer_mr_bwd_scratch_bytes(bs, L, g, dg, hl, kf, code);
    Tensor scratch = at::empty({(int64_t)sbytes}, raw.options().dtype(at::kByte));
    check_rc(gcg_mixer_mr_bwd(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), h.data_ptr(), draw.data_ptr(),
                              dwf.data_ptr(), dh.data_ptr(), scratch.numel() ? scratch.data_ptr() : nullptr,
                              ws.data_ptr(), nbytes, bs, L, g, dg, hl,
                              kf, code, stream_of(raw)),
             "gcg_mixer_mr_bwd");
    return {draw, dwf, dh};
}

// ---- meta implementations: shapes and dtypes only (fake tensors, torch.compile) ----------------

std::tuple<Tensor, Tensor, Tensor> fwd_full_meta(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h,
                                                 bool return_bx, bool return_y2, int64_t)
{
    check_gated(x, B, C, h);
    return {return_bx ? at::empty_like(x) : at::empty({0}, x.options()),
            return_y2 ? at::empty_like(x) : at::empty({0}, x.options()), at::empty_like(x)};
}
Tensor fwd_meta(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h, int64_t)
{
    check_gated(x, B, C, h);
    return at::empty_like(x);
}
void fwd_out_meta(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h, Tensor &y, int64_t)
{
    check_gated(x, B, C, h);
    check_like(y, x, "out");
}
std::tuple<Tensor, Tensor, Tensor, Tensor> bwd_meta(const Tensor &dy, const Tensor &x, const Tensor &B, const Tensor &C,
                                                    const Tensor &h, int64_t)
{
    check_gated(x, B, C, h);
    check_like(dy, x, "dy");
    return {at::empty_like(x), at::empty_like(x), at::empty_like(x), at::empty_like(h)};
}
Tensor fwd_interleaved_meta(const Tensor &feat, const Tensor &h, int64_t)
{
    check_feat(feat, h);
    return at::empty({feat.size(0), feat.size(1), feat.size(2), feat.size(3)}, feat.options());
}
std::tuple<Tensor, Tensor> bwd_interleaved_meta(const Tensor &dy, const Tensor &feat, const Tensor &h, int64_t, bool)
{
    check_feat(feat, h);
    (void)dy;
    return {at::empty_like(feat), at::empty_like(h)};
}
Tensor fwd_planar_meta(const Tensor &feat, const Tensor &h, int64_t)
{
    check_planar(feat, h);
    return at::empty({feat.size(0), feat.size(1), feat.size(3), feat.size(4)}, feat.options());
}
std::tuple<Tensor, Tensor> bwd_planar_meta(const Tensor &dy, const Tensor &feat, const Tensor &h, int64_t)
{
    check_planar(feat, h);
    (void)dy;
    return {at::empty_like(feat), at::empty_like(h)};
}
Tensor dwconv_fwd_meta(const Tensor &x, const Tensor &w, bool)
{
    check_dwconv(x, w);
    return at::empty_like(x);
}
std::tuple<Tensor, Tensor> dwconv_bwd_meta(const Tensor &dy, const Tensor &x, const Tensor &w)
{
    check_dwconv(x, w);
    check_like(dy, x, "dy");
    return {at::empty_like(x), at::empty_like(w)};
}
Tensor mixer_se_fwd_meta(const Tensor &raw, const Tensor &wf, const Tensor &h, bool planar)
{
    check_mixer_se(raw, wf, h, planar);
    return at::empty({raw.size(0), raw.size(1), raw.size(planar ? 3 : 2), raw.size(planar ? 4 : 3)}, raw.options());
}
std::tuple<Tensor, Tensor, Tensor> mixer_se_bwd_meta(const Tensor &dy, const Tensor &raw, const Tensor &wf,
                                                     const Tensor &h, bool planar)
{
    check_mixer_se(raw, wf, h, planar);
    (void)dy;
    return {at::empty_like(raw), at::empty_like(wf), at::empty_like(h)};
}
Tensor filter_decay_fwd_meta(const Tensor &w, const Tensor &decay, int64_t hl, at::ScalarType dtype)
{
    check_filter_params(w, decay);
    TORCH_CHECK(hl > 0 && hl <= w.size(1), "gcg: hl must be in 1..L_cache");
    return at::empty({w.size(0), 1, hl}, w.options().dtype(dtype));
}
Tensor filter_decay_bwd_meta(const Tensor &dh, const Tensor &decay)
{
    (void)dh;
    check_filter_params(decay, decay);
    return at::empty_like(decay);
}

Tensor fwd_decay_meta(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &w, const Tensor &decay,
                      int64_t hl, at::ScalarType filt)
{
    check_xbc(x, B, C);
    check_decay(w, decay, hl, x.size(2), x);
    (void)gated_code_for(x.scalar_type(), filt);
    return at::empty_like(x);
}
std::tuple<Tensor, Tensor, Tensor, Tensor> bwd_decay_meta(const Tensor &dy, const Tensor &x, const Tensor &B,
                                                          const Tensor &C, const Tensor &w, const Tensor &decay,
                                                          int64_t hl, at::ScalarType filt)
{
    check_xbc(x, B, C);
    check_like(dy, x, "dy");
    check_decay(w, decay, hl, x.size(2), x);
    (void)gated_code_for(x.scalar_type(), filt);
    return {at::empty_like(x), at::empty_like(x), at::empty_like(x), at::empty_like(w)};
}
Tensor fwd_interleaved_decay_meta(const Tensor &feat, const Tensor &w, const Tensor &decay, int64_t hl,
                                  at::ScalarType filt)
{
    check_feat_only(feat);
    check_decay(w, decay, hl, feat.size(2), feat);
    (void)gated_code_for(feat.scalar_type(), filt);
    return at::empty({feat.size(0), feat.size(1), feat.size(2), feat.size(3)}, feat.options());
}
std::tuple<Tensor, Tensor> bwd_interleaved_decay_meta(const Tensor &dy, const Tensor &feat, const Tensor &w,
                                                      const Tensor &decay, int64_t hl, at::ScalarType filt, bool)
{
    check_feat_only(feat);
    check_decay(w, decay, hl, feat.size(2), feat);
    (void)dy;
    (void)gated_code_for(feat.scalar_type(), filt);
    return {at::empty_like(feat), at::empty_like(w)};
}

Tensor fwd_time_major_meta(const Tensor &x, const Tensor &B, const Tensor &C, const Tensor &h)
{
    check_time_major(x, B, C, h);
    (void)gated_code(x, h);
    return at::empty({x.size(1), x.size(0), x.size(2), x.size(3)}, x.options());
}
std::tuple<Tensor, Tensor, Tensor, Tensor> bwd_time_major_meta(const Tensor &dy, const Tensor &x, const Tensor &B,
                                                               const Tensor &C, const Tensor &h)
{
    check_time_major(x, B, C, h);
    (void)dy;
    return {at::empty_like(x), at::empty_like(x), at::empty_like(x), at::empty_like(h)};
}

Tensor mixer_mr_fwd_decay_meta(const Tensor &raw, const Tensor &wf, const Tensor &w, const Tensor &decay, int64_t hl,
                               at::ScalarType filt, bool planar)
{
    check_mixer_mr_decay(raw, wf, w, decay, hl, planar);
    (void)gated_code_for(raw.scalar_type(), filt);
    return at::empty({raw.size(0), raw.size(1), raw.size(planar ? 3 : 2), raw.size(planar ? 4 : 3)}, raw.options());
}
std::tuple<Tensor, Tensor, Tensor> mixer_mr_bwd_decay_meta(const Tensor &dy, const Tensor &raw, const Tensor &wf,
                                                           const Tensor &w, const Tensor &decay, int64_t hl,
                                                           at::ScalarType filt, bool planar)
{
    check_mixer_mr_decay(raw, wf, w, decay, hl, planar);
    (void)dy;
    (void)gated_code_for(raw.scalar_type(), filt);
    return {at::empty_like(raw), at::empty_like(wf), at::empty_like(w)};
}

Tensor mixer_mr_fwd_meta(const Tensor &raw, const Tensor &wf, const Tensor &h, bool planar)
{
    check_mixer_mr(raw, wf, h, planar);
    return at::empty({raw.size(0), raw.size(1), raw.size(planar ? 3 : 2), raw.size(planar ? 4 : 3)}, raw.options());
}
std::tuple<Tensor, Tensor, Tensor> mixer_mr_bwd_meta(const Tensor &dy, const Tensor &raw, const Tensor &wf,
                                                     const Tensor &h, bool planar)
{
    check_mixer_mr(raw, wf, h, planar);
    (void)dy;
    return {at::empty_like(raw), at::empty_like(wf), at::empty_like(h)};
}

} // namespace

TORCH_LIBRARY(gcg, m)
{
    m.def("fwd(Tensor x, Tensor B, Tensor C, Tensor h, int algo=0) -> Tensor");
    m.def("fwd_full(Tensor x, Tensor B, Tensor C, Tensor h, bool return_bx, bool return_y2, int algo=0)"
          " -> (Tensor, Tensor, Tensor)");
    m.def("fwd_out(Tensor x, Tensor B, Tensor C, Tensor h, Tensor(a!) out, int algo=0) -> ()");
    m.def("bwd(Tensor dy, Tensor x, Tensor B, Tensor C, Tensor h, int algo=0) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("fwd_interleaved(Tensor feat, Tensor h, int algo=0) -> Tensor");
    m.def("bwd_interleaved(Tensor dy, Tensor feat, Tensor h, int algo=0, bool keep_output=False) -> (Tensor, Tensor)");
    m.def("fwd_planar(Tensor feat, Tensor h, int algo=0) -> Tensor");
    m.def("bwd_planar(Tensor dy, Tensor feat, Tensor h, int algo=0) -> (Tensor, Tensor)");
    m.def("dwconv_fwd(Tensor x, Tensor w, bool keep_output=False) -> Tensor");
    m.def("dwconv_bwd(Tensor dy, Tensor x, Tensor w) -> (Tensor, Tensor)");
    m.def("mixer_se_fwd(Tensor raw, Tensor wf, Tensor h, bool planar=False) -> Tensor");
    m.def("mixer_se_bwd(Tensor dy, Tensor raw, Tensor wf, Tensor h, bool planar=False) -> (Tensor, Tensor, Tensor)");
    m.def("filter_decay_fwd(Tensor w, Tensor decay, int hl, ScalarType dtype) -> Tensor");
    m.def("filter_decay_bwd(Tensor dh, Tensor decay) -> Tensor");
    m.def("mixer_mr_fwd(Tensor raw, Tensor wf, Tensor h, bool planar=False) -> Tensor");
    m.def("mixer_mr_bwd(Tensor dy, Tensor raw, Tensor wf, Tensor h, bool planar=False) -> (Tensor, Tensor, Tensor)");
    m.def("mixer_mr_fwd_decay(Tensor raw, Tensor wf, Tensor w, Tensor decay, int hl, ScalarType filt, bool planar=False)"
          " -> Tensor");
    m.def("mixer_mr_bwd_decay(Tensor dy, Tensor raw, Tensor wf, Tensor w, Tensor decay, int hl, ScalarType filt,"
          " bool planar=False) -> (Tensor, Tensor, Tensor)");
    m.def("fwd_time_major(Tensor x, Tensor B, Tensor C, Tensor h) -> Tensor");
    m.def("bwd_time_major(Tensor dy, Tensor x, Tensor B, Tensor C, Tensor h) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("fwd_decay(Tensor x, Tensor B, Tensor C, Tensor w, Tensor decay, int hl, ScalarType filt) -> Tensor");
    m.def("bwd_decay(Tensor dy, Tensor x, Tensor B, Tensor C, Tensor w, Tensor decay, int hl, ScalarType filt)"
          " -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("fwd_interleaved_decay(Tensor feat, Tensor w, Tensor decay, int hl, ScalarType filt) -> Tensor");
    m.def("bwd_interleaved_decay(Tensor dy, Tensor feat, Tensor w, Tensor decay, int hl, ScalarType filt,"
          " bool keep_output=False) -> (Tensor, Tensor)");
}

TORCH_LIBRARY_IMPL(gcg, CUDA, m)
{
    m.impl("fwd", &fwd);
    m.impl("fwd_full", &fwd_full);
    m.impl("fwd_out", &fwd_out);
    m.impl("bwd", &bwd);
    m.impl("fwd_interleaved", &fwd_interleaved);
    m.impl("bwd_interleaved", &bwd_interleaved);
    m.impl("fwd_planar", &fwd_planar);
    m.impl("bwd_planar", &bwd_planar);
    m.impl("dwconv_fwd", &dwconv_fwd);
    m.impl("dwconv_bwd", &dwconv_bwd);
    m.impl("mixer_se_fwd", &mixer_se_fwd);
    m.impl("mixer_se_bwd", &mixer_se_bwd);
    m.impl("filter_decay_fwd", &filter_decay_fwd);
    m.impl("filter_decay_bwd", &filter_decay_bwd);
    m.impl("mixer_mr_fwd", &mixer_mr_fwd);
    m.impl("mixer_mr_bwd", &mixer_mr_bwd);
    m.impl("mixer_mr_fwd_decay", &mixer_mr_fwd_decay);
    m.impl("mixer_mr_bwd_decay", &mixer_mr_bwd_decay);
    m.impl("fwd_time_major", &fwd_time_major);
    m.impl("bwd_time_major", &bwd_time_major);
    m.impl("fwd_decay", &fwd_decay);
    m.impl("bwd_decay", &bwd_decay);
    m.impl("fwd_interleaved_decay", &fwd_interleaved_decay);
    m.impl("bwd_interleaved_decay", &bwd_interleaved_decay);
}

TORCH_LIBRARY_IMPL(gcg, Meta, m)
{
    m.impl("fwd", &fwd_meta);
    m.impl("fwd_full", &fwd_full_meta);
    m.impl("fwd_out", &fwd_out_meta);
    m.impl("bwd", &bwd_meta);
    m.impl("fwd_interleaved", &fwd_interleaved_meta);
    m.impl("bwd_interleaved", &bwd_interleaved_meta);
    m.impl("fwd_planar", &fwd_planar_meta);
    m.impl("bwd_planar", &bwd_planar_meta);
    m.impl("dwconv_fwd", &dwconv_fwd_meta);
    m.impl("dwconv_bwd", &dwconv_bwd_meta);
    m.impl("mixer_se_fwd", &mixer_se_fwd_meta);
    m.impl("mixer_se_bwd", &mixer_se_bwd_meta);
    m.impl("filter_decay_fwd", &filter_decay_fwd_meta);
    m.impl("filter_decay_bwd", &filter_decay_bwd_meta);
    m.impl("mixer_mr_fwd", &mixer_mr_fwd_meta);
    m.impl("mixer_mr_bwd", &mixer_mr_bwd_meta);
    m.impl("mixer_mr_fwd_decay", &mixer_mr_fwd_decay_meta);
    m.impl("mixer_mr_bwd_decay", &mixer_mr_bwd_decay_meta);
    m.impl("fwd_time_major", &fwd_time_major_meta);
    m.impl("bwd_time_major", &bwd_time_major_meta);
    m.impl("fwd_decay", &fwd_decay_meta);
    m.impl("bwd_decay", &bwd_decay_meta);
    m.impl("fwd_interleaved_decay", &fwd_interleaved_decay_meta);
    m.impl("bwd_interleaved_decay", &bwd_interleaved_decay_meta);
}
