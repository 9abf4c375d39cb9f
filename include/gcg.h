/*
 * gcg.h -- C ABI of the MI355X (gfx950) gated chunked causal convolution
 *
 *     u = B * x ;  y2[b,t,c] = sum_k h[c/dg, k] * u[b, t-(hl-1)+k, c] ;  y = C * y2
 *
 * and its backward (dx, dB, dC, dh).  This is the boundary a replacement for
 * savanna's `gcg_two_pass` path binds to: every entry point takes plain device
 * pointers, sizes and a HIP stream, returns 0 or a negative error code, never
 * throws, never synchronises the host and never allocates device memory.
 *
 * Tensors x, B, C, y, y2, bx, dy, dx, dB, dC are (bs, L, g, dg), contiguous,
 * channel fastest (d = g*dg); h and dh are (g, 1, hl), contiguous.  All share
 * one element type `dtype`.  Cross-correlation convention: tap hl-1 multiplies
 * the current sample and samples before t = 0 are zero
 * (savanna/kernels/triton_src/cgcg/ref_fwd.py:41,109-129).
 */
#ifndef GCG_H
#define GCG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define GCG_API __attribute__((visibility("default")))
#else
#define GCG_API
#endif

/* Element types (the reference's `cgcg_dtype`, savanna/arguments/global_config.py:404).
 *
 * GCG_BF16_F32 and GCG_F16_F32 replace the casts the reference's operators put around the
 * call when `cgcg_dtype` ("float32", the default) differs from the activations' dtype
 * (savanna/model/operators/hyena/hyena.py:499-503 and :533-534, :805-817): the tensors
 * x, B, C, y, dy, dx, dB, dC are 16-bit, the filter h and its gradient dh are fp32, and
 * no activation is rounded to 16 bits between a load and a store -- the values are those of
 * `op(x.float(), B.float(), C.float(), h).to(bf16)` and of its autograd backward, with one
 * qualification in the matrix-core kernels: the taps enter the products with 16 significant
 * bits (2^-17 relative, far below the 16-bit outputs' own rounding; dh is not affected).
 * gcg_fwd, gcg_bwd, gcg_bwd_static, gcg_fwd_interleaved, gcg_bwd_interleaved take them
 * (every kernel family); the featurizer entry points do not (GCG_ERR_BAD_ARG). */
enum { GCG_F32 = 0, GCG_BF16 = 1, GCG_F16 = 2, GCG_BF16_F32 = 3, GCG_F16_F32 = 4 };

/* Kernel families.  GCG_ALGO_AUTO picks by (dtype, hl, dg); the others force one
 * family and fail with GCG_ERR_UNSUPPORTED when the shape does not fit it. */
enum {
    GCG_ALGO_AUTO   = 0,
    GCG_ALGO_DIRECT = 1, /* LDS-tiled sliding window on the vector ALUs, any hl/dg/dtype */
    GCG_ALGO_WINDOW = 2, /* register sliding window, hl <= 8 (Hyena-SE)                   */
    GCG_ALGO_MFMA   = 3  /* banded Toeplitz GEMM on MFMA, any dtype, hl <= 128, dg % 16 == 0 (Hyena-MR) */
};

/* Flags of the entry points whose output another entry point reads back at once (the featurized
 * tensor between gcg_dwconv_fwd and gcg_fwd_interleaved, the gradient of the features between
 * gcg_bwd_interleaved and gcg_dwconv_bwd).  With GCG_KEEP_OUTPUT that output is stored through
 * the cache instead of past it, so part of it is still there when the next kernel starts: the
 * chain gets faster (6 % at the 7B layer shape), the kernel timed alone a few percent slower.
 * Results do not depend on it. */
enum { GCG_KEEP_OUTPUT = 1 };

/* Error codes. */
enum {
    GCG_OK              = 0,
    GCG_ERR_BAD_ARG     = -1, /* null pointer, non-positive size, unknown dtype/algo */
    GCG_ERR_UNSUPPORTED = -2, /* shape outside what the forced algo handles          */
    GCG_ERR_WORKSPACE   = -3, /* workspace missing or smaller than *_workspace_bytes */
    GCG_ERR_LAUNCH      = -4, /* hipLaunchKernel / stream error; see gcg_last_hip_error */
    GCG_ERR_DEVICE      = -5, /* current device is not gfx950                        */
    GCG_ERR_STATIC_SCRATCH = -6 /* gcg_bwd_static: sizes need more scratch than it holds */
};

/* Human-readable text for a code above. */
GCG_API const char *gcg_strerror(int code);

/* hipError_t of the last failed HIP call made by this library on the calling
 * thread (0 when none). */
GCG_API int gcg_last_hip_error(void);

/*
 * Measurement hook; it has no counterpart in the reference.  Arms a pair of HIP events
 * (hipEvent_t, created with timing enabled) on the calling thread.  The next gcg_fwd, gcg_bwd,
 * gcg_fwd_interleaved or gcg_bwd_interleaved call on this thread that runs the register-window
 * or matrix-core kernels has the runtime stamp the two events at the start and at the end of
 * its main kernel -- not of the small filter-gradient reduction that follows a backward -- so
 * that hipEventElapsedTime(start, stop) is that kernel's own duration, as a profiler reports
 * it.  The arming lasts for one call: every entry point that launches kernels clears it on
 * return, whatever it returns and whether its launcher used the events or not.  Two null
 * pointers disarm; one null pointer is GCG_ERR_BAD_ARG.  Not for a stream that is being
 * captured into a graph: a timed launch is not a plain kernel node.
 */
GCG_API int gcg_time_next_kernel(void *start_event, void *stop_event);

/* Library version, e.g. 100 for 0.1.0. */
GCG_API int gcg_version(void);

/*
 * Whether the entry points of a route take these sizes -- every limit they check apart from the
 * alignment of the tensors (16 bytes), which only the call itself can see.  It has no counterpart
 * in the reference; it is what a caller that chooses between a fused entry point and the general
 * ones (gcg_fwd / gcg_bwd, which take any size) asks before it chooses.  kf is the featurizer's
 * filter length for the mixer routes and ignored otherwise.  Returns 1, 0, or GCG_ERR_BAD_ARG.
 */
enum {
    GCG_ROUTE_DECAY           = 1, /* gcg_fwd_decay, gcg_bwd_decay, gcg_*_interleaved_decay              */
    GCG_ROUTE_TIME_MAJOR      = 2, /* gcg_fwd_time_major, gcg_bwd_time_major                             */
    GCG_ROUTE_MIXER_SE        = 3, /* gcg_mixer_se_fwd / _bwd and their _planar forms                    */
    GCG_ROUTE_MIXER_MR        = 4, /* gcg_mixer_mr_fwd / _bwd (and _decay)                               */
    GCG_ROUTE_MIXER_MR_PLANAR = 5  /* gcg_mixer_mr_fwd_planar / _bwd_planar (and _decay): one-kernel form */
};
GCG_API int gcg_route_supported(int32_t route, int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                        int32_t kf, int32_t dtype);

/*
 * Forward.
 * Replaces two_pass_fwd_grouped(x, B, C, h, return_bx=, return_y2=)
 * (savanna/kernels/triton_src/cgcg/src/fwd.py:13-233), which launches
 * _two_pass_fwd_refactor_kernel (src/fwd_kernels.py:585-750).
 *
 *   y            out, required
 *   y2_or_null   out, optional: the convolution before the post-gate (fwd.py `return_y2`)
 *   bx_or_null   out, optional: the pre-gate product B*x             (fwd.py `return_bx`)
 *   stream       hipStream_t to enqueue on (NULL = the null stream)
 */
GCG_API int gcg_fwd(const void *x, const void *B, const void *C, const void *h,
            void *y, void *y2_or_null, void *bx_or_null,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t algo, void *stream);

/*
 * Workspace the backward needs for the deterministic filter-gradient reduction
 * (per-workgroup partial sums of dh).  Depends on the sizes, dtype and algo only.
 * Returns 0 on invalid arguments.
 */
GCG_API size_t gcg_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                               int32_t dtype, int32_t algo);

/*
 * Backward.
 * Replaces two_pass_bwd_refactor(dy, Bx, y2, x, B, C, h, bs, seqlen, g, dg, ...)
 * (savanna/kernels/triton_src/cgcg/src/bwd.py:347-474: pre_conv_kernel,
 * conv1d_input, conv1d_weight, group sum, post_conv_kernel).  The saved
 * activations Bx and y2 of the reference are not needed: both are recomputed
 * on chip from x, B, h.
 *
 *   dx, dB, dC   out, (bs, L, g, dg), element type `dtype`
 *   dh           out, (g, 1, hl), element type `dtype`, overwritten (not accumulated)
 *   workspace    device scratch of at least gcg_bwd_workspace_bytes(...) bytes,
 *                256-byte aligned; contents on entry are ignored
 *
 * Streams (this and every other backward entry point of the matrix-core kernels): the last
 * workgroup of a channel block to finish adds the block's filter-gradient partials, and
 * which one that is is decided with arrival tickets kept inside the library.  A stream
 * owns one set of tickets from its first such launch until the process ends; launches on
 * one stream run in order and share the set, launches on different streams never share
 * one.  Up to 64 streams hold sets; a launch on a further stream, or on a stream that is
 * being captured into a graph, takes none and adds the partials with a second small kernel
 * on the same stream instead (same order of summation, same bits).  The rule for callers:
 * give concurrent launches their own workspace and outputs, as for any kernel; nothing
 * else.  (A launch that does not run to its end -- a device fault -- leaves its stream's
 * tickets mid-count; the process's device context does not survive that either.)
 */
GCG_API int gcg_bwd(const void *dy, const void *x, const void *B, const void *C, const void *h,
            void *dx, void *dB, void *dC, void *dh,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t algo, void *stream);

/*
 * Backward for callers that cannot allocate.  It has no counterpart in the reference: it is
 * gcg_bwd for code that runs where device memory cannot be obtained -- under HIP graph capture,
 * in a tight serving loop, in a harness that forbids hipMalloc -- and so has no workspace to
 * hand over.  The per-workgroup partial sums of dh go to a device array that is part of the
 * library image (GCG_BWD_STATIC_SCRATCH_BYTES per GPU, held from the first call on that GPU until
 * the process ends); the call itself allocates and frees nothing.  Same kernels, same order of
 * summation, hence the same bits as gcg_bwd.
 *
 * Sizes whose gcg_bwd_workspace_bytes(...) exceeds GCG_BWD_STATIC_SCRATCH_BYTES are rejected with
 * GCG_ERR_STATIC_SCRATCH (the Evo2-7B and 40B layer shapes need 0.5 MB on the matrix-core kernels and
 * 3.5 and 7 MB on the register-window kernels).  All calls on one GPU share the one array: two calls that
 * may overlap in time (different streams, different threads) race on it and must be ordered by the
 * caller.  Nothing in it has to start at zero and nothing of a call's result stays in it.
 * The first call on a GPU looks the array's address up, which may load the library's code onto that
 * GPU; make that call before, not during, a graph capture.
 */
#define GCG_BWD_STATIC_SCRATCH_BYTES (8u << 20)
GCG_API int gcg_bwd_static(const void *dy, const void *x, const void *B, const void *C, const void *h,
            void *dx, void *dB, void *dC, void *dh,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t algo, void *stream);

/*
 * Name of the kernel family GCG_ALGO_AUTO resolves to for these sizes
 * (GCG_ALGO_DIRECT / _WINDOW / _MFMA), or a negative error code.
 * `backward` selects the rule for gcg_bwd.
 */
GCG_API int gcg_select_algo(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
                    int32_t dtype, int32_t backward);

/*
 * Forward on interleaved operands.
 * Replaces the three gathers `x.contiguous()`, `B.contiguous()`, `C.contiguous()` of
 * TwoPassChunkedGateConvGate.forward (savanna/kernels/triton_src/cgcg/interface.py:51-54)
 * followed by two_pass_fwd_grouped, for the case those three arguments are the unbound
 * thirds of one projected-features tensor, as the interleaved split of
 * ParallelSequenceMixer.forward produces them (savanna/model/block.py:886-890:
 * `rearrange(features, "b l (g dg p) -> b l g p dg", p=3).unbind(dim=3)` gives x1, x2, v,
 * which the operators pass on as C = x1, B = x2, x = v, hyena.py:517-531, :825-840).
 *
 *   feat   (bs, L, g, dg, 3) contiguous: feat[..., 0] = C, feat[..., 1] = B, feat[..., 2] = x
 *   y      out, (bs, L, g, dg)
 */
GCG_API int gcg_fwd_interleaved(const void *feat, const void *h, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t algo, void *stream);

/*
 * Backward on interleaved operands: the counterpart of gcg_bwd for gcg_fwd_interleaved.
 * Replaces two_pass_bwd_refactor (src/bwd.py:347-474) plus the scatter of dx, dB, dC into
 * the gradient of the features tensor that autograd performs for the unbind / rearrange of
 * block.py:886-890.
 *
 *   dy      (bs, L, g, dg)
 *   dfeat   out, (bs, L, g, dg, 3): dfeat[..., 0] = dC, [..., 1] = dB, [..., 2] = dx
 *   dh      out, (g, 1, hl), overwritten
 *   workspace, workspace_bytes   as for gcg_bwd, sized by gcg_bwd_workspace_bytes
 *   flags   0 or GCG_KEEP_OUTPUT (dfeat is what gcg_dwconv_bwd reads next)
 */
GCG_API int gcg_bwd_interleaved(const void *dy, const void *feat, const void *h,
            void *dfeat, void *dh,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t algo, int32_t flags, void *stream);

/*
 * The gated convolution on planar projected features: one (bs, L, 3, g, dg) tensor whose rows hold the three
 * operands side by side, [..., 0, :, :] = C (post-gate, x1), [..., 1, :, :] = B (pre-gate, x2), [..., 2, :, :] = x (v)
 * -- the split without interleaving of savanna/model/block.py:881-884 ("b l (p g dg) -> b l p g dg", kept for
 * checkpoints trained with interleave_projections = false).  The reference gathers the three strided views into
 * contiguous tensors (kernels/triton_src/cgcg/interface.py:51-54) and autograd re-assembles the gradient; here
 * the kernels read the thirds of the rows in place and write dfeat (same layout) directly.
 *   feat, dfeat  (bs, L, 3, g, dg)   h, dh  (g, 1, hl)   y, dy  (bs, L, g, dg)
 * Same values as gcg_fwd / gcg_bwd on the gathered operands.  dtype: any, GCG_BF16_F32 / GCG_F16_F32 included.
 * Workspace: gcg_bwd_workspace_bytes(...) with the same algo.
 */
GCG_API int gcg_fwd_planar(const void *feat, const void *h, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t algo, void *stream);
GCG_API int gcg_bwd_planar(const void *dy, const void *feat, const void *h,
            void *dfeat, void *dh,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t algo, void *stream);

/*
 * Short causal depthwise convolution without gates: the featurizer that the hyena blocks apply to
 * the projected features before splitting them.
 * Replaces ParallelCausalDepthwiseConv1d.forward (savanna/model/operators/hyena/hyena.py:136-181,
 * the F.conv1d path :159-176; called at savanna/model/block.py:873) together with the permutes
 * to and from its (B, D, L) layout (block.py:867, :875): here the tensors stay (bs, L, g, dg) with
 * the channel fastest, the layout of the dense projection before it and of gcg_fwd_interleaved
 * after it.
 *
 *   y[b, t, c] = sum_k w[c / dg, 0, k] * x[b, t - (hl-1) + k, c]      (zero before the sequence)
 *
 *   x, y   (bs, L, g, dg);  w  (g, 1, hl), hl <= 8.  The reference's filters are one per
 *          channel (weight (D, 1, K), hyena.py:108-110): g = D, dg = 1.  Supported: dg == 1 or
 *          dg % 4 == 0, g * dg % 4 == 0, 16-byte aligned tensors; otherwise GCG_ERR_UNSUPPORTED.
 *   flags  0 or GCG_KEEP_OUTPUT (y is what gcg_fwd_interleaved reads next)
 */
GCG_API int gcg_dwconv_fwd(const void *x, const void *w, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, int32_t flags, void *stream);

/* Workspace of gcg_dwconv_bwd (per-run partial sums of dw); 0 on invalid or unsupported arguments. */
GCG_API size_t gcg_dwconv_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype);

/*
 * Backward of gcg_dwconv_fwd: what autograd derives for the F.conv1d of hyena.py:168-175
 * (conv1d_input / conv1d_weight).
 *   dx  out, (bs, L, g, dg);  dw  out, (g, 1, hl), overwritten, bit-reproducible
 *   workspace  at least gcg_dwconv_bwd_workspace_bytes(...) bytes, 256-byte aligned
 */
GCG_API int gcg_dwconv_bwd(const void *dy, const void *x, const void *w, void *dx, void *dw,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype, void *stream);

/*
 * Featurizer convolution and short gated convolution in one pass: gcg_dwconv_fwd on the
 * (bs, L, 3 * g * dg) projected features followed by gcg_fwd_interleaved on its result, without
 * the featurized tensor ever going to memory.
 * Replaces, for the Hyena-SE layers, the chain of ParallelSequenceMixer.forward
 * (savanna/model/block.py:867-890: permute, ParallelCausalDepthwiseConv1d, permute, interleaved
 * split) and ParallelShortHyenaOperator.forward with use_cgcg_short
 * (savanna/model/operators/hyena/hyena.py:825-840 -> two_pass_chunked_gate_conv_gate).
 *
 *   raw    (bs, L, g, dg, 3) contiguous, i.e. (bs, L, 3 * g * dg): the dense projection's output
 *   wf     (3 * g * dg, 1, kf): one featurizer filter per feature channel, kf <= 4
 *   h      (g, 1, hl), hl <= 8
 *   y      out, (bs, L, g, dg)
 *
 *   f[b, t, j] = dtype( sum_k wf[j, 0, k] * raw[b, t - (kf-1) + k, j] )       (fp32 accumulation)
 *   y          = gcg_fwd_interleaved(f, h)
 *
 * The result equals that of the two calls it replaces up to the rounding of the fp32 sums (the
 * taps are added in another order).
 * dtype GCG_BF16_F32 / GCG_F16_F32: raw, wf, y (and dy, draw, dwf) are 16-bit, h and dh are fp32 -- cgcg_dtype
 * float32 on 16-bit activations (hyena.py:812-816, :842-843) without the casts: f is rounded to 16 bits as the
 * featurizer stores it, the operator's taps and arithmetic are fp32, y is rounded once.
 * Supported: hl <= 8, kf <= 4, dg even, 16-byte aligned tensors; otherwise GCG_ERR_UNSUPPORTED.
 */
GCG_API int gcg_mixer_se_fwd(const void *raw, const void *wf, const void *h, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);

/* Workspace of gcg_mixer_se_bwd (per-run partial sums of dh and dwf); 0 on invalid or unsupported arguments. */
GCG_API size_t gcg_mixer_se_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t kf, int32_t dtype);

/*
 * Backward of gcg_mixer_se_fwd: gcg_bwd_interleaved (recomputing f from raw) followed by
 * gcg_dwconv_bwd, in one pass; the gradient of f is rounded to `dtype` in between as when the two
 * run separately.
 *   dy     (bs, L, g, dg)
 *   draw   out, (bs, L, g, dg, 3)
 *   dwf    out, (3 * g * dg, 1, kf);  dh  out, (g, 1, hl); both overwritten, bit-reproducible
 *   workspace  at least gcg_mixer_se_bwd_workspace_bytes(...) bytes, 256-byte aligned
 */
GCG_API int gcg_mixer_se_bwd(const void *dy, const void *raw, const void *wf, const void *h,
            void *draw, void *dwf, void *dh,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);

/*
 * The same two on planar features -- the split without interleaving of savanna/model/block.py:881-884
 * (interleave_projections = false): raw and draw are (bs, L, 3, g, dg), each row the planes C | B | x one after the
 * other, and wf, dwf hold their 3 * g * dg filters in that channel order.  Same workspace size.
 */
GCG_API int gcg_mixer_se_fwd_planar(const void *raw, const void *wf, const void *h, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);
GCG_API int gcg_mixer_se_bwd_planar(const void *dy, const void *raw, const void *wf, const void *h,
            void *draw, void *dwf, void *dh,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);

/*
 * Featurizer and Hyena-MR operator without the featurized tensor: gcg_dwconv_fwd followed by
 * gcg_fwd_interleaved as one kernel that makes every row of (C, B, x) on the way
 * (savanna/model/block.py:867-890 -> hyena.py:517-531), and a backward that needs the projection output only.
 * Every row of the features is the featurizer's result rounded to the tensors' type, exactly what the two-call
 * chain stores and reads back, so y, dh and the gradients are the chain's (bit for bit at bf16 and fp32; at
 * f16 the compiler sums the featurizer's taps in another grouping in the two kernels, which moves a few results
 * in 10^5 by one unit in the last place).
 *   raw  (bs, L, g, dg, 3)   wf  (3 * g * dg, 1, kf), tensors' type   h  (g, 1, hl)   y  out, (bs, L, g, dg)
 * Forward: reads raw, writes y -- 4 N s of memory traffic instead of 10 N s.
 * Backward, 16-bit tensors with arithmetic in their own type: one kernel goes from dy and raw to draw, dwf and dh --
 * the features are made again from raw, their gradient is handed from the operator's part to the featurizer's
 * part inside the workgroup and never stored: 7 N s of memory traffic (dy and raw in, draw out) instead of the two-call
 * chain's 16 N s.  draw and dh are the chain's bit for bit (bf16), dwf up to the order in which partial sums are added.
 * Other types (fp32 arithmetic): one kernel recomputes the features and writes their gradient into dfeat_scratch
 * ((bs, L, g, dg, 3), caller's memory, contents on return unspecified), then the featurizer's own backward turns
 * it into draw and dwf -- the chain's traffic, but nothing of size 3 N is kept between forward and backward.
 * gcg_mixer_mr_bwd_scratch_bytes(...) says how large dfeat_scratch has to be: 0 (it may then be NULL) where the
 * one-kernel backward runs, the size of raw otherwise.
 *   draw  out, (bs, L, g, dg, 3)   dwf  out, (3 * g * dg, 1, kf)   dh  out, (g, 1, hl), filter's type
 *   workspace  gcg_mixer_mr_bwd_workspace_bytes(...) bytes, 256-byte aligned
 * Matrix-core kernels only: hl <= 128, dg % 16 == 0, kf <= 3, 16-byte aligned tensors; otherwise
 * GCG_ERR_UNSUPPORTED (use the two calls).  The kernels are laid out for filters of 98 to 128 taps (five slices of
 * the banded matrix); a shorter filter leaves the far slices zero and costs the same time.  dtype: any, GCG_BF16_F32 / GCG_F16_F32 included.
 */
GCG_API int gcg_mixer_mr_fwd(const void *raw, const void *wf, const void *h, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);
GCG_API size_t gcg_mixer_mr_bwd_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t kf, int32_t dtype);
GCG_API size_t gcg_mixer_mr_bwd_scratch_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t kf, int32_t dtype);
GCG_API int gcg_mixer_mr_bwd(const void *dy, const void *raw, const void *wf, const void *h,
            void *draw, void *dwf, void *dh, void *dfeat_scratch,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);

/*
 * The same two on planar features (interleave_projections = false, savanna/model/block.py:881-884): raw and draw
 * are (bs, L, 3, g, dg), each row the planes C | B | x one after the other, and wf, dwf hold their filters in that
 * channel order.  One-kernel path only: 16-bit tensors with arithmetic in their own type (GCG_BF16, GCG_F16),
 * otherwise GCG_ERR_UNSUPPORTED (run gcg_dwconv_fwd and gcg_fwd_planar, and their backwards, instead).
 * Workspace: gcg_mixer_mr_bwd_workspace_bytes; no scratch tensor.
 */
GCG_API int gcg_mixer_mr_fwd_planar(const void *raw, const void *wf, const void *h, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);
GCG_API int gcg_mixer_mr_bwd_planar(const void *dy, const void *raw, const void *wf, const void *h,
            void *draw, void *dwf, void *dh,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);

/*
 * The same with the Hyena-MR filter formed inside the kernels, as in gcg_fwd_decay / gcg_bwd_decay: h = F(w * decay)
 * cut to hl taps (ExplicitSingleDecayFilter.filter, savanna/model/operators/hyena/parametrization/explicit.py:68-75,
 * and the cast of hyena.py:499-503), dw the gradient of the parameter w.  A Hyena-MR layer's convolutional part --
 * filter, featurizer, operator -- is then one launch each way.
 *   w, decay  (g, l_cache) fp32   dw  out, (g, l_cache) fp32, zero beyond hl
 * Workspace and scratch sizes: gcg_mixer_mr_bwd_workspace_bytes, gcg_mixer_mr_bwd_scratch_bytes.
 */
GCG_API int gcg_mixer_mr_fwd_decay(const void *raw, const void *wf, const float *w, const float *decay,
            int32_t l_cache, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);
GCG_API int gcg_mixer_mr_bwd_decay(const void *dy, const void *raw, const void *wf, const float *w,
            const float *decay, int32_t l_cache, void *draw, void *dwf, float *dw, void *dfeat_scratch,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);
/* Both at once: planar features and the filter formed in the kernels (one-kernel path only, no scratch tensor). */
GCG_API int gcg_mixer_mr_fwd_planar_decay(const void *raw, const void *wf, const float *w, const float *decay,
            int32_t l_cache, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);
GCG_API int gcg_mixer_mr_bwd_planar_decay(const void *dy, const void *raw, const void *wf, const float *w,
            const float *decay, int32_t l_cache, void *draw, void *dwf, float *dw,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t kf,
            int32_t dtype, void *stream);

/*
 * Explicit decayed filter of Hyena-MR, ready for gcg_fwd, in one launch.
 * Replaces ExplicitSingleDecayFilter.filter (savanna/model/operators/hyena/parametrization/
 * explicit.py:68-75: h = self.h[:, :L] * self.decay[:, :L]) with L = min(hyena_mr_len, seq_len),
 * the [:, None] of hyena.py:440-441 and the cast to cgcg_dtype of hyena.py:499-503.
 *
 *   w, decay   (g, l_cache) fp32: the parameter and the decay buffer
 *   h          out, (g, 1, hl) of element type `dtype`:  h[g, 0, k] = dtype(w[g, k] * decay[g, k])
 */
GCG_API int gcg_filter_decay_fwd(const float *w, const float *decay, void *h,
            int32_t g, int32_t l_cache, int32_t hl, int32_t dtype, void *stream);

/*
 * Its backward, what autograd derives for the cast, product and slice above:
 *   dh   (g, 1, hl) of element type `dtype`, as gcg_bwd writes it
 *   dw   out, (g, l_cache) fp32:  dw[g, k] = float(dh[g, 0, k]) * decay[g, k] for k < hl, else 0
 */
GCG_API int gcg_filter_decay_bwd(const void *dh, const float *decay, float *dw,
            int32_t g, int32_t l_cache, int32_t hl, int32_t dtype, void *stream);

/*
 * The gated convolution of Hyena-MR with its explicit decayed filter built inside the kernels: the filter
 * table a workgroup keeps on chip is filled with F(w[g, k] * decay[g, k]) (F = element type of the filter for
 * `dtype`: the tensors' type, or fp32 for GCG_F32 / GCG_BF16_F32 / GCG_F16_F32) instead of being read from h,
 * and the backward's filter-gradient reduction writes the gradient of the parameter itself,
 *   dw[g, k] = float(F(dh[g, 0, k])) * decay[g, k]  for k < hl,  0 for hl <= k < l_cache,
 * so neither h nor dh exists in memory and the layer needs no launch besides the convolution's.
 * Replaces, around two_pass_fwd_grouped / two_pass_bwd_refactor, ExplicitSingleDecayFilter.filter
 * (savanna/model/operators/hyena/parametrization/explicit.py:68-75), the [:, None] and cast of
 * savanna/model/operators/hyena/hyena.py:440-441 and :499-503, and what autograd derives for them.
 * The values are those of gcg_filter_decay_fwd -> gcg_fwd (gcg_bwd -> gcg_filter_decay_bwd), bit for bit.
 *
 * Matrix-core kernels only: hl <= 128, dg % 16 == 0, 16-byte aligned tensors, else GCG_ERR_UNSUPPORTED
 * (make the filter with gcg_filter_decay_fwd then).  w, decay: (g, l_cache) fp32; dw: out, (g, l_cache)
 * fp32, overwritten; workspace as for gcg_bwd (gcg_bwd_workspace_bytes with GCG_ALGO_MFMA).
 */
GCG_API int gcg_fwd_decay(const void *x, const void *B, const void *C,
            const float *w, const float *decay, int32_t l_cache, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, void *stream);
GCG_API int gcg_bwd_decay(const void *dy, const void *x, const void *B, const void *C,
            const float *w, const float *decay, int32_t l_cache,
            void *dx, void *dB, void *dC, float *dw,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, void *stream);
/* The same on the interleaved features tensor (gcg_fwd_interleaved / gcg_bwd_interleaved). */
GCG_API int gcg_fwd_interleaved_decay(const void *feat,
            const float *w, const float *decay, int32_t l_cache, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, void *stream);
GCG_API int gcg_bwd_interleaved_decay(const void *dy, const void *feat,
            const float *w, const float *decay, int32_t l_cache,
            void *dfeat, float *dw,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, int32_t flags, void *stream);

/*
 * The short-filter operator on time-major operands: x, B, C (and dx, dB, dC) are (L, bs, g, dg) contiguous,
 * y and dy are (bs, L, g, dg).  This is the input layout of the reference's other short-filter kernel family,
 * run_short_hyena / ShortHyenaOperator (savanna/kernels/triton_src/short_hyena/interface.py:8-119: q, k, v of
 * shape (seqlen, bs, g, dg), which its pre-convolution kernel permutes, short_hyena/fwd.py:245-247); with
 * C = q, B = k, x = v the operator is the same gated convolution, read here where it lies instead of from
 * three permuted copies, and the gradients are written in the operands' own layout.
 * Register-window kernels only: hl <= 8, dg % 4 == 0, 16-byte aligned tensors, else GCG_ERR_UNSUPPORTED.
 * dtype: any, GCG_BF16_F32 / GCG_F16_F32 included.  workspace: gcg_bwd_time_major_workspace_bytes, 256-byte aligned.
 */
GCG_API int gcg_fwd_time_major(const void *x, const void *B, const void *C, const void *h, void *y,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, void *stream);
GCG_API size_t gcg_bwd_time_major_workspace_bytes(int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl,
            int32_t dtype);
GCG_API int gcg_bwd_time_major(const void *dy, const void *x, const void *B, const void *C, const void *h,
            void *dx, void *dB, void *dC, void *dh,
            void *workspace, size_t workspace_bytes,
            int64_t bs, int64_t L, int32_t g, int32_t dg, int32_t hl, int32_t dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GCG_H */
