// Banded Toeplitz GEMM on the matrix cores (bf16 / f16 I/O, fp32 accumulate, hl <= 128).
//
// Streaming form of the two-pass chunked convolution.  A workgroup of four waves owns 64
// adjacent channels of one batch row and walks a run of time steps of 32 rows.  Wave w owns
// the 16 channels [16w, 16w+16) -- one filter -- and computes, per step, the transposed
// output tile  Y2^T (16 channels x 32 times) = sum_i  U_{s-i}^T (16 x 32)  *  W_i (32 x 32)
// with v_mfma_f32_16x16x32, where U_{s-i} is the pre-gate product of step s-i and W_i the
// slice of the banded Toeplitz matrix of the filter at time offset 32*i.  The NK = 5 slices
// (10 operand tiles of 16 output times) live in registers for the whole walk, and the last
// NK operand tiles of U are carried in registers, so the "carry from the previous chunk" of
// the two-pass form never goes back to memory: q, k, v are read once and y written once.
//
// Memory side: the four waves load each 32 x 64 tile with full 128-byte rows, form
// u = bf16(x*B) in registers, park it row-major in LDS, and every wave fetches its matrix
// operand from there with the transposing LDS read (ds_read_b64_tr_b16), which hands a lane
// four consecutive time samples of one channel.  The fp32 result tile returns through LDS to
// the row layout, is gated with C in fp32 and stored with full 128-byte rows.
#include "gcg_common.h"

#include <cstdlib>

namespace gcg {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int STEP = 32;          // time rows per step (K of one MFMA)
constexpr int CB = 64;            // channels per workgroup
constexpr int UROW = 160;         // bytes per LDS row of u   (64 x 2 B + 32 B pad)
constexpr int YROW = 272;         // bytes per LDS row of y2  (64 x 4 B + 16 B pad)
constexpr int HPAD = 32;          // filter table holds lags [-32, 160)
constexpr int HTAB = 192;

template <typename T> struct MT;
template <> struct MT<bf16_t> {
    typedef bf16x8 op_t;
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
template <> struct MT<f16_t> {
    typedef f16x8 op_t;
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

template <typename T> __device__ __forceinline__ void unpack8(const uint4 &r, float (&f)[8])
{
    MT<T>::unpack2(r.x, f[0], f[1]);
    MT<T>::unpack2(r.y, f[2], f[3]);
    MT<T>::unpack2(r.z, f[4], f[5]);
    MT<T>::unpack2(r.w, f[6], f[7]);
}
template <typename T> __device__ __forceinline__ uint4 pack8(const float (&f)[8])
{
    return make_uint4(MT<T>::pack2(f[0], f[1]), MT<T>::pack2(f[2], f[3]), MT<T>::pack2(f[4], f[5]),
                      MT<T>::pack2(f[6], f[7]));
}

// Transposing LDS read: within each block of 16 lanes, lane i receives element (i % 4) of
// the 8-byte rows addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4 of that block.
__device__ __forceinline__ s16x4 lds_read_tr(const unsigned char *p)
{
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
}

struct MfmaPlan { int ncb, nseg, steps_per_seg; int64_t nsteps, nwg; };

// Operand tile of the banded Toeplitz matrix at row offset doff = (out time) - (in time) of
// the tile origins: element e of lane (j, q) is the tap for lag doff + j - 8q - e.
template <typename T>
__device__ __forceinline__ typename MT<T>::op_t toeplitz_operand(const uint16_t *htab, int doff, int j, int q)
{
    uint16_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = htab[doff + j - 8 * q - e + HPAD];
    typename MT<T>::op_t r;
    __builtin_memcpy(&r, v, 16);
    return r;
}

// ---------------------------------------------------------------------------- forward
template <typename T, int NK>
__global__ __launch_bounds__(256) void mfma_fwd_kernel(const T *__restrict__ x, const T *__restrict__ B,
                                                       const T *__restrict__ C, const T *__restrict__ h,
                                                       T *__restrict__ y, T *__restrict__ y2o,
                                                       T *__restrict__ bxo, Dims dm, MfmaPlan pl)
{
    typedef typename MT<T>::op_t op_t;
    __shared__ __attribute__((aligned(16))) unsigned char u_rm[STEP * UROW];
    __shared__ __attribute__((aligned(16))) unsigned char y_st[STEP * YROW];
    __shared__ uint16_t htab[4][HTAB];

    int64_t wg = blockIdx.x;
    const int cb = (int)(wg % pl.ncb); wg /= pl.ncb;
    const int seg = (int)(wg % pl.nseg);
    const int64_t b = wg / pl.nseg;

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
    const int r = l >> 3, a = l & 7;     // row layout: row 8w + r of the step, channels 8a..8a+7
    const int j = l & 15, q = l >> 4;    // matrix layout
    const int64_t d = dm.d, L = dm.L;
    const int64_t c0 = (int64_t)cb * CB;
    const int hl = dm.hl;

    // filter table of this wave's group: htab[lag + 32] = h[hl-1-lag] for 0 <= lag < hl, else 0
    {
        const int64_t cw = c0 + 16 * w;
        const int64_t grp = (cw < d) ? cw / dm.dg : 0;
        const uint16_t *hg = (const uint16_t *)h + grp * hl;
        for (int i = l; i < HTAB; i += 64) {
            const int lag = i - HPAD;
            htab[w][i] = (lag >= 0 && lag < hl) ? hg[hl - 1 - lag] : (uint16_t)0;
        }
    }
    __syncthreads();
    op_t W0[NK], W1[NK];   // output rows 0..15 / 16..31 of the step against input step s-i
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        W0[i] = toeplitz_operand<T>(htab[w], 32 * i, j, q);
        W1[i] = toeplitz_operand<T>(htab[w], 32 * i + 16, j, q);
    }

    const int64_t s_lo = (int64_t)seg * pl.steps_per_seg;
    const int64_t s_hi = (s_lo + pl.steps_per_seg < pl.nsteps) ? s_lo + pl.steps_per_seg : pl.nsteps;
    const int64_t s_first = (s_lo - (NK - 1) > 0) ? s_lo - (NK - 1) : 0;

    const bool cvalid = c0 + 8 * a < d;
    const int64_t col = b * L * d + c0 + 8 * a;            // element offset of this lane's columns
    const int row_in_step = 8 * w + r;

    op_t A[NK];
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        uint4 z = make_uint4(0u, 0u, 0u, 0u);
        __builtin_memcpy(&A[i], &z, 16);
    }

    unsigned char *u_wr = u_rm + row_in_step * UROW + 16 * a;
    const unsigned char *u_rd = u_rm + (8 * q + (j >> 2)) * UROW + (16 * w + 4 * (j & 3)) * 2;
    unsigned char *y_wr = y_st + j * YROW + (16 * w + 4 * q) * 4;
    const unsigned char *y_rd = y_st + row_in_step * YROW + 32 * a;

    uint4 xr, Br, Cr;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    auto fetch = [&](int64_t s, uint4 &xo, uint4 &Bo, uint4 &Co) {
        const int64_t t = s * STEP + row_in_step;
        xo = zero4; Bo = zero4; Co = zero4;
        if (cvalid && t < L) {
            const int64_t o = col + t * d;
            xo = *(const uint4 *)(x + o);
            Bo = *(const uint4 *)(B + o);
            if (s >= s_lo) Co = *(const uint4 *)(C + o);
        }
    };
    fetch(s_first, xr, Br, Cr);

    int64_t s = s_first;
    while (s < s_hi) {
#pragma unroll
        for (int ph = 0; ph < NK; ++ph) {
            if (s < s_hi) {
                const bool main_step = s >= s_lo;
                uint4 xn = zero4, Bn = zero4, Cn = zero4;
                if (s + 1 < s_hi) fetch(s + 1, xn, Bn, Cn);

                float xf[8], Bf[8], uf[8];
                unpack8<T>(xr, xf);
                unpack8<T>(Br, Bf);
#pragma unroll
                for (int e = 0; e < 8; ++e) uf[e] = xf[e] * Bf[e];
                const uint4 up = pack8<T>(uf);
                *(uint4 *)u_wr = up;
                const int64_t t = s * STEP + row_in_step;
                const bool store_ok = main_step && cvalid && t < L;
                if (bxo && store_ok) *(uint4 *)(bxo + col + t * d) = up;
                __syncthreads();
                {
                    const s16x4 lo = lds_read_tr(u_rd);
                    const s16x4 hi = lds_read_tr(u_rd + 4 * UROW);
                    short v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    __builtin_memcpy(&A[ph], v, 16);
                }
                if (main_step) {
                    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < NK; ++i) {
                        acc0 = MT<T>::mfma(A[(ph - i + NK) % NK], W0[i], acc0);
                        acc1 = MT<T>::mfma(A[(ph - i + NK) % NK], W1[i], acc1);
                    }
                    *(f32x4 *)y_wr = acc0;
                    *(f32x4 *)(y_wr + 16 * YROW) = acc1;
                }
                __syncthreads();
                if (store_ok) {
                    const f32x4 p0 = *(const f32x4 *)y_rd;
                    const f32x4 p1 = *(const f32x4 *)(y_rd + 16);
                    float y2f[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                    float Cf[8], yf[8];
                    unpack8<T>(Cr, Cf);
#pragma unroll
                    for (int e = 0; e < 8; ++e) yf[e] = Cf[e] * y2f[e];
                    *(uint4 *)(y + col + t * d) = pack8<T>(yf);
                    if (y2o) *(uint4 *)(y2o + col + t * d) = pack8<T>(y2f);
                }
                xr = xn; Br = Bn; Cr = Cn;
                ++s;
            }
        }
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

MfmaPlan plan(const Dims &dm, int wg_per_cu, int min_steps)
{
    MfmaPlan p;
    p.ncb = (int)((dm.d + CB - 1) / CB);
    p.nsteps = (dm.L + STEP - 1) / STEP;
    int64_t cols = dm.bs * p.ncb;
    int64_t want = ((int64_t)cu_count() * wg_per_cu + cols - 1) / cols;   // segments to fill the chip
    int64_t max_seg = p.nsteps / min_steps;
    if (max_seg < 1) max_seg = 1;
    if (want > max_seg) want = max_seg;
    if (want < 1) want = 1;
    static const char *env = getenv("GCG_MFMA_STEPS_PER_SEG");  // tuning override
    int64_t sps = (p.nsteps + want - 1) / want;
    if (env && atoi(env) > 0) sps = atoi(env);
    p.steps_per_seg = (int)sps;
    p.nseg = (int)((p.nsteps + sps - 1) / sps);
    p.nwg = dm.bs * p.nseg * p.ncb;
    return p;
}

// input steps an output step reaches back over: lags up to hl-1 from rows 0..31 of the step
int nk_for(int hl) { const int n = (hl + 30) / 32 + 1; return n > 5 ? 5 : n; }

template <typename T, int NK>
int fwd_nk(const void *x, const void *B, const void *C, const void *h, void *y, void *y2, void *bx,
           const Dims &dm, hipStream_t st)
{
    const MfmaPlan p = plan(dm, 4, 16);
    if (p.nwg > 0x7fffffffLL) return (int)hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((mfma_fwd_kernel<T, NK>), dim3((unsigned)p.nwg), dim3(256), 0, st, (const T *)x,
                       (const T *)B, (const T *)C, (const T *)h, (T *)y, (T *)y2, (T *)bx, dm, p);
    return (int)hipGetLastError();
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
    return (dtype == GCG_BF16 || dtype == GCG_F16) && dm.hl <= 128 && dm.dg % 16 == 0;
}

int mfma_fwd_launch(int dtype, const void *x, const void *B, const void *C, const void *h, void *y,
                    void *y2, void *bx, const Dims &dm, hipStream_t st)
{
    if (dtype == GCG_BF16) return fwd_t<bf16_t>(x, B, C, h, y, y2, bx, dm, st);
    if (dtype == GCG_F16) return fwd_t<f16_t>(x, B, C, h, y, y2, bx, dm, st);
    return (int)hipErrorInvalidValue;
}

bool mfma_bwd_available() { return false; }

size_t mfma_bwd_workspace(const Dims &) { return 0; }

int mfma_bwd_launch(int, const void *, const void *, const void *, const void *, const void *, void *, void *,
                    void *, void *, void *, const Dims &, hipStream_t)
{
    return (int)hipErrorNotSupported;
}

} // namespace gcg
