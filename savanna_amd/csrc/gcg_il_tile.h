// Pieces shared by the kernels that work on interleaved (C, B, x) rows: the lane layout of such rows, the
// conversion between a lane's row pieces and per-tensor values, and the featurizer in front of the operator.
// Included by gcg_mfma_il.hip and gcg_mixer_mr.hip.
#pragma once
#include "gcg_mfma_tile.h"

namespace gcg {
namespace {

template <typename T, int NW> struct GeoIL {
    static constexpr int CH = 4 / MT<T>::ES;                    // channels per lane
    static constexpr int LPR = 16 * NW / CH;                    // lanes per row
    static constexpr int RP = 64 * NW / LPR;                    // rows covered by one pass of the workgroup
    static constexpr int NR = STEP / RP;                        // rows per lane and step
    static_assert(NR * CH == 8, "a lane holds eight elements per tensor and step");
};

// A lane's pieces of one step <-> per-tensor values; element e = k * CH + c is row k, channel c.
// 16 bits: a piece holds [C0 B0 | x0 C1 | B1 x1]; fp32: [C | B | x].
template <typename T, int NR>
__device__ __forceinline__ void il_split(const u32x3 (&p)[NR], float (&xf)[8], float (&Bf)[8], float (&Cf)[8])
{
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        if constexpr (MT<T>::ES == 4) {
            Cf[k] = __uint_as_float(p[k][0]);
            Bf[k] = __uint_as_float(p[k][1]);
            xf[k] = __uint_as_float(p[k][2]);
        } else {
            MT<T>::unpack2(p[k][0], Cf[2 * k], Bf[2 * k]);
            MT<T>::unpack2(p[k][1], xf[2 * k], Cf[2 * k + 1]);
            MT<T>::unpack2(p[k][2], Bf[2 * k + 1], xf[2 * k + 1]);
        }
    }
}
// 16-bit pieces of NR = 4 rows -> the row vectors of x and B as they are (element e = 2 k + c, no conversion) and C
// as fp32
template <typename T>
__device__ __forceinline__ void il_split_rows(const u32x3 (&p)[4], Row<T> &xr, Row<T> &Br, float (&Cf)[8])
{
    static_assert(MT<T>::ES == 2, "16-bit pieces");
    uint32_t xw[4], Bw[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float skip;
        MT<T>::unpack2(p[k][0], Cf[2 * k], skip);
        MT<T>::unpack2(p[k][1], skip, Cf[2 * k + 1]);
        xw[k] = (p[k][1] & 0xffffu) | (p[k][2] & 0xffff0000u);          // x0 | x1
        Bw[k] = __builtin_amdgcn_alignbit(p[k][2], p[k][0], 16);        // B0 | B1
    }
    xr.w[0] = make_uint4(xw[0], xw[1], xw[2], xw[3]);
    Br.w[0] = make_uint4(Bw[0], Bw[1], Bw[2], Bw[3]);
}
template <typename T, int NR>
__device__ __forceinline__ void il_join(const float (&xf)[8], const float (&Bf)[8], const float (&Cf)[8],
                                        u32x3 (&p)[NR])
{
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        if constexpr (MT<T>::ES == 4) {
            p[k][0] = __float_as_uint(Cf[k]);
            p[k][1] = __float_as_uint(Bf[k]);
            p[k][2] = __float_as_uint(xf[k]);
        } else {
            p[k][0] = MT<T>::pack2(Cf[2 * k], Bf[2 * k]);
            p[k][1] = MT<T>::pack2(xf[2 * k], Cf[2 * k + 1]);
            p[k][2] = MT<T>::pack2(Bf[2 * k + 1], xf[2 * k + 1]);
        }
    }
}
// the 4-byte unit of a plain tensor: CH elements of one row
template <typename T> __device__ __forceinline__ uint32_t pack_unit(const float *f)
{
    if constexpr (MT<T>::ES == 4) return __float_as_uint(f[0]);
    else return MT<T>::pack2(f[0], f[1]);
}
// one lane's unit of a row (CH channels) into a matrix-operand tile, in the tile's own element format
template <typename T> __device__ __forceinline__ void store_operand_unit(unsigned char *p, int urow, const float *f)
{
    typedef MT<T> M;
    if constexpr (M::SPLIT && M::ES == 4) {
        uint16_t v[M::NPA];
        M::template split<M::NPA>(f[0], v);
#pragma unroll
        for (int m = 0; m < M::NPA; ++m) *(uint16_t *)(p + m * M::plane(urow)) = v[m];
    } else if constexpr (M::SPLIT) {
        // the two channels plane by plane as pairs (MTSplit::split on each, with one packed conversion per plane)
        float r0 = f[0], r1 = f[1];
#pragma unroll
        for (int m = 0; m < M::NPA; ++m) {
            const uint32_t pk = pack_bf16x2(r0, r1);
            *(uint32_t *)(p + m * M::plane(urow)) = pk;
            if (m + 1 < M::NPA) {
                r0 -= __uint_as_float(pk << 16);
                r1 -= __uint_as_float(pk & 0xffff0000u);
            }
        }
    } else {
        *(uint32_t *)p = M::pack2(f[0], f[1]);
    }
}
// NR units in a row vector: unpack8 then yields them in element order e = k * CH + c
template <typename T, int NR> __device__ __forceinline__ Row<T> units_row(const uint32_t (&u)[NR])
{
    Row<T> r;
    r.w[0] = make_uint4(u[0], u[1], u[2], u[3]);
    if constexpr (NR == 8) r.w[1] = make_uint4(u[4], u[5], u[6], u[7]);
    return r;
}

// ---- featurizer in front of the operator ------------------------------------------------------
// The features need not be given: a kernel with KF > 0 takes the projection output instead and makes every
// row of (C, B, x) on the way -- a short causal depthwise convolution with one filter per feature channel
// (wfeat: (3 * d, 1, kf), kf <= KF), rounded to T as if the featurizer had stored it and the kernel had read
// it back.  A lane then owns NR consecutive rows of a step instead of rows RP apart, and also fetches the
// KF-1 rows before them: rows its neighbours own and request at the same time, so they cost cache hits, not
// memory traffic.
// tap[m][v]: what feature channel f0 + v multiplies the row KF-1-m rows in the past with (zero where kf < KF)
template <typename T, int KF, int NV>
__device__ __forceinline__ void load_feat_taps(const T *wfeat, int64_t f0, int kf, float (&tap)[KF][NV])
{
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int m = 0; m < KF; ++m) {
            const int kk = m - (KF - kf);                // index into the kf taps of the filter
            const float t = Elem<T>::load(wfeat + (f0 + v) * kf + (kk >= 0 ? kk : 0));
            tap[m][v] = kk >= 0 ? t : 0.f;
        }
}
// (C, B, x) of a lane's NR rows from the KF-1 + NR fetched pieces of the projection output, oldest row first;
// sums in the featurizer kernel's order (oldest sample first, fp32) and rounded to T like its output
template <typename T, int NR, int KF>
__device__ __forceinline__ void featurized_rows(const u32x3 (&p)[KF - 1 + NR], const float (&tap)[KF][3 * (4 / MT<T>::ES)],
                                                float (&xf)[8], float (&Bf)[8], float (&Cf)[8])
{
    typedef MT<T> M;
    constexpr int NV = 3 * (4 / M::ES);
    float rv[KF - 1 + NR][NV];
#pragma unroll
    for (int k = 0; k < KF - 1 + NR; ++k) {
        if constexpr (M::ES == 4) {
            rv[k][0] = __uint_as_float(p[k][0]); rv[k][1] = __uint_as_float(p[k][1]); rv[k][2] = __uint_as_float(p[k][2]);
        } else {
            M::unpack2(p[k][0], rv[k][0], rv[k][1]);
            M::unpack2(p[k][1], rv[k][2], rv[k][3]);
            M::unpack2(p[k][2], rv[k][4], rv[k][5]);
        }
    }
    u32x3 fp[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        float acc[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[v] = 0.f;
#pragma unroll
        for (int m = 0; m < KF; ++m)
#pragma unroll
            for (int v = 0; v < NV; ++v) acc[v] = fmaf(tap[m][v], rv[k + m][v], acc[v]);
        if constexpr (M::ES == 4) {
            fp[k][0] = __float_as_uint(acc[0]); fp[k][1] = __float_as_uint(acc[1]); fp[k][2] = __float_as_uint(acc[2]);
        } else {
            fp[k][0] = M::pack2(acc[0], acc[1]); fp[k][1] = M::pack2(acc[2], acc[3]); fp[k][2] = M::pack2(acc[4], acc[5]);
        }
    }
    il_split<T, NR>(fp, xf, Bf, Cf);
}

} // namespace
} // namespace gcg
