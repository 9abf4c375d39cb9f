// Access-pattern ceilings for the convolution kernels: the same reads and writes, no arithmetic.
//
//   ./membench            (built by `make -C savanna_amd/csrc membench`)
//
// Prints the HBM rate of (a) flat streams with R reads and W writes per element, plain and
// nontemporal, and (b) the tile walk the MFMA kernels perform -- a workgroup owns ROWB bytes of
// every row of a (bs, L, d) bf16 tensor set and walks a run of 32-row steps with a one-step
// prefetch -- for several row widths, read/write mixes, run lengths and row strides, and with
// neighbouring column blocks in or out of step, and (c) the row walk of the register-window
// kernels (a lane owns a few bytes of every row of a run).  These are the rates the
// memory system gives the kernels' access pattern; the kernels are compared with them, not
// only with the 8 TB/s nominal peak.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

template <int NT> __device__ __forceinline__ u4 ld(const u4 *p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <int NT> __device__ __forceinline__ void st(u4 *p, u4 v) { if (NT) __builtin_nontemporal_store(v, p); else *p = v; }

template <int R, int W, int NT>
__global__ __launch_bounds__(256) void flat_kernel(const u4 *a, const u4 *b, const u4 *c, const u4 *e, u4 *y, u4 *z, u4 *w, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        u4 v = ld<NT>(a + i);
        if (R > 1) v ^= ld<NT>(b + i);
        if (R > 2) v ^= ld<NT>(c + i);
        if (R > 3) v ^= ld<NT>(e + i);
        if (W > 0) st<NT>(y + i, v); else if (v.x == 0x12345678u) y[0] = v;
        if (W > 1) st<NT>(z + i, v);
        if (W > 2) st<NT>(w + i, v);
    }
}

// THREADS lanes cover (THREADS*16/ROWB) rows of ROWB bytes per step
template <int THREADS, int ROWB, int R, int W>
__global__ __launch_bounds__(THREADS) void tile_kernel(const char *a, const char *b, const char *c, const char *e, char *y, char *z, char *w,
                                                       int64_t L, int64_t rowbytes, int ncb, int nseg, int steps, int skew)
{
    int64_t id = blockIdx.x;
    const int cb = id % ncb; id /= ncb;
    const int seg = id % nseg;
    const int64_t bb = id / nseg;
    constexpr int LPR = ROWB / 16, RPS = THREADS / LPR;
    const int r = threadIdx.x / LPR, l = threadIdx.x % LPR;
    // skew > 0: column block cb starts its run skew*cb steps in and wraps round (same rows, other order)
    const int64_t base = bb * L * rowbytes + (int64_t)cb * ROWB + l * 16 + ((int64_t)seg * steps * RPS + r) * rowbytes;
    const int phi = (int)((int64_t)cb * skew % steps);
    int64_t o = base + (int64_t)phi * RPS * rowbytes;
    u4 v0 = ld<1>((const u4 *)(a + o)), v1 = v0, v2 = v0, v3 = v0;
    if (R > 1) v1 = ld<1>((const u4 *)(b + o));
    if (R > 2) v2 = ld<1>((const u4 *)(c + o));
    if (R > 3) v3 = ld<1>((const u4 *)(e + o));
    for (int s = 0; s < steps; ++s) {
        const int64_t on = base + (int64_t)((s + 1 + phi) % steps) * RPS * rowbytes;
        u4 n0 = v0, n1 = v1, n2 = v2, n3 = v3;
        if (s + 1 < steps) {
            n0 = ld<1>((const u4 *)(a + on));
            if (R > 1) n1 = ld<1>((const u4 *)(b + on));
            if (R > 2) n2 = ld<1>((const u4 *)(c + on));
            if (R > 3) n3 = ld<1>((const u4 *)(e + on));
        }
        const u4 t = v0 ^ v1 ^ v2 ^ v3;
        st<1>((u4 *)(y + o), t);
        if (W > 1) st<1>((u4 *)(z + o), t ^ v1);
        if (W > 2) st<1>((u4 *)(w + o), t ^ v2);
        v0 = n0; v1 = n1; v2 = n2; v3 = n3; o = on;
    }
}

// The register-window kernels' pattern: a lane owns VB bytes of every row and walks a run of ts rows,
// four rows fetched together one batch ahead; a workgroup's 256 lanes cover 256*VB contiguous bytes.
template <int VB, int R, int W>
__global__ __launch_bounds__(256) void walk_kernel(const char *a, const char *b, const char *c, const char *e, char *y, char *z, char *w,
                                                   int64_t L, int64_t rowbytes, int ncvb, int nseg, int ts)
{
    typedef uint32_t vec_t __attribute__((ext_vector_type(VB / 4)));
    int64_t id = blockIdx.x;
    const int cvb = id % ncvb; id /= ncvb;
    const int seg = id % nseg;
    const int64_t bb = id / nseg;
    int64_t o = (bb * L + (int64_t)seg * ts) * rowbytes + ((int64_t)cvb * 256 + threadIdx.x) * VB;
    if (((int64_t)cvb * 256 + threadIdx.x) * VB >= rowbytes) return;
    vec_t v[2][4][4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        v[0][k][0] = __builtin_nontemporal_load((const vec_t *)(a + o + k * rowbytes));
        if (R > 1) v[0][k][1] = __builtin_nontemporal_load((const vec_t *)(b + o + k * rowbytes));
        if (R > 2) v[0][k][2] = __builtin_nontemporal_load((const vec_t *)(c + o + k * rowbytes));
        if (R > 3) v[0][k][3] = __builtin_nontemporal_load((const vec_t *)(e + o + k * rowbytes));
    }
    for (int t = 0; t < ts; t += 8) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int cur = half, nxt = half ^ 1;
            const int64_t on = o + 4 * rowbytes;
            if (t + 4 * half + 4 < ts) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v[nxt][k][0] = __builtin_nontemporal_load((const vec_t *)(a + on + k * rowbytes));
                    if (R > 1) v[nxt][k][1] = __builtin_nontemporal_load((const vec_t *)(b + on + k * rowbytes));
                    if (R > 2) v[nxt][k][2] = __builtin_nontemporal_load((const vec_t *)(c + on + k * rowbytes));
                    if (R > 3) v[nxt][k][3] = __builtin_nontemporal_load((const vec_t *)(e + on + k * rowbytes));
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                vec_t r = v[cur][k][0];
                if (R > 1) r ^= v[cur][k][1];
                if (R > 2) r ^= v[cur][k][2];
                if (R > 3) r ^= v[cur][k][3];
                __builtin_nontemporal_store(r, (vec_t *)(y + o + k * rowbytes));
                if (W > 1) __builtin_nontemporal_store(r ^ v[cur][k][0], (vec_t *)(z + o + k * rowbytes));
                if (W > 2) __builtin_nontemporal_store(r ^ r, (vec_t *)(w + o + k * rowbytes));
            }
            o = on;
        }
    }
}

static hipEvent_t e0, e1;
template <typename F> static void timeit(const char *name, double bytes, F launch)
{
    for (int i = 0; i < 3; ++i) launch();
    CK(hipDeviceSynchronize());
    float best = 1e9f, tot = 0.f;
    const int K = 20;
    for (int i = 0; i < K; ++i) {
        CK(hipEventRecord(e0)); launch(); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        tot += ms; if (ms < best) best = ms;
    }
    printf("%-58s avg %7.1f us  %5.0f GB/s  (best %5.0f)\n", name, tot / K * 1e3, bytes / (tot / K) / 1e6, bytes / best / 1e6);
    fflush(stdout);
}

int main()
{
    const int64_t bs = 2, L = 8192, d = 4096;            // the Evo2-7B layer shape, bf16
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int pad = 0; pad < 2; ++pad) {
        const int64_t rowbytes = d * 2 + (pad ? 256 : 0); // pad = 1: row stride no longer a power of two
        const int64_t bytes = bs * L * rowbytes;
        char *p[7];
        for (int i = 0; i < 7; ++i) { CK(hipMalloc(&p[i], bytes)); CK(hipMemset(p[i], i + 1, bytes)); }
        const double n1 = (double)bs * L * d * 2;
        char nm[128];
        if (!pad) {
            const int64_t n16 = bytes / 16;
            u4 **q = (u4 **)p;
            timeit("flat 1R0W", 1 * n1, [&] { flat_kernel<1, 0, 0><<<8192, 256>>>(q[0], q[1], q[2], q[3], q[4], q[5], q[6], n16); });
            timeit("flat 1R1W", 2 * n1, [&] { flat_kernel<1, 1, 0><<<8192, 256>>>(q[0], q[1], q[2], q[3], q[4], q[5], q[6], n16); });
            timeit("flat 1R1W nontemporal", 2 * n1, [&] { flat_kernel<1, 1, 1><<<8192, 256>>>(q[0], q[1], q[2], q[3], q[4], q[5], q[6], n16); });
            timeit("flat 3R1W", 4 * n1, [&] { flat_kernel<3, 1, 0><<<8192, 256>>>(q[0], q[1], q[2], q[3], q[4], q[5], q[6], n16); });
            timeit("flat 3R1W nontemporal", 4 * n1, [&] { flat_kernel<3, 1, 1><<<8192, 256>>>(q[0], q[1], q[2], q[3], q[4], q[5], q[6], n16); });
            timeit("flat 4R3W nontemporal", 7 * n1, [&] { flat_kernel<4, 3, 1><<<8192, 256>>>(q[0], q[1], q[2], q[3], q[4], q[5], q[6], n16); });
        }
        auto tile = [&](auto kern, int threads, int rowb, int rd, int wr, int steps, int skew = 0) {
            const int ncb = (int)(d * 2 / rowb), rps = threads * 16 / rowb, nseg = (int)(L / rps / steps);
            snprintf(nm, sizeof nm, "tile %dR%dW rows of %3d B, %4d threads, %3d steps%s, stride %lld", rd, wr, rowb, threads, steps, skew ? ", skewed" : "", (long long)rowbytes);
            timeit(nm, (rd + wr) * n1, [&] { kern<<<(unsigned)(bs * nseg * ncb), threads>>>(p[0], p[1], p[2], p[3], p[4], p[5], p[6], L, rowbytes, ncb, nseg, steps, skew); });
        };
        tile(tile_kernel<256, 128, 3, 1>, 256, 128, 3, 1, 128);
        tile(tile_kernel<512, 256, 3, 1>, 512, 256, 3, 1, 64);
        tile(tile_kernel<1024, 512, 3, 1>, 1024, 512, 3, 1, 32);
        tile(tile_kernel<256, 128, 4, 3>, 256, 128, 4, 3, 128);
        tile(tile_kernel<512, 256, 4, 3>, 512, 256, 4, 3, 64);
        tile(tile_kernel<1024, 512, 4, 3>, 1024, 512, 4, 3, 32);
        // the same walks cut into shorter runs: 2 and 4 workgroups resident per CU instead of 1
        tile(tile_kernel<512, 256, 4, 3>, 512, 256, 4, 3, 32);
        tile(tile_kernel<512, 256, 4, 3>, 512, 256, 4, 3, 16);
        tile(tile_kernel<256, 128, 4, 3>, 256, 128, 4, 3, 32);
        tile(tile_kernel<256, 128, 4, 3>, 256, 128, 4, 3, 16);
        // column blocks out of step with their neighbours
        tile(tile_kernel<512, 256, 4, 3>, 512, 256, 4, 3, 64, 1);
        tile(tile_kernel<512, 256, 4, 3>, 512, 256, 4, 3, 64, 5);
        if (!pad) {
            auto walk = [&](auto kern, int vb, int rd, int wr, int ts) {
                const int ncvb = (int)((rowbytes / vb + 255) / 256), nseg = (int)(L / ts);
                snprintf(nm, sizeof nm, "walk %dR%dW %2d B per lane, runs of %4d rows", rd, wr, vb, ts);
                timeit(nm, (rd + wr) * n1, [&] { kern<<<(unsigned)(bs * nseg * ncvb), 256>>>(p[0], p[1], p[2], p[3], p[4], p[5], p[6], L, rowbytes, ncvb, nseg, ts); });
            };
            walk(walk_kernel<8, 3, 1>, 8, 3, 1, 128);
            walk(walk_kernel<16, 3, 1>, 16, 3, 1, 128);
            walk(walk_kernel<8, 4, 3>, 8, 4, 3, 128);
            walk(walk_kernel<16, 4, 3>, 16, 4, 3, 128);
        }
        for (int i = 0; i < 7; ++i) CK(hipFree(p[i]));
    }
    {   // the featurizer's tensors: (2, 8192, 12288) bf16, one read and one written (forward), two read and one written (backward)
        const int64_t rowbytes = 3 * d * 2, bytes = bs * L * rowbytes;
        char *p[3];
        for (int i = 0; i < 3; ++i) { CK(hipMalloc(&p[i], bytes)); CK(hipMemset(p[i], i + 1, bytes)); }
        const double n3 = (double)bytes;
        char nm[128];
        const int64_t n16 = bytes / 16;
        u4 **q = (u4 **)p;
        timeit("featurizer shape: flat 1R1W", 2 * n3, [&] { flat_kernel<1, 1, 0><<<8192, 256>>>(q[0], q[1], q[1], q[1], q[2], q[2], q[2], n16); });
        timeit("featurizer shape: flat 1R1W nontemporal", 2 * n3, [&] { flat_kernel<1, 1, 1><<<8192, 256>>>(q[0], q[1], q[1], q[1], q[2], q[2], q[2], n16); });
        timeit("featurizer shape: flat 2R1W nontemporal", 3 * n3, [&] { flat_kernel<2, 1, 1><<<8192, 256>>>(q[0], q[1], q[1], q[1], q[2], q[2], q[2], n16); });
        auto walk = [&](auto kern, int vb, int rd, int wr, int ts) {
            const int ncvb = (int)((rowbytes / vb + 255) / 256), nseg = (int)(L / ts);
            snprintf(nm, sizeof nm, "featurizer shape: walk %dR%dW %2d B per lane, runs of %4d rows", rd, wr, vb, ts);
            timeit(nm, (rd + wr) * n3, [&] { kern<<<(unsigned)(bs * nseg * ncvb), 256>>>(p[0], p[1], p[1], p[1], p[2], p[2], p[2], L, rowbytes, ncvb, nseg, ts); });
        };
        walk(walk_kernel<8, 1, 1>, 8, 1, 1, 128);
        walk(walk_kernel<16, 1, 1>, 16, 1, 1, 128);
        walk(walk_kernel<8, 2, 1>, 8, 2, 1, 128);
        walk(walk_kernel<16, 2, 1>, 16, 2, 1, 128);
        walk(walk_kernel<8, 1, 1>, 8, 1, 1, 1024);
        walk(walk_kernel<8, 2, 1>, 8, 2, 1, 1024);
        for (int i = 0; i < 3; ++i) CK(hipFree(p[i]));
    }
    return 0;
}
