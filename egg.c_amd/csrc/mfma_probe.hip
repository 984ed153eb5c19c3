// mfma_probe.hip -- what rate of v_mfma_i32_32x32x32_i8 this GPU sustains, measured: a loop of independent MFMAs on
// register operands, nothing else (no memory, no LDS), two waves per SIMD on every CU.  With all-zero operands the
// matrix pipes run at the published rate; with random operand bytes the same loop is slower, because the clock drops
// under the power the switching draws.  bench.py reports both next to the kernels' rates, which are computed on real
// (random-like) int8 data.  Prints one JSON line.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// VARY = false: the same two operand registers feed every MFMA; VARY = true: eight different operand pairs in rotation,
// as in a real product where every MFMA brings new operand bytes
template <bool VARY>
__global__ void __launch_bounds__(256) k_probe(const int *seed, int *out, int iters) {
    // seed[0] = 0: zero operands; otherwise per-lane pseudo-random bytes
    const int h = (int)((threadIdx.x + 77u + blockIdx.x * 256u) * 0x85EBCA6Bu) * seed[0];
    v4i x[8], y[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int hi = VARY ? h * (2 * i + 1) + i * 0x3C6EF372 * seed[0] : h;
        x[i] = v4i{hi, hi * 31, hi * 131, hi * 313}; y[i] = v4i{hi * 17, hi * 5, hi * 1001, hi * 7};
    }
    v16i a = {0}, b = {0}, c = {0}, d = {0};
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const int i0 = VARY ? (u & 7) : 0, i1 = VARY ? ((u * 3 + 1) & 7) : 0;
            a = __builtin_amdgcn_mfma_i32_32x32x32_i8(x[i0], y[i1], a, 0, 0, 0); b = __builtin_amdgcn_mfma_i32_32x32x32_i8(y[i0], x[i1], b, 0, 0, 0);
            c = __builtin_amdgcn_mfma_i32_32x32x32_i8(x[i1], x[i0], c, 0, 0, 0); d = __builtin_amdgcn_mfma_i32_32x32x32_i8(y[i1], y[i0], d, 0, 0, 0);
        }
    }
    // the results must look used; seed[1] is never this value
    if (seed[1] == 0x5EED5EED) out[threadIdx.x] = a[0] + b[1] + c[2] + d[3];
}

template <bool VARY>
static double run(const int *d_seed, int *d_out, int cus, int iters) {
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    const dim3 grid(2 * cus), block(256);
    hipLaunchKernelGGL(k_probe<VARY>, grid, block, 0, 0, d_seed, d_out, 50);
    hipEventRecord(e0);
    hipLaunchKernelGGL(k_probe<VARY>, grid, block, 0, 0, d_seed, d_out, iters);
    hipEventRecord(e1); hipEventSynchronize(e1);
    float ms = 0.f; hipEventElapsedTime(&ms, e0, e1);
    hipEventDestroy(e0); hipEventDestroy(e1);
    const double mfmas = (double)grid.x * 4 * iters * 64.0;
    return mfmas * 65536.0 / (ms * 1e-3);
}

int main() {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0) != hipSuccess || cus < 1) { fprintf(stderr, "no GPU\n"); return 1; }
    int *d_seed, *d_out, h[2] = {0, 0};
    if (hipMalloc(&d_seed, 8) != hipSuccess || hipMalloc(&d_out, 1024) != hipSuccess) return 1;
    hipMemcpy(d_seed, h, 8, hipMemcpyHostToDevice);
    const double zero = run<false>(d_seed, d_out, cus, 3000);
    h[0] = 1; hipMemcpy(d_seed, h, 8, hipMemcpyHostToDevice);
    const double rnd = run<false>(d_seed, d_out, cus, 3000);
    const double vary = run<true>(d_seed, d_out, cus, 3000);
    if (hipDeviceSynchronize() != hipSuccess) return 1;
    printf("{\"instruction\": \"v_mfma_i32_32x32x32_i8\", \"compute_units\": %d, \"waves_per_simd\": 2, \"zero_operands_TOPs\": %.1f, \"random_operands_TOPs\": %.1f, \"random_operands_changing_every_mfma_TOPs\": %.1f}\n",
           cus, zero / 1e12, rnd / 1e12, vary / 1e12);
    return 0;
}
