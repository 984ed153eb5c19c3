// egg_update.hip -- fitness, vote reconstruction and the ES-AdamW step on gfx950.
//
// Reference: compute_fitness_kernel, apply_adam_update, update_matrix_adam_kernel and
// update_vector_adam_kernel, full_cuda_train_transformer_adam_mgpu.cu:1031-1152 ("mgpu.cu").
// The reference recomputes two noise hashes per (weight, pair); here the (rows+cols) x pairs noise
// panels are generated once per matrix and the vote  sum_p fit_p A_p[n] B_p[k]  is an int8 MFMA GEMM
// over the population axis whose epilogue applies AdamW in place (blocked element order).
#include "egg_device.h"
#include "egg_launch.h"

#pragma clang fp contract(off)

__global__ void k_noise_fill(uint32_t seed, uint32_t first, int n, int mask, int8_t *out) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (int8_t)noise_from_hash(seed, first + (uint32_t)i, mask);
}
hipError_t egg_launch_noise_fill(uint32_t seed, uint32_t first, int n, int mask, int8_t *out, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_noise_fill, dim3((n + 255) / 256), dim3(256), 0, s, seed, first, n, mask, out);
    return hipGetLastError();
}

__global__ void k_zero_u64(unsigned long long *p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0ull;
}
hipError_t egg_launch_zero_u64(unsigned long long *p, int64_t n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_zero_u64, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n);
    return hipGetLastError();
}

// accum_loss[p] = (int32_t) my_loss   (mgpu.cu:1028)
__global__ void k_loss_finalize(const unsigned long long *acc, int32_t *loss, int first, int count) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) loss[first + i] = (int32_t)(long long)acc[first + i];
}
hipError_t egg_launch_loss_finalize(const unsigned long long *acc, int32_t *loss, int first, int count, hipStream_t s) {
    if (count <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_loss_finalize, dim3((count + 255) / 256), dim3(256), 0, s, acc, loss, first, count);
    return hipGetLastError();
}

// mgpu.cu:1031-1036
__global__ void k_fitness(const int32_t *loss, int32_t *fit, int pairs) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= pairs) return;
    int32_t p = loss[2 * i], n = loss[2 * i + 1];
    fit[i] = (p < n) ? 1 : ((n < p) ? -1 : 0);
}
hipError_t egg_launch_fitness(const int32_t *loss, int32_t *fit, int pairs, hipStream_t s) {
    if (pairs <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_fitness, dim3((pairs + 255) / 256), dim3(256), 0, s, loss, fit, pairs);
    return hipGetLastError();
}

// apply_adam_update (mgpu.cu:1040-1064); every float operation is a single IEEE-754 operation
struct AdamHyper { float b1, b2, eps, wd; };
__device__ __forceinline__ int adam_apply(float &m, float &v, float &acc, int &w, float gr, float lr, const AdamHyper &h) {
    float t1 = h.b1 * m; float t2 = (1.0f - h.b1) * gr; m = t1 + t2;
    float t3 = h.b2 * v; float gg = gr * gr; float t4 = (1.0f - h.b2) * gg; v = t3 + t4;
    float den = sqrtf(v) + h.eps;
    float q = m / den;
    float wdw = h.wd * (float)w;
    float step = (-lr) * (q + wdw);
    acc += step;
    int change = 0;
    if (acc >= 1.0f) {
        if (w < 127) { w++; change = 1; acc -= 1.0f; } else acc = 1.0f;
    } else if (acc <= -1.0f) {
        if (w > -127) { w--; change = 1; acc += 1.0f; } else acc = -1.0f;
    }
    return change;
}

// noise panels, pair index contiguous: pa[n][p] = fit_p * A_p[n], pb[k][p] = B_p[k]; zero beyond `pairs`
__global__ void k_panels(UpdParams p) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = (int64_t)(p.rows + p.cols) * p.pairs_pad;
    if (i >= total) return;
    int pr = (int)(i % p.pairs_pad); int r = (int)(i / p.pairs_pad);
    int val = 0;
    if (pr < p.pairs) {
        uint32_t s = *p.d_seed + (uint32_t)pr + (uint32_t)p.seed_base;
        if (r < p.cols) val = p.fit[pr] * noise_from_hash(s + p.off_a, r, p.mask);
        else val = noise_from_hash(s + p.off_b, r - p.cols, p.mask);
    }
    if (r < p.cols) p.panel_a[(size_t)r * p.pairs_pad + pr] = (int8_t)val;
    else p.panel_b[(size_t)(r - p.cols) * p.pairs_pad + pr] = (int8_t)val;
}

// one wave per 32(k) x 32(n) tile of the vote matrix; reduction over pairs on the MFMA
__global__ void __launch_bounds__(EGG_THREADS) k_vote_adam(UpdParams p) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const int tiles_n = p.cols / 32, tiles = (p.rows / 32) * tiles_n;
    const int tile = blockIdx.x * EGG_WAVES + wave;
    if (tile >= tiles) return;
    const int k0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
    const int8_t *pb = p.panel_b + (size_t)(k0 + j) * p.pairs_pad + 16 * g;
    const int8_t *pa = p.panel_a + (size_t)(n0 + j) * p.pairs_pad + 16 * g;
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    for (int s = 0; s < p.pairs_pad; s += 32) {
        v4i a = *reinterpret_cast<const v4i *>(pb + s);
        v4i b = *reinterpret_cast<const v4i *>(pa + s);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc, 0, 0, 0);
    }
    // lane (n = n0 + j, half g), register 4q+e -> k = k0 + 8q + 4g + e ; blocked index of (k, n) (mgpu.cu:1085-1089)
    const int n = n0 + j;
    const float lr = p.votes_out ? 0.f : (*p.d_lr) * p.lr_scale;
    const AdamHyper hy = {p.beta1, p.beta2, p.eps, p.wd};
    int changes = 0;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const size_t idx0 = ((size_t)((k0 >> 2) + 2 * q + g) * p.cols + n) * 4;
        if (p.votes_out) {
            v4i o4;
#pragma unroll
            for (int e = 0; e < 4; e++) o4[e] = acc[4 * q + e];
            *reinterpret_cast<v4i *>(p.votes_out + idx0) = o4;
            continue;
        }
        int w4 = *reinterpret_cast<const int *>(p.W + idx0);
        float st[12];
        float4 *sp = reinterpret_cast<float4 *>(p.state + idx0 * 3);
        float4 s0 = sp[0], s1 = sp[1], s2 = sp[2];
        st[0] = s0.x; st[1] = s0.y; st[2] = s0.z; st[3] = s0.w; st[4] = s1.x; st[5] = s1.y; st[6] = s1.z; st[7] = s1.w;
        st[8] = s2.x; st[9] = s2.y; st[10] = s2.z; st[11] = s2.w;
        int wv[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            wv[e] = sx8(w4, e);
            changes += adam_apply(st[3 * e], st[3 * e + 1], st[3 * e + 2], wv[e], -(float)acc[4 * q + e], lr, hy);
        }
        *reinterpret_cast<int *>(p.W + idx0) = pack4(wv[0], wv[1], wv[2], wv[3]);
        sp[0] = make_float4(st[0], st[1], st[2], st[3]);
        sp[1] = make_float4(st[4], st[5], st[6], st[7]);
        sp[2] = make_float4(st[8], st[9], st[10], st[11]);
    }
    if (!p.votes_out) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) changes += __shfl_xor(changes, off, 64);
        if (lane == 0 && changes) atomicAdd(p.counter, (unsigned long long)changes);
    }
}

hipError_t egg_launch_update_matrix(const UpdParams &p, hipStream_t s) {
    if (p.rows % 32 || p.cols % 32 || p.pairs_pad % 32) return hipErrorInvalidValue;
    int64_t total = (int64_t)(p.rows + p.cols) * p.pairs_pad;
    hipLaunchKernelGGL(k_panels, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, p);
    int tiles = (p.rows / 32) * (p.cols / 32);
    hipLaunchKernelGGL(k_vote_adam, dim3((tiles + EGG_WAVES - 1) / EGG_WAVES), dim3(EGG_THREADS), 0, s, p);
    return hipGetLastError();
}

// update_vector_adam_kernel (mgpu.cu:1114-1152): one wave per element, lanes stride over pairs
__global__ void __launch_bounds__(EGG_THREADS) k_vector_adam(UpdParams p) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int idx = blockIdx.x * EGG_WAVES + wave;
    if (idx >= p.cols) return;
    const uint32_t base = *p.d_seed + (uint32_t)p.seed_base;
    int vote = 0;
    for (int pr = lane; pr < p.pairs; pr += 64) {
        int f = p.fit[pr];
        if (f == 0) continue;
        uint32_t s = base + (uint32_t)pr;
        vote += f * noise_from_hash(s + p.off_a, idx, p.mask) * noise_from_hash(s + p.off_b, idx, p.mask);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) vote += __shfl_xor(vote, off, 64);
    if (lane == 0) {
        const AdamHyper hy = {p.beta1, p.beta2, p.eps, p.wd};
        const float lr = (*p.d_lr) * p.lr_scale;
        float *st = p.state + (size_t)idx * 3;
        float m = st[0], v = st[1], acc = st[2];
        int w = p.W[idx];
        int ch = adam_apply(m, v, acc, w, -(float)vote, lr, hy);
        p.W[idx] = (int8_t)w; st[0] = m; st[1] = v; st[2] = acc;
        if (ch) atomicAdd(p.counter, 1ull);
    }
}
hipError_t egg_launch_update_vector(const UpdParams &p, hipStream_t s) {
    hipLaunchKernelGGL(k_vector_adam, dim3((p.cols + EGG_WAVES - 1) / EGG_WAVES), dim3(EGG_THREADS), 0, s, p);
    return hipGetLastError();
}

// canonical blocked weights -> fragment-major copy consumed by the GEMM kernels (layout in egg_device.h)
__global__ void k_swizzle(const uint32_t *src, v4i *dst, int K, int N, int B, int nat) {
    int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= K * N / 16) return;
    const int per_block = B * B / 16;
    int block = c / per_block, idx = c % per_block;
    int p = idx / B, n = idx % B, kb = block / (N / B), nb = block % (N / B), ks = p >> 1, g = p & 1;
    v4i v;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        int kq = (kb * B) / 4 + 8 * ks + (nat ? (4 * g + q) : (2 * q + g));
        v[q] = (int)src[(size_t)kq * N + nb * B + n];
    }
    dst[c] = v;
}
hipError_t egg_launch_swizzle(const int8_t *W, int8_t *Wf, int K, int N, int B, int nat, hipStream_t s) {
    if (K % B || N % B || B % 32) return hipErrorInvalidValue;
    int chunks = K * N / 16;
    hipLaunchKernelGGL(k_swizzle, dim3((chunks + 255) / 256), dim3(256), 0, s, reinterpret_cast<const uint32_t *>(W),
                       reinterpret_cast<v4i *>(Wf), K, N, B, nat);
    return hipGetLastError();
}
