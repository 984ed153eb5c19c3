// egg_update.hip -- fitness, vote reconstruction and the ES-AdamW step on gfx950.
//
// Reference: compute_fitness_kernel, apply_adam_update, update_matrix_adam_kernel and
// update_vector_adam_kernel, full_cuda_train_transformer_adam_mgpu.cu:1031-1152 ("mgpu.cu").
// The reference recomputes two noise hashes per (weight, pair); here the (rows+cols) x pairs noise
// panels are generated once per matrix and the vote  sum_p fit_p A_p[n] B_p[k]  is an int8 MFMA GEMM
// over the population axis whose epilogue applies AdamW in place (blocked element order).
#include "../../include/egg_hip.h"
#include "egg_device.h"
#include "egg_launch.h"
#include <mutex>
#include <string>

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
struct AdamHyper { float b1, b2, eps, wd; int limit; };     // limit: the weight saturates at +-limit (127 in the reference)
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
        if (w < h.limit) { w++; change = 1; acc -= 1.0f; } else acc = 1.0f;
    } else if (acc <= -1.0f) {
        if (w > -h.limit) { w--; change = 1; acc += 1.0f; } else acc = -1.0f;
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

// One workgroup per 32(k) x 32(n) tile of the vote matrix.  The reduction over pairs runs on the MFMA, split four
// ways over the waves (wave w takes the 32-pair steps w, w+4, ...; integer sums do not depend on the order); the
// partial tiles meet in LDS and wave q finishes the four k-rows 8q+4g+e of the tile (the Adam / Muon / raw-vote
// epilogue).  The operand loads are issued several steps ahead of the MFMAs that consume them.
__global__ void __launch_bounds__(EGG_THREADS) k_vote_adam(UpdParams p) {
    __shared__ int red[EGG_WAVES][16][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const int tiles_n = p.cols / 32;
    const int tile = blockIdx.x;
    const int k0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
    const int8_t *pb = p.panel_b + (size_t)(k0 + j) * p.pairs_pad + 16 * g;
    const int8_t *pa = p.panel_a + (size_t)(n0 + j) * p.pairs_pad + 16 * g;
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
#pragma unroll 8
    for (int s = wave * 32; s < p.pairs_pad; s += 32 * EGG_WAVES) {
        v4i a = *reinterpret_cast<const v4i *>(pb + s);
        v4i b = *reinterpret_cast<const v4i *>(pa + s);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) red[wave][r][lane] = acc[r];
    __syncthreads();
    const int q = wave;
    int vote[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        int v = 0;
#pragma unroll
        for (int w = 0; w < EGG_WAVES; w++) v += red[w][4 * q + e][lane];
        vote[e] = v;
    }
    // lane (n = n0 + j, half g), element e -> k = k0 + 8q + 4g + e ; blocked index of (k, n) (mgpu.cu:1085-1089)
    const int n = n0 + j;
    const size_t idx0 = ((size_t)((k0 >> 2) + 2 * q + g) * p.cols + n) * 4;
    if (p.muon_x) {
        // muon_momentum_update_kernel + muon_gather_m_kernel (muon_internal.cuh:15-74): m = mu*m + vote
        float4 *sp = reinterpret_cast<float4 *>(p.state + idx0 * 2);
        float4 s0 = sp[0], s1 = sp[1];
        float mv[4] = {s0.x, s0.z, s1.x, s1.z};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float t = p.muon_momentum * mv[e];
            mv[e] = t + (float)vote[e];
            p.muon_x[(size_t)(k0 + 8 * q + 4 * g + e) * p.cols + n] = mv[e];
        }
        sp[0] = make_float4(mv[0], s0.y, mv[1], s0.w);
        sp[1] = make_float4(mv[2], s1.y, mv[3], s1.w);
        return;
    }
    if (p.votes_out) {
        v4i o4;
#pragma unroll
        for (int e = 0; e < 4; e++) o4[e] = vote[e];
        *reinterpret_cast<v4i *>(p.votes_out + idx0) = o4;
        return;
    }
    const float lr = (*p.d_lr) * p.lr_scale;
    const AdamHyper hy = {p.beta1, p.beta2, p.eps, p.wd, p.limit};
    int changes = 0;
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
        const int ch = adam_apply(st[3 * e], st[3 * e + 1], st[3 * e + 2], wv[e], -(float)vote[e], lr, hy);
        changes += ch;
        // every writer stores the same value, so plain stores do (the overlay rule only asks "any change?")
        if (ch && p.flags) { p.flags[k0 + 8 * q + 4 * g + e] = 1; p.flags[p.rows + n] = 1; }
    }
    *reinterpret_cast<int *>(p.W + idx0) = pack4(wv[0], wv[1], wv[2], wv[3]);
    sp[0] = make_float4(st[0], st[1], st[2], st[3]);
    sp[1] = make_float4(st[4], st[5], st[6], st[7]);
    sp[2] = make_float4(st[8], st[9], st[10], st[11]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) changes += __shfl_xor(changes, off, 64);
    if (lane == 0 && changes) atomicAdd(p.counter, (unsigned long long)changes);
}
hipError_t egg_launch_update_matrix(const UpdParams &p, hipStream_t s) {
    if (p.rows % 32 || p.cols % 32 || p.pairs_pad % 32) return hipErrorInvalidValue;
    int64_t total = (int64_t)(p.rows + p.cols) * p.pairs_pad;
    hipLaunchKernelGGL(k_panels, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, p);
    int tiles = (p.rows / 32) * (p.cols / 32);
    hipLaunchKernelGGL(k_vote_adam, dim3(tiles), dim3(EGG_THREADS), 0, s, p);
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
        const AdamHyper hy = {p.beta1, p.beta2, p.eps, p.wd, 127};     // vector tensors keep the reference's +-127
        const float lr = (*p.d_lr) * p.lr_scale;
        float *st = p.state + (size_t)idx * 3;
        float m = st[0], v = st[1], acc = st[2];
        int w = p.W[idx];
        int ch = adam_apply(m, v, acc, w, -(float)vote, lr, hy);
        p.W[idx] = (int8_t)w; st[0] = m; st[1] = v; st[2] = acc;
        if (ch) atomicAdd(p.counter, 1ull);
    }
}
// the same for all vector tensors at once (one wave per element of any of them), so that the small per-tensor
// launches do not leave most of the GPU idle
__global__ void __launch_bounds__(EGG_THREADS) k_vectors_adam(UpdParams p, const VecDesc *desc, int n_desc, int total) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int gi = blockIdx.x * EGG_WAVES + wave;
    if (gi >= total) return;
    int d = 0;
    while (d + 1 < n_desc && desc[d + 1].first <= gi) d++;
    const VecDesc t = desc[d];
    const int idx = gi - t.first;
    const uint32_t base = *p.d_seed + (uint32_t)t.seed_base;
    int vote = 0;
    for (int pr = lane; pr < p.pairs; pr += 64) {
        int f = p.fit[pr];
        if (f == 0) continue;
        uint32_t s = base + (uint32_t)pr;
        vote += f * noise_from_hash(s + t.off_a, idx, p.mask) * noise_from_hash(s + t.off_b, idx, p.mask);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) vote += __shfl_xor(vote, off, 64);
    if (lane == 0) {
        const AdamHyper hy = {p.beta1, p.beta2, p.eps, p.wd, 127};     // vector tensors keep the reference's +-127
        const float lr = (*p.d_lr) * t.lr_scale;
        float *st = t.state + (size_t)idx * 3;
        float m = st[0], v = st[1], acc = st[2];
        int w = t.W[idx];
        int ch = adam_apply(m, v, acc, w, -(float)vote, lr, hy);
        t.W[idx] = (int8_t)w; st[0] = m; st[1] = v; st[2] = acc;
        if (ch) atomicAdd(p.counter, 1ull);
        if (ch && t.flags) t.flags[idx] = 1;
    }
}
// Ternary-packed matrix weights (no counterpart in the reference, whose weights are plain int8): four consecutive
// elements of the blocked matrix -- the four input rows that share one dword -- per byte, element e in bits 2e+1..2e
// as a 2-bit two's complement number (00 = 0, 01 = +1, 11 = -1).  Unpacking writes the canonical int8 blob, from which
// the fragment-major copy the MFMAs read is rebuilt.
__global__ void k_ternary_unpack(const uint8_t *packed, int *words, int n_words) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_words) return;
    const int b = packed[i];
    int w = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int v = ((b >> (2 * e)) & 3) << 30 >> 30;       // sign-extend the 2-bit field
        w |= (v & 0xff) << (8 * e);
    }
    words[i] = w;
}
__global__ void k_ternary_pack(const int *words, uint8_t *packed, int n_words, int *bad) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_words) return;
    const int w = words[i];
    int b = 0, out_of_range = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int v = sx8(w, e);
        out_of_range |= (v < -1) | (v > 1);
        b |= (v & 3) << (2 * e);
    }
    packed[i] = (uint8_t)b;
    if (out_of_range) *bad = 1;      // every writer stores the same value
}
hipError_t egg_launch_ternary_unpack(const uint8_t *packed, int8_t *dst, int n_elems, hipStream_t s) {
    const int n = n_elems / 4;
    hipLaunchKernelGGL(k_ternary_unpack, dim3((n + 255) / 256), dim3(256), 0, s, packed, reinterpret_cast<int *>(dst), n);
    return hipGetLastError();
}
hipError_t egg_launch_ternary_pack(const int8_t *src, uint8_t *packed, int n_elems, int *d_bad, hipStream_t s) {
    const int n = n_elems / 4;
    hipLaunchKernelGGL(k_ternary_pack, dim3((n + 255) / 256), dim3(256), 0, s, reinterpret_cast<const int *>(src), packed, n, d_bad);
    return hipGetLastError();
}

// update_overlay_kernel (de/src/kernels.cu:61-77) over a list of segments of the overlay blob
__global__ void k_overlay_update(int8_t *overlay, int8_t *q, int8_t *flags, const OvSeg *segs, int inc, int dec) {
    const OvSeg sg = segs[blockIdx.y];
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= sg.count) return;
    const int at = sg.offset + i;
    int ov = overlay[at];
    if (flags[at]) { ov += inc; if (ov > 127) ov = 127; }
    else { ov -= dec; if (ov < -127) ov = -127; }
    flags[at] = 0;
    overlay[at] = (int8_t)ov;
    q[at] = (int8_t)overlay_q(ov);
}
hipError_t egg_launch_overlay_update(int8_t *overlay, int8_t *q, int8_t *flags, const OvSeg *d_segs, int n_segs, int max_count,
                                     int inc, int dec, hipStream_t s) {
    if (n_segs <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_overlay_update, dim3((max_count + 255) / 256, n_segs), dim3(256), 0, s, overlay, q, flags, d_segs, inc, dec);
    return hipGetLastError();
}
__global__ void k_overlay_q(const int8_t *overlay, int8_t *q, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) q[i] = (int8_t)overlay_q(overlay[i]);
}
hipError_t egg_launch_overlay_q(const int8_t *overlay, int8_t *q, int64_t n, hipStream_t s) {
    hipLaunchKernelGGL(k_overlay_q, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, overlay, q, n);
    return hipGetLastError();
}

hipError_t egg_launch_update_vectors(const UpdParams &common, const VecDesc *d_desc, int n_desc, int total, hipStream_t s) {
    if (total <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_vectors_adam, dim3((total + EGG_WAVES - 1) / EGG_WAVES), dim3(EGG_THREADS), 0, s, common, d_desc, n_desc, total);
    return hipGetLastError();
}
hipError_t egg_launch_update_vector(const UpdParams &p, hipStream_t s) {
    hipLaunchKernelGGL(k_vector_adam, dim3((p.cols + EGG_WAVES - 1) / EGG_WAVES), dim3(EGG_THREADS), 0, s, p);
    return hipGetLastError();
}

// Three-pass LUT sampling of generate_sequence_kernel (mgpu.cu:1212-1283) for one position: maximum logit,
// sum of EXP_LUT[clamp(max - logit)], threshold hash_rng(seed + t*555, 0) % sum, then the first vocabulary entry
// whose running sum exceeds the threshold.  The reference accumulates in thread order with thread `tid` owning
// v = tid, tid + bt, ... (bt = its block size = hidden rounded up to 32, at most 1024), so for bt < vocab the scan
// order is thread-major, not natural; `bt` reproduces that: every reference thread's sum is formed (in parallel), the
// thread in whose range the threshold falls is found from their prefix sums, and its entries are walked.
// One workgroup; `ws` holds the vocab weights.  TOK: the token type of the buffer (bytes, or uint32 above vocab 256).
__device__ __forceinline__ void sample_select(const int *ex, int vocab, int bt, uint32_t seed, int t, long long *tsum, int *selected) {
    for (int tid = threadIdx.x; tid < bt; tid += 256) {
        long long sum = 0;
        for (int v = tid; v < vocab; v += bt) sum += ex[v];
        tsum[tid] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        long long total = 0;
        for (int tid = 0; tid < bt; tid++) total += tsum[tid];
        const uint32_t r = hash_rng(seed + (uint32_t)t * 555u, 0);
        const long long thresh = total > 0 ? (long long)r % total : 0;
        int sel = 0; long long running = 0; bool done = false;
        for (int tid = 0; tid < bt && !done; tid++) {
            if (running + tsum[tid] <= thresh) { running += tsum[tid]; continue; }
            for (int v = tid; v < vocab; v += bt) {
                running += ex[v];
                if (running > thresh) { sel = v; done = true; break; }
            }
        }
        *selected = sel;
    }
}
template <typename TOK>
__global__ void __launch_bounds__(256) k_sample(const int32_t *logits, const int32_t *exp_lut, int vocab, int bt,
                                                uint32_t seed, int t, int *ws, TOK *out) {
    __shared__ long long tsum[1024];
    __shared__ int red[256];
    __shared__ int sel;
    int mx = INT_MIN;
    for (int v = threadIdx.x; v < vocab; v += 256) mx = max(mx, logits[v]);
    red[threadIdx.x] = mx; __syncthreads();
    for (int o = 128; o > 0; o >>= 1) { if ((int)threadIdx.x < o) red[threadIdx.x] = max(red[threadIdx.x], red[threadIdx.x + o]); __syncthreads(); }
    mx = red[0];
    for (int v = threadIdx.x; v < vocab; v += 256) {
        int idx = mx - logits[v];
        idx = idx < 0 ? 0 : (idx > 255 ? 255 : idx);
        ws[v] = exp_lut[idx];
    }
    __syncthreads();
    sample_select(ws, vocab, bt, seed, t, tsum, &sel);
    if (threadIdx.x == 0) *out = (TOK)sel;
}
hipError_t egg_launch_sample(const int32_t *logits, const int32_t *exp_lut, int vocab, int bt, uint32_t seed, int t,
                             int *ws, void *out, int token_bytes, hipStream_t s) {
    if (bt < 1 || bt > 1024 || !ws) return hipErrorInvalidValue;
    if (token_bytes == 4) hipLaunchKernelGGL(k_sample<uint32_t>, dim3(1), dim3(256), 0, s, logits, exp_lut, vocab, bt, seed, t, ws, (uint32_t *)out);
    else hipLaunchKernelGGL(k_sample<uint8_t>, dim3(1), dim3(256), 0, s, logits, exp_lut, vocab, bt, seed, t, ws, (uint8_t *)out);
    return hipGetLastError();
}

// The d-eggs sampler (d-eggs/src/kernels.cu:382-478): every occurrence of v among the tokens up to position t lowers
// v's logit by penalty_int (repeated int32 subtraction: wraps), the differences to the maximum are divided by the
// temperature in float and truncated, entries below min_p_limit are left out, the rest weigh
// EXP_LUT[clamp(-scaled, 0, 255)]; threshold and scan order as above.  `ws` holds 2 * vocab ints.
// float -> int32 as the GPU's conversion does it: truncation toward zero, saturation at the ends, NaN -> 0
__device__ __forceinline__ int sat_f2i(float x) {
    if (x != x) return 0;
    if (x >= 2147483648.0f) return INT_MAX;
    if (x <= -2147483648.0f) return INT_MIN;
    return (int)x;
}
template <typename TOK>
__global__ void __launch_bounds__(256) k_sample_deggs(const int32_t *logits, const int32_t *exp_lut, int vocab, int bt, uint32_t seed, int t,
                                                      const TOK *tokens, float temp, int min_p_limit, int penalty_int, int *ws, TOK *out) {
    __shared__ long long tsum[1024];
    __shared__ int red[256];
    __shared__ int sel;
    int *lg = ws, *ex = ws + vocab;
    int mx = INT_MIN;
    for (int v = threadIdx.x; v < vocab; v += 256) {
        uint32_t count = 0;
        for (int i = 0; i <= t; i++) count += (int)tokens[i] == v;
        const int l = (int)((uint32_t)logits[v] - count * (uint32_t)penalty_int);
        lg[v] = l;
        mx = max(mx, l);
    }
    red[threadIdx.x] = mx; __syncthreads();
    for (int o = 128; o > 0; o >>= 1) { if ((int)threadIdx.x < o) red[threadIdx.x] = max(red[threadIdx.x], red[threadIdx.x + o]); __syncthreads(); }
    mx = red[0];
    for (int v = threadIdx.x; v < vocab; v += 256) {
        const int shifted = (int)((uint32_t)lg[v] - (uint32_t)mx);
        const int scaled = sat_f2i((float)shifted / temp);
        int e = 0;
        if (scaled >= min_p_limit) {
            int idx = (int)(0u - (uint32_t)scaled);
            idx = idx < 0 ? 0 : (idx > 255 ? 255 : idx);
            e = exp_lut[idx];
        }
        ex[v] = e;
    }
    __syncthreads();
    sample_select(ex, vocab, bt, seed, t, tsum, &sel);
    if (threadIdx.x == 0) *out = (TOK)sel;
}
hipError_t egg_launch_sample_deggs(const int32_t *logits, const int32_t *exp_lut, int vocab, int bt, uint32_t seed, int t,
                                   const void *tokens, float temp, int min_p_limit, int penalty_int, int *ws, void *out, int token_bytes, hipStream_t s) {
    if (bt < 1 || bt > 1024 || t < 0 || !ws) return hipErrorInvalidValue;
    if (token_bytes == 4)
        hipLaunchKernelGGL(k_sample_deggs<uint32_t>, dim3(1), dim3(256), 0, s, logits, exp_lut, vocab, bt, seed, t, (const uint32_t *)tokens, temp,
                           min_p_limit, penalty_int, ws, (uint32_t *)out);
    else
        hipLaunchKernelGGL(k_sample_deggs<uint8_t>, dim3(1), dim3(256), 0, s, logits, exp_lut, vocab, bt, seed, t, (const uint8_t *)tokens, temp,
                           min_p_limit, penalty_int, ws, (uint8_t *)out);
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

hipError_t egg_launch_muon_momentum(const UpdParams &p, hipStream_t s) {
    if (!p.muon_x) return hipErrorInvalidValue;
    return egg_launch_update_matrix(p, s);
}

// ---------------------------------------------------------------- Newton-Schulz (muon_internal.cuh:182-342)
typedef float v16f __attribute__((ext_vector_type(16)));

// Every kernel of the chain takes a batch of same-shape matrices, one per blockIdx.y (matrix b's operands sit b strides
// further on); what is computed for a matrix does not depend on the batch it runs in.
// sum of squares in two deterministic stages (cublasSnrm2 in the reference): 256 partial sums per matrix
__global__ void __launch_bounds__(256) k_sumsq_partial(const float *x, int n, float *partials) {
    __shared__ float sh[256];
    x += (size_t)blockIdx.y * n; partials += (size_t)blockIdx.y * 256;
    float s = 0.f;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) { float v = x[i]; s += v * v; }
    sh[threadIdx.x] = s; __syncthreads();
    for (int o = 128; o > 0; o >>= 1) { if (threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o]; __syncthreads(); }
    if (threadIdx.x == 0) partials[blockIdx.x] = sh[0];
}
__global__ void __launch_bounds__(256) k_norm_finish(const float *partials, int n, float *norm) {
    __shared__ float sh[256];
    partials += (size_t)blockIdx.y * 256;
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) s += partials[i];
    sh[threadIdx.x] = s; __syncthreads();
    for (int o = 128; o > 0; o >>= 1) { if (threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o]; __syncthreads(); }
    if (threadIdx.x == 0) norm[blockIdx.y] = sqrtf(sh[0]);
}
// muon_scale_by_norm_kernel (muon_internal.cuh:77-87)
__global__ void k_scale_by_norm(float *x, const float *norm, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) { float nv = norm[blockIdx.y]; if (nv > 1e-6f) x[(size_t)blockIdx.y * n + i] /= nv; }
}

// C[M][N] (row-major, ldc = N) = epilogue(sum_k A(i,k) B(k,j)), one workgroup per 32x32 tile on
// v_mfma_f32_32x32x2_f32.  Each operand is given by two strides of which one is 1 (a row-major matrix or its
// transpose); AK / BK say that it is the k stride.  An operand whose k stride is 1 is read with one 16-byte load per lane
// (four consecutive k of the lane's row or column); the other kind has its rows or columns side by side in memory and is
// read with fully coalesced 4-byte loads.  The k range is dealt to the four waves in blocks of eight (wave w takes blocks
// w, w + 4, ...); within a block, MFMA e multiplies the k pair {8c + e, 8c + 4 + e}.  The partial tiles are added in wave
// order in LDS, so the summation order is fixed and results are reproducible; wave q writes rows 8q + 4g + e of the
// tile.  mode 0: C = alpha * acc.  mode 1: C = (i == j ? 3 : 0) - acc  (3I - G, muon_internal.cuh:91-109).
typedef float v4f __attribute__((ext_vector_type(4)));
template <bool AK, bool BK>
__global__ void __launch_bounds__(EGG_THREADS) k_sgemm(const float *A, long lda, long batch_a, const float *B, long ldb, long batch_b,
                                                      float *C, int M, int N, int K, float alpha, int mode) {
    __shared__ float red[EGG_WAVES][16][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const int tiles_n = N / 32, tile = blockIdx.x;
    const int i0 = (tile / tiles_n) * 32, j0 = (tile % tiles_n) * 32;
    A += (long)blockIdx.y * batch_a; B += (long)blockIdx.y * batch_b; C += (size_t)blockIdx.y * M * N;
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    // lane (j, g) supplies A(i0 + j, k) and B(k, j0 + j) for k = 8c + 4g + e
    const float *ap = AK ? A + (long)(i0 + j) * lda + 4 * g : A + (long)(4 * g) * lda + i0 + j;
    const float *bp = BK ? B + (long)(j0 + j) * ldb + 4 * g : B + (long)(4 * g) * ldb + j0 + j;
#pragma unroll 4
    for (int c = wave; c < K / 8; c += EGG_WAVES) {
        v4f a4, b4;
        if (AK) a4 = *reinterpret_cast<const v4f *>(ap + 8 * c);
        else {
#pragma unroll
            for (int e = 0; e < 4; e++) a4[e] = ap[(long)(8 * c + e) * lda];
        }
        if (BK) b4 = *reinterpret_cast<const v4f *>(bp + 8 * c);
        else {
#pragma unroll
            for (int e = 0; e < 4; e++) b4[e] = bp[(long)(8 * c + e) * ldb];
        }
#pragma unroll
        for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[e], b4[e], acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) red[wave][r][lane] = acc[r];
    __syncthreads();
    const int q = wave;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float v = red[0][4 * q + e][lane];
#pragma unroll
        for (int w = 1; w < EGG_WAVES; w++) v += red[w][4 * q + e][lane];
        const int i = i0 + 8 * q + 4 * g + e, jj = j0 + j;
        C[(size_t)i * N + jj] = (mode == 1) ? ((i == jj ? 3.0f : 0.0f) - v) : alpha * v;
    }
}
// The same product for M and N that are multiples of 64, with the operands staged once per workgroup through LDS and every
// output element summed by one wave over the whole of K (no partial tiles to add up).  A workgroup owns a TILE x TILE
// block of C, TILE = 64 WT: wave (wm, wn) owns the 32 WT x 32 WT quarter as WT x WT MFMA tiles.  A TILE x 32 chunk of A
// and a 32 x TILE chunk of B go global -> registers -> LDS (the next chunk's loads are in flight while the MFMAs of the
// current one run); with WT = 2 every value read from LDS feeds two MFMAs and the L2 traffic per flop is a quarter of
// the 32 x 32 kernel's.  An operand whose k stride is 1 sits in LDS as [row][k] with rows 36 floats apart (16-byte
// reads of four consecutive k, a 2-way bank conflict at most); the other kind as [k][row] with k rows TILE + 8 floats
// apart (4-byte reads; the two lane halves, four k rows apart, fall on different banks).
// Within a block of eight k, MFMA e multiplies the pair {8c + e, 8c + 4 + e}, blocks in ascending order, whatever WT
// is: the two tile sizes give bit-identical results, so the host may pick by the size of the grid.  Epilogues as above.
template <bool AK, bool BK, int WT>
__global__ void __launch_bounds__(EGG_THREADS, 2) k_sgemm_lds(const float *A, long lda, long batch_a, const float *B, long ldb, long batch_b,
                                                             float *C, int M, int N, int K, float alpha, int mode) {
    constexpr int TILE = 64 * WT, KC = 32, LDK = 36, LDI = TILE + 8, PIECES = TILE * KC / 4 / EGG_THREADS;
    constexpr int ASZ = AK ? TILE * LDK : KC * LDI, BSZ = BK ? TILE * LDK : KC * LDI;
    constexpr int RPI = TILE / 4;                 // 16-byte pieces per k row of an [k][row] chunk
    __shared__ __align__(16) float As[ASZ];
    __shared__ __align__(16) float Bs[BSZ];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31, tid = threadIdx.x;
    const int wm = wave >> 1, wn = wave & 1;
    const int tiles_n = N / TILE, tile = blockIdx.x;
    const int i0 = (tile / tiles_n) * TILE, j0 = (tile % tiles_n) * TILE;
    A += (long)blockIdx.y * batch_a; B += (long)blockIdx.y * batch_b; C += (size_t)blockIdx.y * M * N;
    v16f acc[WT][WT];
#pragma unroll
    for (int a = 0; a < WT; a++)
#pragma unroll
        for (int b = 0; b < WT; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;
    // global -> registers: PIECES 16-byte pieces of each operand's chunk per thread
    v4f ra[PIECES], rb[PIECES];
    auto load_chunk = [&](int k0) {
#pragma unroll
        for (int p = 0; p < PIECES; p++) {
            const int idx = tid + EGG_THREADS * p;
            if (AK) ra[p] = *reinterpret_cast<const v4f *>(A + (long)(i0 + (idx >> 3)) * lda + k0 + 4 * (idx & 7));
            else ra[p] = *reinterpret_cast<const v4f *>(A + (long)(k0 + idx / RPI) * lda + i0 + 4 * (idx % RPI));
            if (BK) rb[p] = *reinterpret_cast<const v4f *>(B + (long)(j0 + (idx >> 3)) * ldb + k0 + 4 * (idx & 7));
            else rb[p] = *reinterpret_cast<const v4f *>(B + (long)(k0 + idx / RPI) * ldb + j0 + 4 * (idx % RPI));
        }
    };
    auto store_chunk = [&]() {
#pragma unroll
        for (int p = 0; p < PIECES; p++) {
            const int idx = tid + EGG_THREADS * p;
            if (AK) *reinterpret_cast<v4f *>(As + (idx >> 3) * LDK + 4 * (idx & 7)) = ra[p];
            else *reinterpret_cast<v4f *>(As + (idx / RPI) * LDI + 4 * (idx % RPI)) = ra[p];
            if (BK) *reinterpret_cast<v4f *>(Bs + (idx >> 3) * LDK + 4 * (idx & 7)) = rb[p];
            else *reinterpret_cast<v4f *>(Bs + (idx / RPI) * LDI + 4 * (idx % RPI)) = rb[p];
        }
    };
    load_chunk(0);
    for (int k0 = 0; k0 < K; k0 += KC) {
        __syncthreads();                    // every wave has finished reading the previous chunk
        store_chunk();
        __syncthreads();
        if (k0 + KC < K) load_chunk(k0 + KC);
#pragma unroll
        for (int c = 0; c < KC / 8; c++) {
            v4f a4[WT], b4[WT];
#pragma unroll
            for (int t = 0; t < WT; t++) {
                const int row = 32 * WT * wm + 32 * t + j, col = 32 * WT * wn + 32 * t + j;
                if (AK) a4[t] = *reinterpret_cast<const v4f *>(As + row * LDK + 8 * c + 4 * g);
                else {
#pragma unroll
                    for (int e = 0; e < 4; e++) a4[t][e] = As[(8 * c + 4 * g + e) * LDI + row];
                }
                if (BK) b4[t] = *reinterpret_cast<const v4f *>(Bs + col * LDK + 8 * c + 4 * g);
                else {
#pragma unroll
                    for (int e = 0; e < 4; e++) b4[t][e] = Bs[(8 * c + 4 * g + e) * LDI + col];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int ta = 0; ta < WT; ta++)
#pragma unroll
                    for (int tb = 0; tb < WT; tb++)
                        acc[ta][tb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[ta][e], b4[tb][e], acc[ta][tb], 0, 0, 0);
        }
    }
    // accumulator register r of lane (j, g) is row 8 (r / 4) + 4 g + r % 4, column j of its 32 x 32 tile
#pragma unroll
    for (int ta = 0; ta < WT; ta++)
#pragma unroll
        for (int tb = 0; tb < WT; tb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = i0 + 32 * WT * wm + 32 * ta + 8 * (r >> 2) + 4 * g + (r & 3), jj = j0 + 32 * WT * wn + 32 * tb + j;
                const float v = acc[ta][tb][r];
                C[(size_t)i * N + jj] = (mode == 1) ? ((i == jj ? 3.0f : 0.0f) - v) : alpha * v;
            }
}
template <int WT>
static hipError_t sgemm_lds(bool ak, bool bk, const float *A, long lda, long batch_a, const float *B, long ldb, long batch_b, float *C,
                            int M, int N, int K, float alpha, int mode, int batch, hipStream_t s) {
    const dim3 grid((M / (64 * WT)) * (N / (64 * WT)), batch), block(EGG_THREADS);
    if (ak && bk) hipLaunchKernelGGL((k_sgemm_lds<true, true, WT>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    else if (ak) hipLaunchKernelGGL((k_sgemm_lds<true, false, WT>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    else if (bk) hipLaunchKernelGGL((k_sgemm_lds<false, true, WT>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    else hipLaunchKernelGGL((k_sgemm_lds<false, false, WT>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    return hipGetLastError();
}
static int egg_update_cu_count() {
    static int n = 0;
    if (!n) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) n = v;
        else n = 256;
    }
    return n;
}
// A(i,k) at A[i * sa_i + k * sa_k], B(k,j) at B[k * sb_k + j * sb_j]; one stride of each pair must be 1 and the other a
// multiple of 4 (16-byte loads)
static hipError_t sgemm(const float *A, long sa_i, long sa_k, long batch_a, const float *B, long sb_k, long sb_j, long batch_b, float *C, int M, int N, int K,
                        float alpha, int mode, int batch, hipStream_t s) {
    const bool ak = sa_k == 1, bk = sb_k == 1;
    if ((!ak && sa_i != 1) || (!bk && sb_j != 1) || M % 32 || N % 32 || K % 32) return hipErrorInvalidValue;
    const long lda = ak ? sa_i : sa_k, ldb = bk ? sb_j : sb_k;
    if (lda % 4 || ldb % 4 || batch_a % 4 || batch_b % 4) return hipErrorInvalidValue;
    // The LDS-staged kernel where the shape allows it: 128 x 128 tiles when they still fill the GPU, 64 x 64 tiles otherwise
    // (bit-identical results, so the choice may depend on the batch)
    if (M % 64 == 0 && N % 64 == 0) {
        const bool big = M % 128 == 0 && N % 128 == 0 && (long)(M / 128) * (N / 128) * batch >= 2 * egg_update_cu_count();
        return big ? sgemm_lds<2>(ak, bk, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode, batch, s)
                   : sgemm_lds<1>(ak, bk, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode, batch, s);
    }
    const dim3 grid((M / 32) * (N / 32), batch), block(EGG_THREADS);
    if (ak && bk) hipLaunchKernelGGL((k_sgemm<true, true>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    else if (ak) hipLaunchKernelGGL((k_sgemm<true, false>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    else if (bk) hipLaunchKernelGGL((k_sgemm<false, true>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    else hipLaunchKernelGGL((k_sgemm<false, false>), grid, block, 0, s, A, lda, batch_a, B, ldb, batch_b, C, M, N, K, alpha, mode);
    return hipGetLastError();
}
__global__ void k_copy_f32(float *dst, const float *src, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// `batch` matrices of rows x cols, matrix b at w.x + b * rows * cols (w.swap likewise), its 3I - G term at
// w.bterm + b * K * K (K = min(rows, cols)), its 256 norm partials at w.partials + 256 b, its norm at w.norm + b
hipError_t egg_launch_newton_schulz_batched(const MuonWork &w, int rows, int cols, int iters, int batch, hipStream_t s) {
    if (rows % 32 || cols % 32 || batch < 1 || batch > 65535) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(w.x) | reinterpret_cast<uintptr_t>(w.swap) | reinterpret_cast<uintptr_t>(w.bterm)) & 15) return hipErrorInvalidValue;   // 16-byte loads
    const int n = rows * cols;
    const bool use_rows = rows < cols;
    const int K = use_rows ? rows : cols;
    const long kk = (long)K * K;
    hipLaunchKernelGGL(k_sumsq_partial, dim3(256, batch), dim3(256), 0, s, w.x, n, w.partials);
    hipLaunchKernelGGL(k_norm_finish, dim3(1, batch), dim3(256), 0, s, w.partials, 256, w.norm);
    hipLaunchKernelGGL(k_scale_by_norm, dim3((n + 255) / 256, batch), dim3(256), 0, s, w.x, w.norm, n);
    float *cur = w.x, *nxt = w.swap;          // ping-pong instead of copying back after every iteration
    hipError_t e = hipSuccess;
    for (int it = 0; it < iters && e == hipSuccess; it++) {
        if (use_rows) {
            // G = X X^T (rows x rows); X <- 0.5 (3I - G) X
            e = sgemm(cur, cols, 1, n, cur, 1, cols, n, w.bterm, K, K, cols, 1.f, 1, batch, s);
            if (e == hipSuccess) e = sgemm(w.bterm, K, 1, kk, cur, cols, 1, n, nxt, rows, cols, K, 0.5f, 0, batch, s);
        } else {
            // G = X^T X (cols x cols); X <- 0.5 X (3I - G)
            e = sgemm(cur, 1, cols, n, cur, cols, 1, n, w.bterm, K, K, rows, 1.f, 1, batch, s);
            if (e == hipSuccess) e = sgemm(cur, cols, 1, n, w.bterm, K, 1, kk, nxt, rows, cols, K, 0.5f, 0, batch, s);
        }
        float *t = cur; cur = nxt; nxt = t;
    }
    if (e != hipSuccess) return e;
    const size_t total = (size_t)n * batch;
    if (cur != w.x) hipLaunchKernelGGL(k_copy_f32, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, w.x, cur, total);
    return hipGetLastError();
}
hipError_t egg_launch_newton_schulz(const MuonWork &w, int rows, int cols, int iters, hipStream_t s) {
    return egg_launch_newton_schulz_batched(w, rows, cols, iters, 1, s);
}

// ---------------------------------------------------------------- Newton-Schulz for callers that cannot allocate
// The same kernels with their workspace (ping-pong matrix, 3I - G term, norm partials) in a file-scope device array
// instead of a context's hipMalloc'd buffers.  Each GPU holds its own copy of the array; its address on a device is
// looked up once per device with hipGetSymbolAddress and used from then on in place of the array's name.
struct NsScratch {
    float swap[EGG_NS_STATIC_MAX_ELEMS];
    float bterm[EGG_NS_STATIC_MAX_SHORT * EGG_NS_STATIC_MAX_SHORT];
    float partials[1024];
    float norm[4];
};
static __device__ __align__(256) unsigned char scratch[sizeof(NsScratch)];
static NsScratch *g_ns_scratch[EGG_MAX_DEVICES];      // per device; written once, under g_ns_mutex
static std::mutex g_ns_mutex;

static hipError_t ns_scratch_on_current_device(NsScratch **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= EGG_MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_ns_mutex);
    if (!g_ns_scratch[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!ptr) return hipErrorInvalidSymbol;
        g_ns_scratch[dev] = static_cast<NsScratch *>(ptr);
    }
    *out = g_ns_scratch[dev];
    return hipSuccess;
}

extern "C" int egg_newton_schulz_static(float *d_X, int rows, int cols, int iters, void *hip_stream) {
    if (!d_X || (reinterpret_cast<uintptr_t>(d_X) & 15) || rows < 32 || cols < 32 || rows % 32 || cols % 32 || iters < 0 || iters > 64) {
        egg_set_thread_error("egg_newton_schulz_static: need a 16-byte aligned device matrix with rows and cols multiples of 32 and 0 <= iters <= 64");
        return EGG_E_INVALID;
    }
    if ((long long)rows * cols > EGG_NS_STATIC_MAX_ELEMS || (rows < cols ? rows : cols) > EGG_NS_STATIC_MAX_SHORT) {
        egg_set_thread_error("egg_newton_schulz_static: matrix exceeds the static workspace (rows * cols <= 1,048,576 and min(rows, cols) <= 512)");
        return EGG_E_INVALID;
    }
    NsScratch *sc = nullptr;
    hipError_t e = ns_scratch_on_current_device(&sc);
    if (e == hipSuccess) {
        // nothing in the workspace has to start at zero: every partial, the norm, the 3I - G term and the ping-pong
        // matrix are written in full before they are read
        MuonWork w = {d_X, sc->swap, nullptr, sc->bterm, sc->partials, sc->norm};
        e = egg_launch_newton_schulz(w, rows, cols, iters, static_cast<hipStream_t>(hip_stream));
    }
    if (e != hipSuccess) {
        egg_set_thread_error((std::string("egg_newton_schulz_static: ") + hipGetErrorString(e)).c_str());
        return EGG_E_HIP;
    }
    return EGG_OK;
}

// muon_apply_update_kernel (muon_internal.cuh:112-170)
__global__ void __launch_bounds__(256) k_muon_apply(UpdParams p, float wd) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    int change = 0;
    if (idx < p.rows * p.cols) {
        int byte_off = idx & 3, word = idx >> 2, n = word % p.cols, k = (word / p.cols) * 4 + byte_off;
        int w = p.W[idx];
        float *st = p.state + (size_t)idx * 2;
        float acc = st[1];
        float u = p.muon_x[(size_t)k * p.cols + n];
        float lr = (*p.d_lr) * p.lr_scale;
        float wdw = wd * (float)w;
        float step = (-lr) * (u + wdw);
        acc += step;
        if (acc >= 1.0f) { if (w < p.limit) { w++; change = 1; acc -= 1.0f; } else acc = 1.0f; }
        else if (acc <= -1.0f) { if (w > -p.limit) { w--; change = 1; acc += 1.0f; } else acc = -1.0f; }
        p.W[idx] = (int8_t)w; st[1] = acc;
    }
    unsigned long long m = __ballot(change);
    if ((threadIdx.x & 63) == 0 && m) atomicAdd(p.counter, (unsigned long long)__popcll(m));
}
hipError_t egg_launch_muon_apply(const UpdParams &p, float wd, hipStream_t s) {
    int n = p.rows * p.cols;
    hipLaunchKernelGGL(k_muon_apply, dim3((n + 255) / 256), dim3(256), 0, s, p, wd);
    return hipGetLastError();
}
