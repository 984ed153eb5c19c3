// egg_device.h -- device-side building blocks shared by the gfx950 kernels.
//
// Conventions used by every kernel in this directory
// ---------------------------------------------------
// * wave64; a "tile" is 32 consecutive tokens of ONE population member (seq_len % 32 == 0).
// * GEMMs are computed transposed, Y^T = W^T . X^T, with v_mfma_i32_32x32x32_i8:
//     A operand = 32 output columns of W (lane i = l%32 -> column, lane half g = l/32),
//     B operand = 32 tokens (lane j = l%32 -> token, g = l/32),
//     C/D       = lane (token j, half g), register r -> output column 8*(r/4) + 4*g + (r%4).
//   So a lane always owns one token; per-token reductions (sum|x|, max|x|, x.B) are in-lane plus one
//   exchange between the two lane halves, and the 16 int8 results a lane holds per 32-column group
//   are exactly the B-operand bytes the next GEMM needs: chained GEMMs never transpose.
// * "slot order": within each group of 32 hidden indices, index n = 8q + 4g + e (q<4, g<2, e<4)
//   lives at byte 16g + 4q + e.  Internal int8 activations in HBM are stored in slot order, so a lane
//   loads / stores its 16 bytes per group with one 128-bit access.
// * The MFMA sums over all 32 k-bytes it is given, whatever k they stand for; only A and B must agree.
//   W blocks are staged into LDS so that lane (column, g) reads, as one 128-bit word, the 16 k-bytes
//   matching the token operand's order (slot order, or natural order for row-major inputs).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

#define EGG_WAVES 4
#define EGG_THREADS (EGG_WAVES * 64)

// ---------------------------------------------------------------- RNG (mgpu.cu:525-538)
__device__ __forceinline__ uint32_t hash_rng(uint32_t s, uint32_t idx) {
    uint32_t x = s + idx * 0x9e3779b9u;
    x ^= x >> 16; x *= 0x85ebca6bu; x ^= x >> 13; x *= 0xc2b2ae35u; x ^= x >> 16;
    return x;
}
__device__ __forceinline__ int noise_from_hash(uint32_t s, uint32_t idx, int mask) {
    uint32_t r = hash_rng(s, idx);
    int mag = (int)((r >> 1) & (uint32_t)mask);
    return (r & 1) ? mag : -mag;
}
__device__ __forceinline__ int clip127(int a) { return min(127, max(-127, a)); }

// ---------------------------------------------------------------- lane helpers
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
// value held by the same token's lane in the other half
__device__ __forceinline__ int other_half(int v) { return __shfl_xor(v, 32, 64); }
__device__ __forceinline__ long long other_half64(long long v) {
    int lo = __shfl_xor((int)(v & 0xffffffffll), 32, 64);
    int hi = __shfl_xor((int)(v >> 32), 32, 64);
    return ((long long)hi << 32) | (unsigned int)lo;
}
// hidden index of accumulator register r of column group nt for lane half g
__device__ __forceinline__ int col_of(int nt, int r, int g) { return nt * 32 + ((r >> 2) << 3) + (g << 2) + (r & 3); }

__device__ __forceinline__ int sx8(int packed, int e) { return (int)(int8_t)(packed >> (8 * e)); }
__device__ __forceinline__ int pack4(int a, int b, int c, int d) {
    return (a & 255) | ((b & 255) << 8) | ((c & 255) << 16) | ((d & 255) << 24);
}
// dot of 4 signed bytes
__device__ __forceinline__ int dot4(int a, int b, int c) {
#if __has_builtin(__builtin_amdgcn_sdot4)
    return __builtin_amdgcn_sdot4(a, b, c, false);
#else
    return c + sx8(a, 0) * sx8(b, 0) + sx8(a, 1) * sx8(b, 1) + sx8(a, 2) * sx8(b, 2) + sx8(a, 3) * sx8(b, 3);
#endif
}
// sum of |bytes| of 4 signed bytes (none equal to -128)
__device__ __forceinline__ int sumabs4(int a, int c) {
    return c + abs(sx8(a, 0)) + abs(sx8(a, 1)) + abs(sx8(a, 2)) + abs(sx8(a, 3));
}

// truncating division of a by a divisor in [1,127] for |a| < 2^24, via a per-token magic number
struct MagicDiv { uint32_t m; int one; };
__device__ __forceinline__ MagicDiv make_magic(int d) {
    MagicDiv r; r.one = (d == 1);
    r.m = r.one ? 0u : (uint32_t)(0x100000000ull / (uint32_t)d) + 1u;
    return r;
}
__device__ __forceinline__ int div_trunc(int a, MagicDiv md) {
    int sg = a >> 31; uint32_t ua = (uint32_t)((a ^ sg) - sg);
    uint32_t uq = md.one ? ua : __umulhi(ua, md.m);
    return ((int)uq ^ sg) - sg;
}

// ---------------------------------------------------------------- W block staging
// Copies the block rows [k0, k0+KB) x cols [n0, n0+NB) of a blocked [K/4][N][4] matrix into LDS as
// [KB/16][NB][16 bytes]: entry (p = 2*ks + g, n) holds the 16 k-bytes lane half g consumes in k-step ks,
// i.e. dwords kq = 8ks + 2q + g (slot order) or 8ks + 4g + q (natural order), q = 0..3.
template <int KB, int NB, bool NAT>
__device__ __forceinline__ void stage_w_block(int8_t *lds, const int8_t *Wg, int n_total, int k0, int n0) {
    const uint32_t *W32 = reinterpret_cast<const uint32_t *>(Wg);
    constexpr int ITEMS = (KB / 16) * NB;
    for (int it = threadIdx.x; it < ITEMS; it += EGG_THREADS) {
        int n = it % NB, p = it / NB, ks = p >> 1, g = p & 1;
        v4i v;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int kq = (k0 >> 2) + 8 * ks + (NAT ? (4 * g + q) : (2 * q + g));
            v[q] = (int)W32[(size_t)kq * n_total + n0 + n];
        }
        *reinterpret_cast<v4i *>(lds + ((size_t)p * NB + n) * 16) = v;
    }
}

// acc[nt] += W_block^T . xop for one staged block; xop[ks] is the token operand of k-step ks of the block
template <int KB, int NB>
__device__ __forceinline__ void mfma_block(v16i *acc, const v4i *xop, const int8_t *lds, int lane) {
    const int i = lane & 31, g = lane >> 5;
#pragma unroll
    for (int ks = 0; ks < KB / 32; ks++) {
#pragma unroll
        for (int nt = 0; nt < NB / 32; nt++) {
            v4i a = *reinterpret_cast<const v4i *>(lds + ((size_t)(ks * 2 + g) * NB + nt * 32 + i) * 16);
            acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, xop[ks], acc[nt], 0, 0, 0);
        }
    }
}

// Full GEMM for one tile: acc[NOUT/32] (+)= W[k_off.., n_off..]^T . xop[KTOT/32], W streamed through LDS
// in blocks of at most 256 x 256.  Every wave of the workgroup must call it (it synchronises).
template <int KTOT, int NOUT, bool NAT>
__device__ __forceinline__ void gemm_stream(v16i *acc, const v4i *xop, const int8_t *Wg, int n_total,
                                            int k_off, int n_off, int8_t *wlds, int lane) {
    constexpr int KB = KTOT < 256 ? KTOT : 256;
    constexpr int NB = NOUT < 256 ? NOUT : 256;
#pragma unroll
    for (int nb = 0; nb < NOUT / NB; nb++) {
#pragma unroll
        for (int kb = 0; kb < KTOT / KB; kb++) {
            __syncthreads();
            stage_w_block<KB, NB, NAT>(wlds, Wg, n_total, k_off + kb * KB, n_off + nb * NB);
            __syncthreads();
            mfma_block<KB, NB>(acc + nb * (NB / 32), xop + kb * (KB / 32), wlds, lane);
        }
    }
}

template <int N>
__device__ __forceinline__ void zero_acc(v16i *acc) {
#pragma unroll
    for (int i = 0; i < N; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
}

// ---------------------------------------------------------------- per-member noise tables (one wave fills its own)
__device__ __forceinline__ void fill_noise_i8(int8_t *dst, uint32_t seed, int n, int mask, int lane) {
    for (int i = lane; i < n; i += 64) dst[i] = (int8_t)noise_from_hash(seed, i, mask);
}
// dst[i] = noise(seed, i) * mult
__device__ __forceinline__ void fill_noise_i32(int *dst, uint32_t seed, int n, int mask, int mult, int lane) {
    for (int i = lane; i < n; i += 64) dst[i] = noise_from_hash(seed, i, mask) * mult;
}
// dst[i] = base[i] + ((noise(seed_a,i) * noise(seed_b,i) * ns) >> shift)       (mgpu.cu:666-675, :733-735)
__device__ __forceinline__ void fill_vec_i32(int *dst, const int8_t *base, uint32_t seed_a, uint32_t seed_b,
                                             int n, int mask, int ns, int shift, int lane) {
    for (int i = lane; i < n; i += 64) {
        int v = base[i];
        if (ns != 0) v += (noise_from_hash(seed_a, i, mask) * noise_from_hash(seed_b, i, mask) * ns) >> shift;
        dst[i] = v;
    }
}
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// x . B over the operand's k-steps; btab is the int8 noise table in natural order.
// slot order: dword q of k-step ks covers k = 32ks + 8q + 4g + (0..3); natural: 32ks + 16g + 4q + (0..3)
template <int KS, bool NAT>
__device__ __forceinline__ int dot_noise(const v4i *xop, const int8_t *btab, int k_off, int g) {
    const int *b32 = reinterpret_cast<const int *>(btab + k_off);
    int s = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int kd = NAT ? (8 * ks + 4 * g + q) : (8 * ks + 2 * q + g);
            s = dot4(xop[ks][q], b32[kd], s);
        }
    return s + other_half(s);
}

// ---------------------------------------------------------------- norms on a token held as a packed operand
// apply_standard_norm (mgpu.cu:646-678): wt / bt are int32 tables already holding w + noise, b + noise
template <int KS>
__device__ __forceinline__ void standard_norm(const v4i *x, v4i *out, const int *wt, const int *bt, int H, int g) {
    int tot = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int q = 0; q < 4; q++) tot = sumabs4(x[ks][q], tot);
    tot += other_half(tot);
    int mn = tot / H; if (!mn) mn = 1;
    MagicDiv md = make_magic(mn);
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int n0 = 32 * ks + 8 * q + 4 * g;
            v4i w4 = *reinterpret_cast<const v4i *>(wt + n0);
            v4i b4 = *reinterpret_cast<const v4i *>(bt + n0);
            int o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = clip127(div_trunc(sx8(x[ks][q], e) * w4[e], md) + b4[e]);
            out[ks][q] = pack4(o[0], o[1], o[2], o[3]);
        }
}

// adaptive_*_normalize (egg_adaptive_normalize.h:10-103) over NT column groups held in acc; result packed
template <int NT>
__device__ __forceinline__ void adaptive_norm(const v16i *val, v4i *out) {
    int mx = 0;
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int r = 0; r < 16; r++) mx = max(mx, abs(val[nt][r]));
    mx = max(mx, other_half(mx));
    float scale = 127.0f / ((float)mx + 1e-9f);
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float sf = (float)val[nt][4 * q + e] * scale;
                int s = (int)roundf(sf);
                o[e] = min(127, max(-127, s));
            }
            out[nt][q] = pack4(o[0], o[1], o[2], o[3]);
        }
}

// 128-bit load/store of a token's 16 bytes of column group `grp` in a slot-ordered [.][H] int8 buffer
__device__ __forceinline__ v4i load_op(const int8_t *row, int grp, int g) {
    return *reinterpret_cast<const v4i *>(row + grp * 32 + g * 16);
}
__device__ __forceinline__ void store_op(int8_t *row, int grp, int g, v4i v) {
    *reinterpret_cast<v4i *>(row + grp * 32 + g * 16) = v;
}
