// egg_gru.hip -- the reference's CPU program (full_trained_egg.c, "egg.c": GRU-style recurrent byte LM with
// sequential-xorshift rank-1 noise and the +-1 threshold update) on gfx950.
//
// The model is recurrent, so tokens are serial; the GEMM's free dimension is the population.  A workgroup of 16
// waves owns 32 members (16 antithetic pairs): every perturbed matmul (egg.c:108-177) is one
// v_mfma_i32_32x32x32_i8 strip per wave (A operand = 32 output rows of W read straight from the fragment-major
// copy in L2, B operand = the 32 members' input vectors in LDS), output rows are split over the waves and the
// int8 results go back to LDS as the next matmul's input.  Noise vectors of all (pair, matrix) are generated once
// per step by replaying the reference's xorshift stream (4 discarded draws per block of 16, egg.c:87-105).
#include <type_traits>
#include "egg_device.h"
#include "egg_launch.h"
#include "../../include/egg_hip.h"

#include <math.h>
#include <stdio.h>
#include <string.h>
#include <string>
#include <algorithm>
#include <tuple>
#include <vector>

#define GRU_WAVES 16
#define GRU_THREADS (GRU_WAVES * 64)

struct GruMat {            // one weight matrix, W[rows = out][cols = in] row-major (egg.c:42-50)
    long long w_off;       // byte offset in the model blob (and in the fragment copy)
    int rows, cols;
    long long a_off, b_off;   // offsets of the per-pair noise vectors (slot order), [pair][rows] / [pair][cols]
    long long pa_off, pb_off; // offsets of the update panels [rows][pairs_pad] / [cols][pairs_pad]
    int seed_off;          // 100*l + k, or 999 for the head (egg.c:242-290)
    int shift;
};

struct GruParams {
    const GruMat *mats;
    const int8_t *model;      // canonical blob (embedding, biases, ln weights)
    const int8_t *frag;       // fragment-major copies of the matrices
    const int8_t *noise;      // per-pair noise vectors
    const uint8_t *data; long long data_len; long long start_idx;
    int8_t *states;           // [population][L][H]
    int32_t *loss;            // [population]
    int H, L, T, V, population, sigma;   // sigma = fixed_point + sigma_shift
    long long off_emb, off_gru_b, off_ln_w, off_ln_out;
    const int32_t *exp2;      // [256]
};

__device__ __forceinline__ uint32_t xorshift32(uint32_t &x) { x ^= x << 13; x ^= x >> 17; x ^= x << 5; return x; }
__device__ __forceinline__ int slot_pos(int n) { int w = n & 31; return (n & ~31) + 16 * ((w >> 2) & 1) + 4 * (w >> 3) + (w & 3); }

// gen_noise_vector_neon (egg.c:87-105) for every (matrix, pair): A[rows] then B[cols] from one stream seeded
// step_seed + pair + seed_off.  Writes the vectors in slot order for the forward, [pair][count], a second copy by tiles
// of 16 pairs, [pair tile][32-group][half][pair][16 bytes], and the raw panels for the vote.
__global__ void k_gru_noise(const GruMat *mats, int n_mats, int pairs, int pairs_pad, uint32_t step_seed,
                            int8_t *noise, int8_t *nfrag, int8_t *panels) {
    int id = blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= n_mats * pairs) return;
    const GruMat m = mats[id / pairs]; const int p = id % pairs;
    uint32_t rng = step_seed + (uint32_t)p + (uint32_t)m.seed_off;
    for (int part = 0; part < 2; part++) {
        const int count = part ? m.cols : m.rows;
        int8_t *vec = noise + (part ? m.b_off + (long long)p * m.cols : m.a_off + (long long)p * m.rows);
        int8_t *tvec = nfrag + (part ? m.b_off : m.a_off) + (long long)(p >> 4) * 16 * count + (p & 15) * 16;
        int8_t *pan = panels + (part ? m.pb_off : m.pa_off);
        for (int i = 0; i < count; i += 16) {
            xorshift32(rng); xorshift32(rng); xorshift32(rng); xorshift32(rng);
            for (int jj = 0; jj < 16 && i + jj < count; jj++) {
                uint32_t r = xorshift32(rng);
                int v = (int)((r >> 1) & 31u); if (!(r & 1)) v = -v;
                const int sp = slot_pos(i + jj);
                vec[sp] = (int8_t)v;
                tvec[(sp >> 4) * 256 + (sp & 15)] = (int8_t)v;
                pan[(long long)(i + jj) * pairs_pad + p] = (int8_t)v;
            }
        }
    }
}

// W[rows][cols] row-major -> [rows/32][cols/16][32][16 B]: entry (nt, 2ks+g, i) holds W[32nt+i][32ks + 8q+4g+e]
__global__ void k_gru_swizzle(const int8_t *W, int8_t *F, int rows, int cols) {
    int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= rows * cols / 16) return;
    int i = c & 31, p = (c >> 5) % (cols / 16), nt = (c >> 5) / (cols / 16), ks = p >> 1, g = p & 1;
    const int *src = reinterpret_cast<const int *>(W + (size_t)(32 * nt + i) * cols + 32 * ks);
    v4i v;
#pragma unroll
    for (int q = 0; q < 4; q++) v[q] = src[2 * q + g];
    reinterpret_cast<v4i *>(F)[c] = v;
}

// one 32-row strip: acc += W[32nt.., :] . in, in = LDS [32 members][K (+16 pad)] in slot order.  The W fragments come
// straight from global memory (L2); eight k-steps' worth are in flight ahead of the MFMAs that use them, so
// the strip pays for one memory latency instead of one per k-step.
template <int KS>
struct GruStrip {
    static constexpr int K = KS * 32, stride = K + 16, BATCH = KS < 8 ? KS : 8;
    static_assert(KS % BATCH == 0, "k-steps come in whole batches");
    v4i a[BATCH];
    const int8_t *fa;
    // request the first batch of fragments (call it as early as the strip is known, before unrelated work)
    __device__ __forceinline__ void begin(const int8_t *ftile, int lane) {
        fa = ftile + ((size_t)(lane >> 5) * 32 + (lane & 31)) * 16;          // k-step ks adds ks * 1024
#pragma unroll
        for (int u = 0; u < BATCH; u++) a[u] = *reinterpret_cast<const v4i *>(fa + (size_t)u * 1024);
    }
    __device__ __forceinline__ void run(v16i &acc, const int8_t *ldsB, int lane) {
        const int8_t *fb = ldsB + (size_t)(lane & 31) * stride + 16 * (lane >> 5);   // k-step ks adds ks * 32
#pragma unroll 1
        for (int k0 = 0; k0 < KS; k0 += BATCH) {
#pragma unroll
            for (int u = 0; u < BATCH; u++) {
                const v4i b = *reinterpret_cast<const v4i *>(fb + (k0 + u) * 32);
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u], b, acc, 0, 0, 0);
                // the register set is refilled for the next batch as soon as its MFMA has been issued
                if (k0 + BATCH < KS) a[u] = *reinterpret_cast<const v4i *>(fa + (size_t)(k0 + BATCH + u) * 1024);
            }
        }
    }
};
template <int KS>
__device__ __forceinline__ void gru_strip(v16i &acc, const int8_t *ftile, const int8_t *ldsB, int lane) {
    GruStrip<KS> st;
    st.begin(ftile, lane);
    st.run(acc, ldsB, lane);
}
// xB = sum_c in[c] * B[c] for the lane's member (egg.c:122-140); the noise rows are requested a batch ahead as well
template <int KS>
__device__ __forceinline__ int gru_xb(const int8_t *ldsB, const int8_t *bvec, int lane) {
    constexpr int K = KS * 32, stride = K + 16, BATCH = KS < 8 ? KS : 8;
    static_assert(KS % BATCH == 0, "k-steps come in whole batches");
    const int j = lane & 31, g = lane >> 5;
    int s = 0;
#pragma unroll 1
    for (int k0 = 0; k0 < KS; k0 += BATCH) {
        v4i n[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; u++) n[u] = *reinterpret_cast<const v4i *>(bvec + 32 * (k0 + u) + 16 * g);
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const v4i b = *reinterpret_cast<const v4i *>(ldsB + (size_t)j * stride + 32 * (k0 + u) + 16 * g);
#pragma unroll
            for (int q = 0; q < 4; q++) s = dot4(b[q], n[u][q], s);
        }
    }
    return sum_halves(s);
}
// rank-1 term, shift and clamp of one strip (egg.c:167-175); returns the 16 int8 results packed in slot order
__device__ __forceinline__ v4i gru_finish(const v16i &acc, int xb, const v4i &a4, int ns, int sigma, int shift) {
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        int o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int noise = (xb * sx8(a4[q], e)) * ns;
            o[e] = clip127((acc[4 * q + e] + (noise >> sigma)) >> shift);
        }
        out[q] = pack4(o[0], o[1], o[2], o[3]);
    }
    return out;
}
__device__ __forceinline__ v4i gru_finish(const v16i &acc, int xb, const int8_t *avec, int nt, int ns, int sigma, int shift, int g) {
    return gru_finish(acc, xb, *reinterpret_cast<const v4i *>(avec + 32 * nt + 16 * g), ns, sigma, shift);
}
__device__ __forceinline__ int cadd(int a, int b) { return clip127(a + b); }   // clipped_add, egg.c:62-67

template <int H>
__global__ void __launch_bounds__(GRU_THREADS) k_gru_forward(GruParams p) {
    constexpr int NTH = H / 32;                 // strips of an H-wide output
    constexpr int NT4 = 4 * H / 32;
    constexpr int MAXT4 = (NT4 + GRU_WAVES - 1) / GRU_WAVES;
    constexpr int SH = H + 16, S4 = 4 * H + 16; // padded LDS row strides
    constexpr std::integral_constant<int, H / 32> KH{};          // k-steps of an H-deep and of a 4H-deep matmul
    constexpr std::integral_constant<int, 4 * H / 32> K4H{};
    extern __shared__ __align__(16) int8_t smem[];
    int8_t *XN = smem, *HB = XN + 32 * SH, *MB = HB + 32 * SH;
    int *psum = reinterpret_cast<int *>(MB + 32 * S4);          // [GRU_WAVES][32]
    int *tl = psum + GRU_WAVES * 32;                            // [32]
    int *lut = tl + 32;                                         // [256]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const bool own = wave < NTH;
    const int member = blockIdx.x * 32 + j, pair = member >> 1, ns = (member & 1) ? -1 : 1;
    const int L = p.L, V = p.V;
    for (int i = threadIdx.x; i < 256; i += GRU_THREADS) lut[i] = p.exp2[i];

    // stream position of the pair (egg.c:553-554)
    const long long stride = p.data_len / (p.population / 2);
    const long long spos = (p.start_idx + (long long)pair * stride) % (p.data_len - p.T);

    // the recurrent state (egg.c:515-517, persists across steps) stays in global memory; a lane re-reads and
    // rewrites only the 16 bytes of its own strip, once per layer and token
    int loss = 0;
    __syncthreads();

    auto put = [&](int8_t *buf, int strideb, int nt, v4i v) { *reinterpret_cast<v4i *>(buf + (size_t)j * strideb + 32 * nt + 16 * g) = v; };
    // egg_ln (egg.c:180-210) of the H-wide vector whose own strip is x; result packed
    auto layer_norm = [&](v4i x, const int8_t *w) -> v4i {
        int part = 0;
        if (own) {
#pragma unroll
            for (int q = 0; q < 4; q++) part = sumabs4(x[q], part);
            part = sum_halves(part);
            if (g == 0) psum[wave * 32 + j] = part;
        }
        __syncthreads();
        int sum = 0;
        for (int w2 = 0; w2 < NTH; w2++) sum += psum[w2 * 32 + j];
        if (sum == 0) sum = 1;
        int mean = sum / H; if (mean == 0) mean = 1;
        const float rcp = 1.0f / (float)mean;
        v4i out = {0, 0, 0, 0};
        if (own) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int w4 = *reinterpret_cast<const int *>(w + 32 * wave + 8 * q + 4 * g);
                int o[4];
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = clip127(div_trunc(sx8(x[q], e) * sx8(w4, e), rcp));
                out[q] = pack4(o[0], o[1], o[2], o[3]);
            }
        }
        return out;
    };
    // perturbed matmul of an H-wide output: the own strip's packed result
    auto matmul_h = [&](int mi, const int8_t *in, auto ks_tag) -> v4i {
        constexpr int KS = decltype(ks_tag)::value, K = KS * 32;
        v4i r = {0, 0, 0, 0};
        if (own) {
            const GruMat m = p.mats[mi];
            GruStrip<KS> st;
            st.begin(p.frag + m.w_off + (size_t)wave * 32 * K, lane);       // on its way while x.B is summed
            const int xb = gru_xb<KS>(in, p.noise + m.b_off + (long long)pair * K, lane);
            v16i acc;
#pragma unroll
            for (int t = 0; t < 16; t++) acc[t] = 0;
            st.run(acc, in, lane);
            r = gru_finish(acc, xb, p.noise + m.a_off + (long long)pair * m.rows, wave, ns, p.sigma, m.shift, g);
        }
        return r;
    };

    for (int t = 0; t < p.T; t++) {
        const int tok = p.data[spos + t];
        v4i x = {0, 0, 0, 0}, resid = {0, 0, 0, 0};
        if (own) {
            const int *e = reinterpret_cast<const int *>(p.model + p.off_emb + (size_t)tok * H + 32 * wave);
#pragma unroll
            for (int q = 0; q < 4; q++) x[q] = e[2 * q + g];
        }
        for (int l = 0; l < L; l++) {
            const int8_t *lnw = p.model + p.off_ln_w + (size_t)l * 2 * H;
            const int8_t *gb = p.model + p.off_gru_b + (size_t)l * 2 * H;
            resid = x;
            int *hptr = reinterpret_cast<int *>(p.states + ((size_t)member * L + l) * H + 32 * wave);
            v4i hcur = {0, 0, 0, 0};
            if (own)
#pragma unroll
                for (int q = 0; q < 4; q++) hcur[q] = hptr[2 * q + g];
            v4i xn = layer_norm(x, lnw);
            if (own) { put(XN, SH, wave, xn); put(HB, SH, wave, hcur); }
            __syncthreads();
            v4i b1 = matmul_h(6 * l + 0, XN, KH);
            v4i b2 = matmul_h(6 * l + 1, HB, KH);
            v4i ft = {0, 0, 0, 0}, gated = {0, 0, 0, 0};
            if (own) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int bf4 = *reinterpret_cast<const int *>(gb + 32 * wave + 8 * q + 4 * g);
                    int f[4], gp[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        f[e] = cadd(cadd(sx8(b1[q], e), sx8(b2[q], e)), sx8(bf4, e));
                        gp[e] = ((f[e] + 127) * sx8(hcur[q], e)) >> 8;
                    }
                    ft[q] = pack4(f[0], f[1], f[2], f[3]); gated[q] = pack4(gp[0], gp[1], gp[2], gp[3]);
                }
            }
            __syncthreads();                       // every wave has finished reading HB (old state)
            if (own) put(HB, SH, wave, gated);
            __syncthreads();
            b1 = matmul_h(6 * l + 2, XN, KH);
            b2 = matmul_h(6 * l + 3, HB, KH);
            if (own) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int bh4 = *reinterpret_cast<const int *>(gb + H + 32 * wave + 8 * q + 4 * g);
                    int hn[4], xo[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        int ht = cadd(cadd(sx8(b1[q], e), sx8(b2[q], e)), sx8(bh4, e));
                        int hv = sx8(hcur[q], e);
                        int upd = ((sx8(ft[q], e) + 127) * (ht - hv)) >> 8;
                        hn[e] = cadd(hv, upd);
                        xo[e] = cadd(hn[e], sx8(resid[q], e));
                    }
                    hptr[2 * q + g] = pack4(hn[0], hn[1], hn[2], hn[3]); x[q] = pack4(xo[0], xo[1], xo[2], xo[3]);
                }
            }
            // MLP (egg.c:273-285)
            resid = x;
            xn = layer_norm(x, lnw + H);             // its barrier also orders the XN reads above before the write below
            if (own) put(XN, SH, wave, xn);
            __syncthreads();
            {
                const GruMat m = p.mats[6 * l + 4];
                const int xb = gru_xb<H / 32>(XN, p.noise + m.b_off + (long long)pair * H, lane);
                for (int ti = 0; ti < MAXT4; ti++) {
                    const int nt = wave + GRU_WAVES * ti;
                    if (nt < NT4) {
                        v16i acc;
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[r] = 0;
                        gru_strip<H / 32>(acc, p.frag + m.w_off + (size_t)nt * 32 * H, XN, lane);
                        put(MB, S4, nt, gru_finish(acc, xb, p.noise + m.a_off + (long long)pair * m.rows, nt, ns, p.sigma, m.shift, g));
                    }
                }
            }
            __syncthreads();
            v4i pr = matmul_h(6 * l + 5, MB, K4H);
            if (own)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int xo[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) xo[e] = cadd(sx8(pr[q], e), sx8(resid[q], e));
                    x[q] = pack4(xo[0], xo[1], xo[2], xo[3]);
                }
        }
        // head + loss (egg.c:288-294, :321-330)
        v4i xn = layer_norm(x, p.model + p.off_ln_out);
        if (own) put(XN, SH, wave, xn);
        __syncthreads();
        const int target = p.data[spos + t + 1];
        int part = 0;
        if (wave < V / 32) {
            const GruMat m = p.mats[6 * L];
            const int xb = gru_xb<H / 32>(XN, p.noise + m.b_off + (long long)pair * H, lane);
            v16i acc;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = 0;
            gru_strip<H / 32>(acc, p.frag + m.w_off + (size_t)wave * 32 * H, XN, lane);
            v4i lg = gru_finish(acc, xb, p.noise + m.a_off + (long long)pair * m.rows, wave, ns, p.sigma, m.shift, g);
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int v = sx8(lg[q], e);
                    part += lut[v + 128];
                    if (32 * wave + 8 * q + 4 * g + e == target) tl[j] = v;
                }
            part = sum_halves(part);
        }
        if (g == 0) psum[wave * 32 + j] = part;
        __syncthreads();
        {
            int sum_exp = 0;
            for (int w2 = 0; w2 < V / 32; w2++) sum_exp += psum[w2 * 32 + j];
            // log2_fixed (egg.c:309-319)
            int lg2 = 0;
            if (sum_exp > 0) {
                int k = 31 - __clz(sum_exp);
                int frac = (k >= 4) ? ((sum_exp - (1 << k)) >> (k - 4)) : ((sum_exp - (1 << k)) << (4 - k));
                lg2 = (k << 4) + frac - 64;
            }
            loss += lg2 - (tl[j] + 128);
        }
        __syncthreads();                           // psum is rewritten by the next token's first norm
    }
    if (wave == 0 && g == 0) p.loss[member] = loss;
}

// ============================================================================ the same forward, spread over the GPU
// k_gru_forward keeps a member tile on one workgroup for the whole sequence, so four workgroups stream every weight
// once per token from L2 and the rest of the GPU idles.  Here the work is cut into stages whose units spread over the
// CUs: a wave owns one (strip of 32 rows of W, tile of 32 members) pair, reads its W fragments and the tile's input
// straight from global memory and writes its 32 x 32 results back.  Same arithmetic helpers, bit-identical results.
//
// Every operand of a product is kept in the order the MFMA wants it, so that a wave's load of one k-step is one
// contiguous block: an activation buffer is [tile][k-step][half g][member j][16 bytes], the 16 bytes being a k-step's
// lane half in slot order, which is also exactly what a wave's 32 x 32 result packs to; the noise vectors have a
// second copy [pair tile][k-step][half][pair][16 bytes].  The recurrent state keeps its natural-order copy, the
// reference's layout, beside a copy in this order.
//
// Launches that depend on each other cost some microseconds apiece however small they are, so the sequence is walked as
// a pipeline in which one launch (a tick) carries every stage that is ready.  A layer's token passes six stages, one
// per tick:
//   0 norm (after the embedding for layer 0)   1 gate products, ft, gated   2 candidate, new state, residual
//   3 norm                                     4 MLP expand                 5 MLP project, residual
// Only stage 1 reads the state that stage 2 of the previous token wrote, so a layer starts a token every second tick;
// layer l runs six ticks behind layer l - 1, whose stage 5 hands it the residual stream.  Stage k of layer l's token t
// runs at tick 2 t + 6 l + k: even ticks carry stages 0, 2, 4 of every layer (tokens t, t - 1, t - 2), odd ticks stages
// 1, 3, 5.  The head is "layer L" with three stages: output norm, logits with their partial sums, loss.  A sequence is
// 2 T + 6 L + 1 ticks instead of T (6 L + 2) dependent launches.  Every layer has its own temporaries, each written at
// one tick and read at the next; the residual stream after each layer lives from stage 2 of the layer that writes it to
// stage 2 of the layer that reads it, seven ticks, so it is kept four times, by token number mod 4.
// The launches of several ticks form one linear hipGraph; the tick counter and the step's arguments sit in device
// memory (GruStep).  tick_base: ticks finished before the running graph (even); launch number `step` of the graph is
// tick tick_base + step.
struct GruStep { const uint8_t *data; long long data_len, start_idx; int tick_base; };
// how a tick's workgroups (256 threads) are dealt to the stages
struct GsGrid {
    int ln, g2, up, loss;                          // even ticks: workgroups per layer of stages 0, 2, 4; of the loss
    int g1, down, head;                            // odd ticks: per layer of stages 1 (3 waves a unit), 5 (4 waves a unit); of the logits
    __host__ __device__ int even(int L) const { return (up + g2) * L + ln * (L + 1) + loss; }
    __host__ __device__ int odd(int L) const { return (down + g1 + ln) * L + head; }
};
static GsGrid gs_grid(int population, int H, int V) {
    const int tiles = population / 32, nth = H / 32;
    GsGrid g;
    g.ln = tiles;
    g.g2 = (nth * tiles + 3) / 4; g.up = nth * tiles; g.loss = (population + 255) / 256;
    g.g1 = nth * tiles; g.down = nth * tiles; g.head = (V / 32 * tiles + 3) / 4;
    return g;
}
struct GsMat { long long w_off, a_off, b_off; int rows, shift; };      // what a product needs of a GruMat
enum { GS_MAX_MATS = 6 * 8 + 1 };
struct GruStage {
    const int8_t *model, *frag, *nfrag;            // nfrag: the noise vectors by pair tile, at the offsets of the plain copy
    GruStep *step;
    int8_t *states, *act;
    int32_t *head_sum, *head_tl;                  // [P][V / 32] sums of exp2 over a strip of logits, [P] the target's logit
    int32_t *loss;
    int H, L, V, T, population, sigma;
    long long off_emb, off_gru_b, off_ln_w, off_ln_out;
    const int32_t *exp2;
    GsGrid grid;
    GsMat m[GS_MAX_MATS];
};
// activations, [P][H] bytes each unless noted: the residual stream after li layers (li 0..L, four copies by token), the
// normed rows in front of layer li's gates (li == L: of the head) and in front of its MLP, the three gate temporaries,
// the state's copy in product order and the [P][4H] MLP intermediate of layer l
__device__ __forceinline__ size_t gs_ph(const GruStage &p) { return (size_t)p.population * p.H; }
__device__ __forceinline__ int8_t *gs_x(const GruStage &p, int li, int t) { return p.act + (size_t)(4 * li + (t & 3)) * gs_ph(p); }
__device__ __forceinline__ int8_t *gs_xn(const GruStage &p, int li) { return p.act + (size_t)(4 * (p.L + 1) + li) * gs_ph(p); }
__device__ __forceinline__ int8_t *gs_tmp(const GruStage &p, int which, int l) { return p.act + (size_t)(5 * (p.L + 1) + which * p.L + l) * gs_ph(p); }
__device__ __forceinline__ int8_t *gs_mb(const GruStage &p, int l) { return p.act + (size_t)(5 * (p.L + 1) + 5 * p.L + 4 * l) * gs_ph(p); }
enum { GS_XN2 = 0, GS_GATE = 1, GS_FT = 2, GS_M2 = 3, GS_HF = 4, GS_GRAPH_TICKS = 64 };
static size_t gs_act_bytes(int population, int H, int L) { return (size_t)population * H * (5 * (L + 1) + 9 * L); }
// where lane (g, j) keeps its 16 bytes of k-step ks of member tile `tile` in a buffer of K bytes per member
__device__ __forceinline__ size_t gs_at(int K, int tile, int ks, int g, int j) { return (size_t)tile * 32 * K + ((size_t)(ks * 2 + g) * 32 + j) * 16; }
// the same for a noise vector of `count` bytes per pair: the two members of a pair read the same 16 bytes
__device__ __forceinline__ size_t gs_noise_at(int count, int tile, int ks, int g, int j) { return (size_t)tile * 16 * count + ((size_t)(ks * 2 + g) * 16 + (j >> 1)) * 16; }
// the token whose stage k layer l runs at `tick` (their parities agree), or -1 while the pipeline fills or drains
__device__ __forceinline__ int gs_token(const GruStage &p, int tick, int l, int k) {
    const int d = tick - 6 * l - k;
    return (d < 0 || (d >> 1) >= p.T) ? -1 : d >> 1;
}
__device__ __forceinline__ long long gs_stream_pos(const GruStage &p, const GruStep &st, int member) {
    const long long stride = st.data_len / (p.population / 2);                    // egg.c:553-554
    return (st.start_idx + (long long)(member >> 1) * stride) % (st.data_len - p.T);
}

// KSN k-steps of a strip product starting at k-step ks0: acc += W[strip rows, k] . in[member, k], xb += in . B.
// fa, fb, fn: the lane's 16 bytes of k-step 0 of the W fragments, of the input tile and of the B noise.
template <int KSN>
__device__ __forceinline__ void gs_strip(v16i &acc, int &xb, const int8_t *fa, const int8_t *fb, const int8_t *fn, int ks0) {
    constexpr int BATCH = KSN < 8 ? KSN : 8;
    static_assert(KSN % BATCH == 0, "k-steps come in whole batches");
#pragma unroll 1
    for (int k0 = 0; k0 < KSN; k0 += BATCH) {
        v4i a[BATCH], b[BATCH], n[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const int ks = ks0 + k0 + u;
            a[u] = *reinterpret_cast<const v4i *>(fa + (size_t)ks * 1024);
            b[u] = *reinterpret_cast<const v4i *>(fb + (size_t)ks * 1024);
            n[u] = *reinterpret_cast<const v4i *>(fn + (size_t)ks * 512);
        }
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u], b[u], acc, 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 4; q++) xb = dot4(b[u][q], n[u][q], xb);
        }
    }
}
// one whole perturbed product of matrix mi for strip nt and member tile `tile`, whose input rows (KS * 32 bytes a
// member) start at in_tile: the lane's 16 packed int8 results, which are its piece (nt, g, j) of the output tile
template <int KS>
__device__ __forceinline__ v4i gs_matmul(const GruStage &p, int mi, int nt, const int8_t *in_tile, int tile, int lane) {
    const GsMat m = p.m[mi];
    const int j = lane & 31, g = lane >> 5, ns = (j & 1) ? -1 : 1;
    const v4i a4 = *reinterpret_cast<const v4i *>(p.nfrag + m.a_off + gs_noise_at(m.rows, tile, nt, g, j));
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    int xb = 0;
    gs_strip<KS>(acc, xb, p.frag + m.w_off + (size_t)nt * 32 * (KS * 32) + gs_at(0, 0, 0, g, j), in_tile + gs_at(0, 0, 0, g, j),
                 p.nfrag + m.b_off + gs_noise_at(KS * 32, tile, 0, g, j), 0);
    xb = sum_halves(xb);
    return gru_finish(acc, xb, a4, ns, p.sigma, m.shift);
}

// stages 0 and 3, and the head's stage 0: egg_ln (egg.c:180-210) of the rows of one member tile by one workgroup.
// Wave w holds the 32-groups w, w + 4, ... of the tile's rows, lane (g, j) its half g of member j's group.  Reads the
// residual stream after xi layers (embed: fills it first with the embedding row, egg.c:238) and writes `out`.
// lds: 4 x 32 ints.
template <int H>
__device__ __forceinline__ void gs_stage_ln(const GruStage &p, int tile, int t, int xi, bool embed, long long w_off, int8_t *out, int *lds) {
    constexpr int NTH = H / 32, NP = (NTH + 3) / 4;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31, member = tile * 32 + j;
    int8_t *xt = gs_x(p, xi, t);
    const int8_t *erow = nullptr;
    if (embed) {
        const GruStep st = *p.step;
        erow = p.model + p.off_emb + (size_t)st.data[gs_stream_pos(p, st, member) + t] * H;
    }
    v4i x[NP], wv[NP];
    int sum = 0;
    const int8_t *w = p.model + w_off;
#pragma unroll
    for (int i = 0; i < NP; i++) {                 // the gains are asked for here so that they arrive with the rows
        const int nt = wave + 4 * i;
        if (nt < NTH)
#pragma unroll
            for (int q = 0; q < 4; q++) wv[i][q] = *reinterpret_cast<const int *>(w + 32 * nt + 8 * q + 4 * g);
    }
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int nt = wave + 4 * i;
        if (nt < NTH) {
            if (embed) {
                const int *e = reinterpret_cast<const int *>(erow + 32 * nt);
#pragma unroll
                for (int q = 0; q < 4; q++) x[i][q] = e[2 * q + g];
                *reinterpret_cast<v4i *>(xt + gs_at(H, tile, nt, g, j)) = x[i];
            } else x[i] = *reinterpret_cast<const v4i *>(xt + gs_at(H, tile, nt, g, j));
#pragma unroll
            for (int q = 0; q < 4; q++) sum = sumabs4(x[i][q], sum);
        }
    }
    sum = sum_halves(sum);
    if (g == 0) lds[wave * 32 + j] = sum;
    __syncthreads();
    sum = lds[j] + lds[32 + j] + lds[64 + j] + lds[96 + j];
    if (sum == 0) sum = 1;
    int mean = sum / H; if (mean == 0) mean = 1;
    const float rcp = 1.0f / (float)mean;
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int nt = wave + 4 * i;
        if (nt < NTH) {
            v4i o4;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int w4 = wv[i][q];
                int o[4];
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = clip127(div_trunc(sx8(x[i][q], e) * sx8(w4, e), rcp));
                o4[q] = pack4(o[0], o[1], o[2], o[3]);
            }
            *reinterpret_cast<v4i *>(out + gs_at(H, tile, nt, g, j)) = o4;
        }
    }
}

// stage 1, gate products (egg.c:246-258): wave 0 W0.xn, wave 1 W1.h, wave 2 W2.xn of one (strip, member tile); then
// ft = cadd(cadd(W0 x, W1 h), b_f) and gated = ((ft + 127) h) >> 8 for the strip.  A whole workgroup; lds: 2 x 64 v4i.
template <int H>
__device__ __forceinline__ void gs_stage_gates1(const GruStage &p, int l, int nt, int tile, int *lds) {
    v4i *ex = reinterpret_cast<v4i *>(lds);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const size_t tile0 = gs_at(H, tile, 0, 0, 0), piece = gs_at(H, tile, nt, g, j);
    const int8_t *hf = gs_tmp(p, GS_HF, l);
    const int8_t *gb = p.model + p.off_gru_b + (size_t)l * 2 * H;
    v4i h, bf;                                     // what wave 0 needs behind the products, asked for in front of them
    if (wave == 0) {
        h = *reinterpret_cast<const v4i *>(hf + piece);
#pragma unroll
        for (int q = 0; q < 4; q++) bf[q] = *reinterpret_cast<const int *>(gb + 32 * nt + 8 * q + 4 * g);
    }
    v4i r;
    if (wave == 1) r = gs_matmul<H / 32>(p, 6 * l + 1, nt, hf + tile0, tile, lane);
    else if (wave != 3) r = gs_matmul<H / 32>(p, 6 * l + (wave == 0 ? 0 : 2), nt, gs_xn(p, l) + tile0, tile, lane);
    if (wave < 2) ex[wave * 64 + lane] = r;
    else if (wave == 2) *reinterpret_cast<v4i *>(gs_tmp(p, GS_M2, l) + piece) = r;
    __syncthreads();
    if (wave != 0) return;
    const v4i b1 = ex[lane], b2 = ex[64 + lane];
    v4i ft, gated;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int bf4 = bf[q];
        int f[4], gp[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            f[e] = cadd(cadd(sx8(b1[q], e), sx8(b2[q], e)), sx8(bf4, e));
            gp[e] = ((f[e] + 127) * sx8(h[q], e)) >> 8;
        }
        ft[q] = pack4(f[0], f[1], f[2], f[3]); gated[q] = pack4(gp[0], gp[1], gp[2], gp[3]);
    }
    *reinterpret_cast<v4i *>(gs_tmp(p, GS_FT, l) + piece) = ft;
    *reinterpret_cast<v4i *>(gs_tmp(p, GS_GATE, l) + piece) = gated;
}

// stage 2, candidate and state update (egg.c:260-271): ht = cadd(cadd(W2 x, W3 gated), b_h);
// h += ((ft + 127)(ht - h)) >> 8; x = cadd(h, x).  One wave per (strip, member tile).  The new state goes to the copy in
// product order only; the natural-order copy is brought up to date once, behind the last tick (k_gs_end).
// (Measured: as one workgroup per member tile with a wave per strip, which holds whole rows and can apply the following
// norm itself, it saves a stage but draws all of a matrix through four CUs: 8.2 instead of 4.6 us.)
template <int H>
__device__ __forceinline__ void gs_stage_gates2(const GruStage &p, int l, int t, int nt, int tile, int lane) {
    const int g = lane >> 5, j = lane & 31;
    const size_t piece = gs_at(H, tile, nt, g, j);
    int8_t *hf = gs_tmp(p, GS_HF, l) + piece;
    const v4i b1 = *reinterpret_cast<const v4i *>(gs_tmp(p, GS_M2, l) + piece), ft = *reinterpret_cast<const v4i *>(gs_tmp(p, GS_FT, l) + piece);
    const v4i h = *reinterpret_cast<const v4i *>(hf);
    v4i x = *reinterpret_cast<const v4i *>(gs_x(p, l, t) + piece);
    const int8_t *gb = p.model + p.off_gru_b + (size_t)l * 2 * H;
    v4i bh;
#pragma unroll
    for (int q = 0; q < 4; q++) bh[q] = *reinterpret_cast<const int *>(gb + H + 32 * nt + 8 * q + 4 * g);
    const v4i b2 = gs_matmul<H / 32>(p, 6 * l + 3, nt, gs_tmp(p, GS_GATE, l) + gs_at(H, tile, 0, 0, 0), tile, lane);
    v4i hnew;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int bh4 = bh[q];
        int hn[4], xo[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int ht = cadd(cadd(sx8(b1[q], e), sx8(b2[q], e)), sx8(bh4, e));
            const int hv = sx8(h[q], e);
            const int upd = ((sx8(ft[q], e) + 127) * (ht - hv)) >> 8;
            hn[e] = cadd(hv, upd);
            xo[e] = cadd(hn[e], sx8(x[q], e));
        }
        hnew[q] = pack4(hn[0], hn[1], hn[2], hn[3]); x[q] = pack4(xo[0], xo[1], xo[2], xo[3]);
    }
    *reinterpret_cast<v4i *>(hf) = hnew;
    *reinterpret_cast<v4i *>(gs_x(p, l + 1, t) + piece) = x;
}

// stage 4, MLP expand (egg.c:276-278): one wave per (strip of the 4H-wide intermediate, member tile)
template <int H>
__device__ __forceinline__ void gs_stage_up(const GruStage &p, int l, int nt, int tile, int lane) {
    const v4i r = gs_matmul<H / 32>(p, 6 * l + 4, nt, gs_tmp(p, GS_XN2, l) + gs_at(H, tile, 0, 0, 0), tile, lane);
    *reinterpret_cast<v4i *>(gs_mb(p, l) + gs_at(4 * H, tile, nt, lane >> 5, lane & 31)) = r;
}

// stage 5, MLP project + residual (egg.c:280-285): the 4H-deep product of one (strip, member tile) is dealt to the four
// waves of a workgroup by k range.  lds: 3 x 16 x 64 + 3 x 64 ints.
template <int H>
__device__ __forceinline__ void gs_stage_down(const GruStage &p, int l, int t, int nt, int tile, int *lds) {
    constexpr int KS4 = 4 * H / 32, KSW = KS4 / 4;
    int *red = lds, *xbp = lds + 3 * 16 * 64;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31, ns = (j & 1) ? -1 : 1;
    const GsMat m = p.m[6 * l + 5];
    int8_t *xrow = gs_x(p, l + 1, t) + gs_at(H, tile, nt, g, j);
    v4i x, a4;
    if (wave == 0) {
        x = *reinterpret_cast<const v4i *>(xrow);
        a4 = *reinterpret_cast<const v4i *>(p.nfrag + m.a_off + gs_noise_at(m.rows, tile, nt, g, j));
    }
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    int xb = 0;
    gs_strip<KSW>(acc, xb, p.frag + m.w_off + (size_t)nt * 32 * (4 * H) + gs_at(0, 0, 0, g, j), gs_mb(p, l) + gs_at(4 * H, tile, 0, g, j),
                  p.nfrag + m.b_off + gs_noise_at(4 * H, tile, 0, g, j), wave * KSW);
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) red[((wave - 1) * 16 + r) * 64 + lane] = acc[r];
        xbp[(wave - 1) * 64 + lane] = xb;
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 0; w < 3; w++) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] += red[(w * 16 + r) * 64 + lane];
        xb += xbp[w * 64 + lane];
    }
    xb = sum_halves(xb);
    const v4i pr = gru_finish(acc, xb, a4, ns, p.sigma, m.shift);
#pragma unroll
    for (int q = 0; q < 4; q++) {
        int xo[4];
#pragma unroll
        for (int e = 0; e < 4; e++) xo[e] = cadd(sx8(pr[q], e), sx8(x[q], e));
        x[q] = pack4(xo[0], xo[1], xo[2], xo[3]);
    }
    *reinterpret_cast<v4i *>(xrow) = x;
}

// the head's stage 1 (egg.c:288-294): a wave forms one strip of 32 logits of a member tile, sums their exp2 and keeps
// the target's logit
template <int H>
__device__ __forceinline__ void gs_stage_logits(const GruStage &p, int t, int nt, int tile, int lane) {
    const int g = lane >> 5, member = tile * 32 + (lane & 31);
    const GruStep st = *p.step;
    const int target = st.data[gs_stream_pos(p, st, member) + t + 1];
    const v4i lg = gs_matmul<H / 32>(p, 6 * p.L, nt, gs_xn(p, p.L) + gs_at(H, tile, 0, 0, 0), tile, lane);
    int part = 0, tl = 0;
    bool mine = false;
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int v = sx8(lg[q], e);
            part += p.exp2[v + 128];
            if (32 * nt + 8 * q + 4 * g + e == target) { tl = v; mine = true; }
        }
    part = sum_halves(part);
    if (g == 0) p.head_sum[(size_t)member * (p.V / 32) + nt] = part;
    if (mine) p.head_tl[member] = tl;
}
// the head's stage 2: a member's loss for the token (egg.c:321-330) from the strips' sums
__device__ __forceinline__ void gs_stage_loss(const GruStage &p, int member) {
    int sum_exp = 0;
    for (int s = 0; s < p.V / 32; s++) sum_exp += p.head_sum[(size_t)member * (p.V / 32) + s];
    int lg2 = 0;                                   // log2_fixed (egg.c:309-319)
    if (sum_exp > 0) {
        const int k = 31 - __clz(sum_exp);
        const int frac = (k >= 4) ? ((sum_exp - (1 << k)) >> (k - 4)) : ((sum_exp - (1 << k)) << (4 - k));
        lg2 = (k << 4) + frac - 64;
    }
    p.loss[member] += lg2 - (p.head_tl[member] + 128);
}

// One tick.  ODD false: stages 4, 2, 0 of every layer, the output norm and the loss; true: stages 5, 1, 3 and the logits.
// The workgroups are dealt to the stages in that order (the deepest products first); every branch below is taken by a
// whole workgroup, except that waves past a stage's last unit leave where the stage has no barrier.
template <int H, bool ODD>
__global__ void __launch_bounds__(256) k_gs_tick(GruStage p, int step) {
    __shared__ int lds[3 * 16 * 64 + 3 * 64];
    const int tick = p.step->tick_base + step, L = p.L, tiles = p.population / 32, nth = H / 32;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const GsGrid &gr = p.grid;
    int b = blockIdx.x;
    if (!ODD) {
        if (b < gr.up * L) {
            const int l = b / gr.up, unit = (b % gr.up) * 4 + wave, t = gs_token(p, tick, l, 4);
            if (t >= 0) gs_stage_up<H>(p, l, unit % (4 * nth), unit / (4 * nth), lane);
            return;
        }
        b -= gr.up * L;
        if (b < gr.g2 * L) {
            const int l = b / gr.g2, unit = (b % gr.g2) * 4 + wave, t = gs_token(p, tick, l, 2);
            if (t >= 0 && unit < nth * tiles) gs_stage_gates2<H>(p, l, t, unit % nth, unit / nth, lane);
            return;
        }
        b -= gr.g2 * L;
        if (b < gr.ln * (L + 1)) {
            const int l = b / gr.ln, t = gs_token(p, tick, l, 0);
            if (t >= 0) gs_stage_ln<H>(p, b % gr.ln, t, l, l == 0, l == L ? p.off_ln_out : p.off_ln_w + (long long)l * 2 * H, gs_xn(p, l), lds);
            return;
        }
        b -= gr.ln * (L + 1);
        const int member = b * 256 + threadIdx.x;
        if (gs_token(p, tick, L, 2) >= 0 && member < p.population) gs_stage_loss(p, member);
    } else {
        if (b < gr.down * L) {
            const int l = b / gr.down, unit = b % gr.down, t = gs_token(p, tick, l, 5);
            if (t >= 0) gs_stage_down<H>(p, l, t, unit % nth, unit / nth, lds);
            return;
        }
        b -= gr.down * L;
        if (b < gr.g1 * L) {
            const int l = b / gr.g1, unit = b % gr.g1;
            if (gs_token(p, tick, l, 1) >= 0) gs_stage_gates1<H>(p, l, unit % nth, unit / nth, lds);
            return;
        }
        b -= gr.g1 * L;
        if (b < gr.ln * L) {
            const int l = b / gr.ln, t = gs_token(p, tick, l, 3);
            if (t >= 0) gs_stage_ln<H>(p, b % gr.ln, t, l + 1, false, p.off_ln_w + (long long)l * 2 * H + H, gs_tmp(p, GS_XN2, l), lds);
            return;
        }
        b -= gr.ln * L;
        const int nv = p.V / 32, unit = b * 4 + wave, t = gs_token(p, tick, L, 1);
        if (t >= 0 && unit < nv * tiles) gs_stage_logits<H>(p, t, unit % nv, unit / nv, lane);
    }
}
// last node of a graph: its ticks are finished
__global__ void k_gs_advance(GruStep *st, int ticks) { if (threadIdx.x == 0) st->tick_base += ticks; }
// before the first tick: the step's arguments, zero losses, and the state's copy in product order from the natural one
__global__ void k_gs_begin(GruStage p, const uint8_t *data, long long data_len, long long start_idx) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) { GruStep *st = p.step; st->data = data; st->data_len = data_len; st->start_idx = start_idx; st->tick_base = 0; }
    if (i < p.population) p.loss[i] = 0;
    const int H = p.H, per_member = p.L * (H / 16);
    if (i >= p.population * per_member) return;
    const int member = i / per_member, r = i % per_member, l = r / (H / 16), piece = r % (H / 16), nt = piece >> 1, g = piece & 1;
    const int *h32 = reinterpret_cast<const int *>(p.states + ((size_t)member * p.L + l) * H + 32 * nt);
    v4i h;
#pragma unroll
    for (int q = 0; q < 4; q++) h[q] = h32[2 * q + g];
    *reinterpret_cast<v4i *>(gs_tmp(p, GS_HF, l) + gs_at(H, member >> 5, nt, g, member & 31)) = h;
}
// behind the last tick: the natural-order state from its copy in product order
__global__ void k_gs_end(GruStage p) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int H = p.H, per_member = p.L * (H / 16);
    if (i >= p.population * per_member) return;
    const int member = i / per_member, r = i % per_member, l = r / (H / 16), piece = r % (H / 16), nt = piece >> 1, g = piece & 1;
    const v4i h = *reinterpret_cast<const v4i *>(gs_tmp(p, GS_HF, l) + gs_at(H, member >> 5, nt, g, member & 31));
    int *h32 = reinterpret_cast<int *>(p.states + ((size_t)member * p.L + l) * H + 32 * nt);
#pragma unroll
    for (int q = 0; q < 4; q++) h32[2 * q + g] = h[q];
}

// A panel *= fitness of the pair (A_T[r][p] = A[r] * f, egg.c:362-366)
__global__ void k_gru_scale_panel(int8_t *panel, long long n, int pairs_pad, int pairs, const int32_t *fit) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int pp = (int)(i % pairs_pad);
    panel[i] = (pp < pairs) ? (int8_t)(panel[i] * fit[pp]) : (int8_t)0;
}

// update_matrix (egg.c:332-409): vote[r][c] = sum_p A_T[r][p] B_T[c][p] on the MFMA, then the +-1 threshold rule
__global__ void __launch_bounds__(256) k_gru_vote_update(int8_t *W, const int8_t *pa, const int8_t *pb, int rows, int cols,
                                                        int pairs_pad, int threshold) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const int tiles_c = cols / 32, tile = blockIdx.x * 4 + wave;
    if (tile >= (rows / 32) * tiles_c) return;
    const int r0 = (tile / tiles_c) * 32, c0 = (tile % tiles_c) * 32;
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    for (int s = 0; s < pairs_pad; s += 32) {
        v4i a = *reinterpret_cast<const v4i *>(pb + (size_t)(c0 + j) * pairs_pad + s + 16 * g);   // rows of the MFMA = input index c
        v4i b = *reinterpret_cast<const v4i *>(pa + (size_t)(r0 + j) * pairs_pad + s + 16 * g);   // columns = output row r
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc, 0, 0, 0);
    }
    // lane (r = r0 + j, half g), register 4q+e -> c = c0 + 8q + 4g + e
#pragma unroll
    for (int q = 0; q < 4; q++) {
        int *wp = reinterpret_cast<int *>(W + (size_t)(r0 + j) * cols + c0 + 8 * q + 4 * g);
        int w4 = *wp, o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int w = sx8(w4, e), vote = acc[4 * q + e];
            if (vote > threshold && w < 127) w++;
            else if (vote < -threshold && w > -127) w--;
            o[e] = w;
        }
        *wp = pack4(o[0], o[1], o[2], o[3]);
    }
}

// ---------------------------------------------------------------------------------------------- host side / C ABI
struct egg_gru_ctx {
    egg_gru_config cfg;
    hipStream_t stream = nullptr;
    std::vector<GruMat> mats;
    long long model_bytes = 0, noise_bytes = 0, panel_bytes = 0, off_emb = 0, off_gru_w = 0, off_gru_b = 0, off_mlp_w = 0,
              off_head = 0, off_ln_w = 0, off_ln_out = 0;
    int pairs_pad = 0;
    int8_t *d_model = nullptr, *d_frag = nullptr, *d_noise = nullptr, *d_panels = nullptr, *d_states = nullptr;
    GruMat *d_mats = nullptr; int32_t *d_loss = nullptr, *d_fit = nullptr, *d_exp2 = nullptr;
    // the forward spread over the GPU (egg_gru_forward_mode): activations in global memory, the head's partial sums, the
    // step's arguments, and two graphs: one of `graph_ticks` ticks, one of two ticks for what is left of the sequence
    bool staged = true;
    int8_t *d_act = nullptr, *d_nfrag = nullptr; GruStep *d_step = nullptr; int32_t *d_head = nullptr;
    int graph_ticks = 0;
    hipGraph_t tok_graph[2] = {nullptr, nullptr}; hipGraphExec_t tok_exec[2] = {nullptr, nullptr};
    std::string err;
};
static int gfail(egg_gru_ctx *c, int code, const char *what, hipError_t e = hipSuccess) {
    if (c) { c->err = what; if (e != hipSuccess) { c->err += ": "; c->err += hipGetErrorString(e); } }
    return code;
}
#define GTRY(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return gfail(ctx, EGG_E_HIP, #call, e_); } while (0)

extern "C" void egg_gru_default_config(egg_gru_config *c) {
    c->hidden = 512; c->n_layers = 4; c->seq_len = 4096; c->vocab = 256; c->population = 128;
    c->fixed_point = 4; c->sigma_shift = 4; c->update_threshold = 160;
}

static size_t gru_lds_bytes(int H) { return (size_t)32 * (H + 16) * 2 + (size_t)32 * (4 * H + 16) + (GRU_WAVES * 32 + 32 + 256) * 4; }

template <int H>
static hipError_t gru_prepare() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gru_forward<H>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)gru_lds_bytes(H));
}

static int gru_refresh_frag(egg_gru_ctx *ctx) {
    for (const GruMat &m : ctx->mats) {
        int chunks = m.rows * m.cols / 16;
        hipLaunchKernelGGL(k_gru_swizzle, dim3((chunks + 255) / 256), dim3(256), 0, ctx->stream, ctx->d_model + m.w_off,
                           ctx->d_frag + m.w_off, m.rows, m.cols);
    }
    GTRY(hipGetLastError());
    return EGG_OK;
}

extern "C" int egg_gru_create(const egg_gru_config *cfg, egg_gru_ctx **out) {
    if (!cfg || !out) return EGG_E_INVALID;
    *out = nullptr;
    const egg_gru_config &c = *cfg;
    if (!(c.hidden == 64 || c.hidden == 128 || c.hidden == 256 || c.hidden == 512)) return EGG_E_INVALID;
    if (c.vocab != 256 || c.n_layers < 1 || c.n_layers > 8 || c.population < 32 || c.population % 32 || c.seq_len < 1) return EGG_E_INVALID;
    egg_gru_ctx *ctx = new egg_gru_ctx(); ctx->cfg = c;
    const long long H = c.hidden, V = c.vocab, L = c.n_layers;
    long long o = 0;
    ctx->off_emb = o; o += V * H;
    ctx->off_gru_w = o; o += L * 4 * H * H;
    ctx->off_gru_b = o; o += L * 2 * H;
    ctx->off_mlp_w = o; o += L * 2 * H * 4 * H;
    ctx->off_head = o; o += H * V;
    ctx->off_ln_w = o; o += L * 2 * H;
    ctx->off_ln_out = o; o += H;
    ctx->model_bytes = o;
    const int pairs = c.population / 2;
    ctx->pairs_pad = (pairs + 31) / 32 * 32;
    long long no = 0, po = 0;
    auto add = [&](long long w_off, int rows, int cols, int seed_off, int shift) {
        GruMat m; m.w_off = w_off; m.rows = rows; m.cols = cols; m.seed_off = seed_off; m.shift = shift;
        m.a_off = no; no += (long long)pairs * rows; m.b_off = no; no += (long long)pairs * cols;
        m.pa_off = po; po += (long long)rows * ctx->pairs_pad; m.pb_off = po; po += (long long)cols * ctx->pairs_pad;
        ctx->mats.push_back(m);
    };
    for (int l = 0; l < L; l++) {
        for (int g = 0; g < 4; g++) add(ctx->off_gru_w + ((long long)l * 4 + g) * H * H, (int)H, (int)H, 100 * l + 1 + g, 8);
        add(ctx->off_mlp_w + ((long long)l * 2) * H * 4 * H, (int)(4 * H), (int)H, 100 * l + 5, 8);
        add(ctx->off_mlp_w + ((long long)l * 2 + 1) * H * 4 * H, (int)H, (int)(4 * H), 100 * l + 6, 9);
    }
    add(ctx->off_head, (int)V, (int)H, 999, 8);
    ctx->noise_bytes = no; ctx->panel_bytes = po;
    auto bail = [&](const char *what, hipError_t e) { fprintf(stderr, "egg_gru_create: %s: %s\n", what, hipGetErrorString(e)); egg_gru_destroy(ctx); return EGG_E_HIP; };   // frees what was allocated so far
#define CR(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return bail(#call, e_); } while (0)
    CR(hipStreamCreate(&ctx->stream));
    switch (c.hidden) {
        case 64: CR(gru_prepare<64>()); break;
        case 128: CR(gru_prepare<128>()); break;
        case 256: CR(gru_prepare<256>()); break;
        default: CR(gru_prepare<512>()); break;
    }
    CR(hipMalloc(&ctx->d_model, ctx->model_bytes)); CR(hipMemset(ctx->d_model, 0, ctx->model_bytes));
    CR(hipMalloc(&ctx->d_frag, ctx->model_bytes));
    CR(hipMalloc(&ctx->d_noise, ctx->noise_bytes)); CR(hipMalloc(&ctx->d_panels, ctx->panel_bytes));
    CR(hipMemset(ctx->d_panels, 0, ctx->panel_bytes));
    CR(hipMalloc(&ctx->d_states, (size_t)c.population * L * H)); CR(hipMemset(ctx->d_states, 0, (size_t)c.population * L * H));
    CR(hipMalloc(&ctx->d_mats, ctx->mats.size() * sizeof(GruMat)));
    CR(hipMemcpy(ctx->d_mats, ctx->mats.data(), ctx->mats.size() * sizeof(GruMat), hipMemcpyHostToDevice));
    CR(hipMalloc(&ctx->d_loss, (size_t)c.population * 4)); CR(hipMalloc(&ctx->d_fit, (size_t)pairs * 4));
    int32_t ex[256];
    for (int i = 0; i < 256; i++) ex[i] = (int32_t)(pow(2.0, (double)i / (1 << c.fixed_point)) * (1 << c.fixed_point));   // egg.c:57-60
    CR(hipMalloc(&ctx->d_exp2, 1024)); CR(hipMemcpy(ctx->d_exp2, ex, 1024, hipMemcpyHostToDevice));
    CR(hipMalloc(&ctx->d_act, gs_act_bytes(c.population, c.hidden, c.n_layers)));
    CR(hipMalloc(&ctx->d_nfrag, ctx->noise_bytes));
    CR(hipMalloc(&ctx->d_head, (size_t)c.population * (c.vocab / 32 + 1) * 4));
    CR(hipMalloc(&ctx->d_step, sizeof(GruStep))); CR(hipMemset(ctx->d_step, 0, sizeof(GruStep)));
#undef CR
    *out = ctx;
    return EGG_OK;
}
extern "C" void egg_gru_destroy(egg_gru_ctx *ctx) {
    if (!ctx) return;
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    for (int i = 0; i < 2; i++) {
        if (ctx->tok_exec[i]) (void)hipGraphExecDestroy(ctx->tok_exec[i]);
        if (ctx->tok_graph[i]) (void)hipGraphDestroy(ctx->tok_graph[i]);
    }
    void *ptrs[] = {ctx->d_model, ctx->d_frag, ctx->d_noise, ctx->d_panels, ctx->d_states, ctx->d_mats, ctx->d_loss, ctx->d_fit, ctx->d_exp2,
                    ctx->d_act, ctx->d_step, ctx->d_head, ctx->d_nfrag};
    for (void *q : ptrs) if (q) (void)hipFree(q);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}
extern "C" const char *egg_gru_last_error(const egg_gru_ctx *ctx) { return ctx ? ctx->err.c_str() : "null context"; }
extern "C" int64_t egg_gru_model_bytes(const egg_gru_ctx *ctx) { return ctx ? ctx->model_bytes : 0; }

// model init of egg.c:487-509: one xorshift32 stream, noise magnitude mask 31
extern "C" int egg_gru_model_init(egg_gru_ctx *ctx, uint32_t seed) {
    if (!ctx) return EGG_E_INVALID;
    const long long H = ctx->cfg.hidden, V = ctx->cfg.vocab, L = ctx->cfg.n_layers;
    std::vector<int8_t> m((size_t)ctx->model_bytes, 0);
    uint32_t rng = seed;
    auto draw = [&]() { uint32_t x = rng; x ^= x << 13; x ^= x >> 17; x ^= x << 5; rng = x; return (int8_t)((x & 1 ? 1 : -1) * (int)((x >> 1) & 31)); };
    for (long long i = 0; i < V * H; i++) m[ctx->off_emb + i] = draw();
    for (long long i = 0; i < H * V; i++) m[ctx->off_head + i] = draw();
    for (long long l = 0; l < L; l++) {
        for (long long i = 0; i < 4 * H * H; i++) m[ctx->off_gru_w + l * 4 * H * H + i] = draw();
        for (long long i = 0; i < 2 * H * 4 * H; i++) m[ctx->off_mlp_w + l * 2 * H * 4 * H + i] = draw();
    }
    for (long long i = 0; i < L * 2 * H; i++) m[ctx->off_ln_w + i] = 16;
    for (long long i = 0; i < H; i++) m[ctx->off_ln_out + i] = 16;
    GTRY(hipStreamSynchronize(ctx->stream));
    GTRY(hipMemcpy(ctx->d_model, m.data(), m.size(), hipMemcpyHostToDevice));
    return gru_refresh_frag(ctx);
}
extern "C" int egg_gru_model_upload(egg_gru_ctx *ctx, const void *h, size_t bytes) {
    if (!ctx || !h || (long long)bytes != ctx->model_bytes) return gfail(ctx, EGG_E_INVALID, "model size mismatch");
    GTRY(hipStreamSynchronize(ctx->stream));
    GTRY(hipMemcpy(ctx->d_model, h, bytes, hipMemcpyHostToDevice));
    return gru_refresh_frag(ctx);
}
extern "C" int egg_gru_model_download(egg_gru_ctx *ctx, void *h, size_t bytes) {
    if (!ctx || !h || (long long)bytes != ctx->model_bytes) return gfail(ctx, EGG_E_INVALID, "model size mismatch");
    GTRY(hipStreamSynchronize(ctx->stream));
    GTRY(hipMemcpy(h, ctx->d_model, bytes, hipMemcpyDeviceToHost));
    return EGG_OK;
}
extern "C" int egg_gru_state_reset(egg_gru_ctx *ctx) {
    if (!ctx) return EGG_E_INVALID;
    GTRY(hipStreamSynchronize(ctx->stream));
    GTRY(hipMemset(ctx->d_states, 0, (size_t)ctx->cfg.population * ctx->cfg.n_layers * ctx->cfg.hidden));
    return EGG_OK;
}
extern "C" int egg_gru_state_download(egg_gru_ctx *ctx, void *h, size_t bytes) {
    if (!ctx) return EGG_E_INVALID;
    const size_t want = (size_t)ctx->cfg.population * ctx->cfg.n_layers * ctx->cfg.hidden;
    if (!h || bytes != want) return gfail(ctx, EGG_E_INVALID, "state size mismatch");
    GTRY(hipStreamSynchronize(ctx->stream));
    GTRY(hipMemcpy(h, ctx->d_states, want, hipMemcpyDeviceToHost));
    return EGG_OK;
}

// A kernel node whose arguments are the values given (the graph keeps its own copy of them)
template <typename... KA, typename... A>
static hipError_t gs_node(hipGraph_t g, hipGraphNode_t *out, const std::vector<hipGraphNode_t> &deps, void (*fn)(KA...), dim3 grid, dim3 block, A... args) {
    std::tuple<KA...> vals{static_cast<KA>(args)...};
    void *params[sizeof...(KA)];
    int n = 0;
    std::apply([&](auto &...v) { ((params[n++] = (void *)&v), ...); }, vals);
    hipKernelNodeParams kp = {};
    kp.func = reinterpret_cast<void *>(fn); kp.gridDim = grid; kp.blockDim = block; kp.sharedMemBytes = 0; kp.kernelParams = params; kp.extra = nullptr;
    return hipGraphAddKernelNode(out, g, deps.empty() ? nullptr : deps.data(), deps.size(), &kp);
}
// The graph of `ticks` ticks (an even number) of the forward: a chain of launches, then the tick counter moves on
template <int H>
static hipError_t gru_build_graph(egg_gru_ctx *ctx, const GruStage &p, int ticks, hipGraph_t *out) {
    const int L = ctx->cfg.n_layers;
    hipGraph_t g = nullptr;
    hipError_t e = hipGraphCreate(&g, 0);
    if (e != hipSuccess) return e;
#define GR(call) do { e = (call); if (e != hipSuccess) { (void)hipGraphDestroy(g); return e; } } while (0)
    hipGraphNode_t n = nullptr;
    auto after = [&]() { return n ? std::vector<hipGraphNode_t>{n} : std::vector<hipGraphNode_t>{}; };
    for (int i = 0; i < ticks; i++) {
        if (i & 1) GR(gs_node(g, &n, after(), k_gs_tick<H, true>, dim3((unsigned)p.grid.odd(L)), dim3(256), p, i));
        else GR(gs_node(g, &n, after(), k_gs_tick<H, false>, dim3((unsigned)p.grid.even(L)), dim3(256), p, i));
    }
    GR(gs_node(g, &n, after(), k_gs_advance, dim3(1), dim3(64), p.step, ticks));
#undef GR
    *out = g;
    return hipSuccess;
}
static hipError_t gru_build_graph_h(egg_gru_ctx *ctx, const GruStage &p, int ticks, hipGraph_t *out) {
    switch (ctx->cfg.hidden) {
        case 64: return gru_build_graph<64>(ctx, p, ticks, out);
        case 128: return gru_build_graph<128>(ctx, p, ticks, out);
        case 256: return gru_build_graph<256>(ctx, p, ticks, out);
        default: return gru_build_graph<512>(ctx, p, ticks, out);
    }
}
static int gru_forward_staged(egg_gru_ctx *ctx, const uint8_t *d_data, int64_t data_len, int64_t start_idx) {
    const egg_gru_config &c = ctx->cfg;
    GruStage p;
    p.model = ctx->d_model; p.frag = ctx->d_frag; p.nfrag = ctx->d_nfrag; p.step = ctx->d_step;
    p.states = ctx->d_states; p.act = ctx->d_act; p.head_sum = ctx->d_head; p.head_tl = ctx->d_head + (size_t)c.population * (c.vocab / 32);
    p.loss = ctx->d_loss;
    p.H = c.hidden; p.L = c.n_layers; p.V = c.vocab; p.T = c.seq_len; p.population = c.population; p.sigma = c.fixed_point + c.sigma_shift;
    p.off_emb = ctx->off_emb; p.off_gru_b = ctx->off_gru_b; p.off_ln_w = ctx->off_ln_w; p.off_ln_out = ctx->off_ln_out; p.exp2 = ctx->d_exp2;
    p.grid = gs_grid(c.population, c.hidden, c.vocab);
    for (size_t i = 0; i < ctx->mats.size(); i++) { const GruMat &m = ctx->mats[i]; p.m[i] = GsMat{m.w_off, m.a_off, m.b_off, m.rows, m.shift}; }
    const long long pieces = (long long)c.population * c.n_layers * (c.hidden / 16);
    hipLaunchKernelGGL(k_gs_begin, dim3((unsigned)((std::max<long long>(pieces, c.population) + 255) / 256)), dim3(256), 0, ctx->stream, p, d_data,
                       (long long)data_len, (long long)start_idx);
    GTRY(hipGetLastError());
    // a sequence is 2 T + 6 L + 1 ticks, rounded up to an even number (a tick past the end finds no token).  Ticks per
    // graph: the largest power of two up to 64 that fits (a graph launch costs more than the gap between two of its
    // nodes); a two-tick graph takes what is left
    const int total = (2 * c.seq_len + 6 * c.n_layers + 2) & ~1;
    if (!ctx->graph_ticks) { int k = 2; while (2 * k <= total && 2 * k <= GS_GRAPH_TICKS) k *= 2; ctx->graph_ticks = k; }
    const int K = ctx->graph_ticks;
    for (int which = 0; which < 2; which++) {
        const int ticks = which == 0 ? K : 2;
        if (ctx->tok_exec[which] || (which == 1 && (K == 2 || total % K == 0))) continue;
        // every argument of the launches is fixed for the life of the context (the step's own arguments sit in *d_step)
        hipGraph_t g = nullptr;
        const hipError_t e = gru_build_graph_h(ctx, p, ticks, &g);
        if (e != hipSuccess) return gfail(ctx, EGG_E_HIP, "graph of the forward's ticks", e);
        ctx->tok_graph[which] = g;
        GTRY(hipGraphInstantiate(&ctx->tok_exec[which], g, nullptr, nullptr, 0));
    }
    int t = 0;
    for (; t + K <= total; t += K) GTRY(hipGraphLaunch(ctx->tok_exec[0], ctx->stream));
    for (; t < total; t += 2) GTRY(hipGraphLaunch(ctx->tok_exec[1], ctx->stream));
    hipLaunchKernelGGL(k_gs_end, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, ctx->stream, p);
    GTRY(hipGetLastError());
    return EGG_OK;
}
// 1 (default): the stages spread over the whole GPU, a launch per pipeline tick; 0: one persistent workgroup per 32 members
extern "C" int egg_gru_forward_mode(egg_gru_ctx *ctx, int staged) {
    if (!ctx) return EGG_E_INVALID;
    ctx->staged = staged != 0;
    return EGG_OK;
}

extern "C" int egg_gru_step(egg_gru_ctx *ctx, const uint8_t *d_data, int64_t data_len, int64_t start_idx, uint32_t step_seed, int do_update) {
    if (!ctx || !d_data || data_len <= ctx->cfg.seq_len + 1) return gfail(ctx, EGG_E_INVALID, "egg_gru_step arguments");
    const egg_gru_config &c = ctx->cfg;
    const int pairs = c.population / 2, nm = (int)ctx->mats.size();
    hipLaunchKernelGGL(k_gru_noise, dim3((nm * pairs + 63) / 64), dim3(64), 0, ctx->stream, ctx->d_mats, nm, pairs, ctx->pairs_pad,
                       step_seed, ctx->d_noise, ctx->d_nfrag, ctx->d_panels);
    GruParams p;
    p.mats = ctx->d_mats; p.model = ctx->d_model; p.frag = ctx->d_frag; p.noise = ctx->d_noise;
    p.data = d_data; p.data_len = data_len; p.start_idx = start_idx; p.states = ctx->d_states; p.loss = ctx->d_loss;
    p.H = c.hidden; p.L = c.n_layers; p.T = c.seq_len; p.V = c.vocab; p.population = c.population; p.sigma = c.fixed_point + c.sigma_shift;
    p.off_emb = ctx->off_emb; p.off_gru_b = ctx->off_gru_b; p.off_ln_w = ctx->off_ln_w; p.off_ln_out = ctx->off_ln_out; p.exp2 = ctx->d_exp2;
    if (ctx->staged) {
        int rc = gru_forward_staged(ctx, d_data, data_len, start_idx);
        if (rc) return rc;
    } else {
        dim3 grid(c.population / 32), block(GRU_THREADS);
        size_t lds = gru_lds_bytes(c.hidden);
        switch (c.hidden) {
            case 64: hipLaunchKernelGGL((k_gru_forward<64>), grid, block, lds, ctx->stream, p); break;
            case 128: hipLaunchKernelGGL((k_gru_forward<128>), grid, block, lds, ctx->stream, p); break;
            case 256: hipLaunchKernelGGL((k_gru_forward<256>), grid, block, lds, ctx->stream, p); break;
            default: hipLaunchKernelGGL((k_gru_forward<512>), grid, block, lds, ctx->stream, p); break;
        }
        GTRY(hipGetLastError());
    }
    // pair fitness (egg.c:559-561) has the same rule as the transformer's
    GTRY(egg_launch_fitness(ctx->d_loss, ctx->d_fit, pairs, ctx->stream));
    if (do_update) {
        for (const GruMat &m : ctx->mats) {
            long long n = (long long)m.rows * ctx->pairs_pad;
            hipLaunchKernelGGL(k_gru_scale_panel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, ctx->d_panels + m.pa_off, n,
                               ctx->pairs_pad, pairs, ctx->d_fit);
            int tiles = (m.rows / 32) * (m.cols / 32);
            hipLaunchKernelGGL(k_gru_vote_update, dim3((tiles + 3) / 4), dim3(256), 0, ctx->stream, ctx->d_model + m.w_off,
                               ctx->d_panels + m.pa_off, ctx->d_panels + m.pb_off, m.rows, m.cols, ctx->pairs_pad, c.update_threshold);
        }
        GTRY(hipGetLastError());
        return gru_refresh_frag(ctx);
    }
    return EGG_OK;
}
extern "C" int egg_gru_losses(egg_gru_ctx *ctx, int32_t *h_loss, int32_t *h_fit) {
    if (!ctx) return EGG_E_INVALID;
    GTRY(hipStreamSynchronize(ctx->stream));
    if (h_loss) GTRY(hipMemcpy(h_loss, ctx->d_loss, (size_t)ctx->cfg.population * 4, hipMemcpyDeviceToHost));
    if (h_fit) GTRY(hipMemcpy(h_fit, ctx->d_fit, (size_t)(ctx->cfg.population / 2) * 4, hipMemcpyDeviceToHost));
    return EGG_OK;
}
