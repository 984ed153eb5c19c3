// egg_linear.hip -- one perturbed int8 linear layer over a [members*T][K] activation matrix.
// Reference: compute_linear_projection, full_cuda_train_transformer_adam_mgpu.cu:553-572, applied to
// every (member, token) row: acc = x.W + (((x.B) * A[n]) * ns >> sigma), out = acc >> shift.
// Same tile scheme as the forward kernels (wave = 32 tokens of one member, W through LDS,
// v_mfma_i32_32x32x32_i8), with the row-major input read in natural k order.
//
// This kernel has almost no elementwise work per output, so memory behaviour decides: W units of at most 16 KB go
// through a ring of three LDS buffers and are requested two units ahead of their use, the activation rows of the
// next token tile are loaded while the current one is multiplied, and results leave through a per-wave LDS
// transpose so that eight lanes write one full 128-byte line of a row (in the MFMA result layout a store
// instruction would touch 32 rows with 32 bytes each).
#include <type_traits>
#include "egg_device.h"
#include "egg_launch.h"

template <int K, int N>
struct Plin {
    static constexpr int cmin(int a, int b) { return a < b ? a : b; }
    static constexpr int B = cmin(cmin(K, N), 128);              // fragment block size = output columns per accumulator
    static constexpr int NTB = B / 32, KS = K / 32;
    static constexpr int PR = cmin(B / 16, 1024 / B);            // p-rows per unit (two per k-step)
    static constexpr int KSU = PR / 2;                           // k-steps per unit
    static constexpr int UPB = (B / 16) / PR;                    // units per block
    static constexpr int UNITS_NB = (K / B) * UPB;               // units per column block
    static constexpr int NBLK = N / B;
    static constexpr int UPP = UNITS_NB * NBLK;                  // units per token tile
    static constexpr int UNIT = PR * B * 16;
    static constexpr int NBUF = 3, AHEAD = 2;
    static constexpr int PER_WAVE = N * 4 + K;                   // A noise * sign (int32), B noise (int8)
    static constexpr int STAGE = 32 * 128;                       // per-wave transpose tile: 32 rows x 128 bytes
    static constexpr int TOTAL = NBUF * UNIT + EGG_WAVES * (PER_WAVE + STAGE);
    static constexpr bool PREFETCH_X = false;                   // the next tile's rows fit in registers next to the current
};

// Wait until at most `units` later W units (PER copy instructions each) plus EXTRA other vector memory operations of
// this wave are outstanding.  Vector memory operations of a wave complete in issue order, so this leaves exactly the
// operations issued after the wanted unit in flight; EXTRA may be an undercount (the wait is then stricter), never
// an overcount.
template <int PER, int EXTRA>
__device__ __forceinline__ void wait_unit(int units) {
    constexpr int A = PER + EXTRA, Z = EXTRA;
    static_assert(A < 64, "vmcnt has six bits");
    if (units >= 1) __builtin_amdgcn_s_waitcnt(0x0F70 | (A & 15) | ((A >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0F70 | (Z & 15) | ((Z >> 4) << 14));
}

// OUT32: int32 results (as the reference keeps them) or clipped int8.  A padding wave (member index past the end)
// recomputes the last member and stores the same values to the same rows again.
// FUSE: (acc + (sb*a >> sigma)) >> shift evaluated as ((acc << sigma) + sb*a) >> (sigma + shift), the same value
// with one instruction less; the host selects it only when the sum cannot leave 32 bits.
template <bool FUSE>
__device__ __forceinline__ int perturbed(int acc, int sb, int a, int sigma, int shift) {
    if (FUSE) return (int)(((unsigned)acc << sigma) + (unsigned)mul24(sb, a)) >> (sigma + shift);
    return (acc + (mul24(sb, a) >> sigma)) >> shift;
}

template <int K, int N, bool OUT32, bool FUSE>
__global__ void __launch_bounds__(EGG_THREADS, 2) k_plinear(PlinParams p) {
    typedef Plin<K, N> P;
    typedef DmaPlan<P::PR, P::B> Plan;
    constexpr int KS = P::KS, NTB = P::NTB, B = P::B;
    constexpr int STORES = (!OUT32 && B == 128) ? 4 : 4 * NTB;   // global stores of one column block's results, per wave
    constexpr int XLOADS = P::PREFETCH_X ? KS : 0;                // row loads issued at the start of a token tile
    extern __shared__ __align__(16) int8_t smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    int8_t *tb = smem + P::NBUF * P::UNIT + wave * P::PER_WAVE;
    int *At = reinterpret_cast<int *>(tb);
    int8_t *Bt = reinterpret_cast<int8_t *>(At + N);
    // transpose tile of this wave: row r (token) holds eight 16-byte chunks, chunk c kept at position c ^ (r & 7) so
    // that both the writes (lane = row) and the reads (eight lanes = one row) are free of bank conflicts
    int8_t *stage = smem + P::NBUF * P::UNIT + EGG_WAVES * P::PER_WAVE + wave * P::STAGE;
    const int rr = lane >> 3, rc = lane & 7;       // read side: row within a group of eight, chunk

    int member = blockIdx.x * EGG_WAVES + wave;
    if (member >= p.members) member = p.members - 1;
    int32_t *y32 = p.Y32; int8_t *y8 = p.Y8;
    // reference indexing: a pair shares one draw, the odd member takes it negated (mgpu.cu:864-871); own_noise: every
    // member its own draw, applied with ns = +1
    const int ns = (!p.own_noise && (member & 1)) ? -1 : 1;
    const uint32_t ps = p.seed + (uint32_t)(p.own_noise ? member : member / 2);

    // the W stream: unit u of a token tile (every tile walks the same UPP units), fragment-major blocks of B x B
    const Plan plan = dma_plan<P::PR, P::B>(B);
    auto unit_src = [&](int u) {
        const int nb = u / P::UNITS_NB, r = u % P::UNITS_NB, kb = r / P::UPB, h = r % P::UPB;
        return p.Wfrag + ((size_t)kb * P::NBLK + nb) * (B * B) + (size_t)h * P::UNIT;
    };
    const int passes = p.T / 32;
    const int total_units = passes * P::UPP;       // uniform over the workgroup
    int issued = 0;                                // units requested so far
    auto request = [&]() {
        if (issued < total_units) {
            dma_unit<P::PR, P::B>(smem + (issued % P::NBUF) * P::UNIT, unit_src(issued % P::UPP), plan);
            issued++;
        }
    };
    for (int i = 0; i < P::AHEAD; i++) request();
    if (!p.plain) {
        fill_noise_i32(At, ps + p.off_a, N, p.mask, ns, lane);
        fill_noise_i8(Bt, ps + p.off_b, K, p.mask, lane);
    }
    __syncthreads();

    int used = 0;                                  // units consumed so far
    v4i xop[KS], xnext[P::PREFETCH_X ? KS : 1];
    {
        const size_t row0 = (size_t)member * p.T + j;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            v4i v = load_op(p.X + row0 * K, ks, g);
            if (P::PREFETCH_X) xnext[P::PREFETCH_X ? ks : 0] = v; else xop[ks] = v;
        }
    }
    // nothing pending when the tile loop is entered: the compiler's wait for the row loads inside the loop then only
    // has to cover the loads of the previous iteration, which are a whole tile old
    __builtin_amdgcn_s_waitcnt(0x0F70);
    for (int pass = 0; pass < passes; pass++) {
        const size_t row = (size_t)member * p.T + pass * 32 + j;
        const bool prefetch = P::PREFETCH_X && pass + 1 < passes;
        if (P::PREFETCH_X) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) xop[ks] = xnext[P::PREFETCH_X ? ks : 0];
        }
        if (prefetch) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) xnext[P::PREFETCH_X ? ks : 0] = load_op(p.X + (row + 32) * K, ks, g);
        }
        const int sb = p.plain ? 0 : dot_noise<KS, true>(xop, Bt, 0, g);
#pragma unroll 1
        for (int nb = 0; nb < P::NBLK; nb++) {
            v16i acc[NTB];
            zero_acc<NTB>(acc);
            v4i frag[2][NTB], xlast = xop[0];
#pragma unroll
            for (int r = 0; r < P::UNITS_NB; r++) {
                // Unit `used` must have landed.  It was requested two iterations ago; what this wave issued since then
                // may stay in flight: the next unit, and, when one of those two iterations ended a column block, that
                // block's result stores and (at the start of a token tile) the row loads for the next tile.  The first
                // tile counts none of them.
                const int later = issued - used - 1;              // 0 or 1
                const bool after_block = r == 0 || (r == 1 && P::UNITS_NB >= 2);
                if (after_block && nb > 0) wait_unit<Plan::PER, STORES>(later);
                else if (after_block && pass > 0) {
                    if (prefetch) wait_unit<Plan::PER, STORES + XLOADS>(later);
                    else wait_unit<Plan::PER, STORES>(later);
                } else wait_unit<Plan::PER, 0>(later);
                __syncthreads();                 // also: every wave is done with the buffer the next request overwrites
                request();
                const int8_t *cur = smem + (used % P::NBUF) * P::UNIT;
                used++;
                // fragments are read one k-step ahead of the MFMAs that use them; the last k-step of a unit is
                // multiplied after the next unit's barrier, behind that unit's first fragment reads
                const v4i *xu = xop + (r / P::UPB) * (B / 32) + (r % P::UPB) * P::KSU;
#pragma unroll
                for (int ks = 0; ks < P::KSU; ks++) {
                    constexpr int dummy = 0; (void)dummy;
                    const int slot = (r * P::KSU + ks) & 1;
#pragma unroll
                    for (int nt = 0; nt < NTB; nt++)
                        frag[slot][nt] = *reinterpret_cast<const v4i *>(cur + ((size_t)(ks * 2 + g) * B + nt * 32 + j) * 16);
                    __builtin_amdgcn_sched_barrier(0);
                    if (r > 0 || ks > 0) {
                        const v4i xprev = (ks > 0) ? xu[ks - 1] : xlast;
#pragma unroll
                        for (int nt = 0; nt < NTB; nt++)
                            acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[slot ^ 1][nt], xprev, acc[nt], 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                xlast = xu[P::KSU - 1];
            }
            {
                constexpr int slot = (P::UNITS_NB * P::KSU - 1) & 1;
#pragma unroll
                for (int nt = 0; nt < NTB; nt++)
                    acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[slot][nt], xlast, acc[nt], 0, 0, 0);
            }
            const size_t row_base = (size_t)member * p.T + pass * 32;
            // PLAIN: acc >> shift without the rank-1 term (a wave-uniform choice made once per column block)
            auto finish_block = [&](auto plain_tag) {
            constexpr bool PLAIN = decltype(plain_tag)::value;
            auto fin = [&](int a, int an) { return PLAIN ? (a >> p.shift) : perturbed<FUSE>(a, sb, an, p.sigma, p.shift); };
            if (OUT32) {
                // one 32 x 32 int32 tile (128 bytes per row) at a time
#pragma unroll
                for (int nt = 0; nt < NTB; nt++) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        int n0 = nb * B + 32 * nt + 8 * q + 4 * g;
                        v4i a4 = {0, 0, 0, 0}; if (!PLAIN) a4 = *reinterpret_cast<const v4i *>(At + n0);
                        v4i o4;
#pragma unroll
                        for (int e = 0; e < 4; e++) o4[e] = fin(acc[nt][4 * q + e], a4[e]);
                        *reinterpret_cast<v4i *>(stage + j * 128 + (((2 * q + g) ^ (j & 7)) * 16)) = o4;
                    }
                    wave_lds_fence();
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int r = rr + 8 * i;
                        v4i v = *reinterpret_cast<const v4i *>(stage + r * 128 + ((rc ^ (r & 7)) * 16));
                        *reinterpret_cast<v4i *>(y32 + (row_base + r) * N + nb * B + 32 * nt + 4 * rc) = v;
                    }
                    wave_lds_fence();
                }
            } else if (B == 128) {
                // the block's 128 int8 columns of a row are one 128-byte line
#pragma unroll
                for (int nt = 0; nt < NTB; nt++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        int n0 = nb * B + 32 * nt + 8 * q + 4 * g;
                        v4i a4 = {0, 0, 0, 0}; if (!PLAIN) a4 = *reinterpret_cast<const v4i *>(At + n0);
                        int o[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) o[e] = clip127(fin(acc[nt][4 * q + e], a4[e]));
                        const int col = 32 * nt + 8 * q + 4 * g;                 // byte column inside the 128-byte row
                        *reinterpret_cast<int *>(stage + j * 128 + (((col >> 4) ^ (j & 7)) * 16) + (col & 15)) = pack4(o[0], o[1], o[2], o[3]);
                    }
                wave_lds_fence();
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = rr + 8 * i;
                    v4i v = *reinterpret_cast<const v4i *>(stage + r * 128 + ((rc ^ (r & 7)) * 16));
                    *reinterpret_cast<v4i *>(y8 + (row_base + r) * N + nb * B + 16 * rc) = v;
                }
                wave_lds_fence();
            } else {
#pragma unroll
                for (int nt = 0; nt < NTB; nt++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        int n0 = nb * B + 32 * nt + 8 * q + 4 * g;
                        v4i a4 = {0, 0, 0, 0}; if (!PLAIN) a4 = *reinterpret_cast<const v4i *>(At + n0);
                        int o[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) o[e] = clip127(fin(acc[nt][4 * q + e], a4[e]));
                        *reinterpret_cast<int *>(y8 + row * N + n0) = pack4(o[0], o[1], o[2], o[3]);
                    }
            }
            };
            if (p.plain) finish_block(std::true_type{}); else finish_block(std::false_type{});
        }
        if (!P::PREFETCH_X && pass + 1 < passes) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) xop[ks] = load_op(p.X + (row + 32) * K, ks, g);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Two token tiles per wave.  In k_plinear every W fragment a wave reads from LDS (1 KB) feeds one MFMA; four SIMDs
// issuing one v_mfma_i32_32x32x32_i8 per 32 clocks then ask the LDS for its whole 128 bytes per clock, so the matrix
// pipe cannot run much above half rate.  Here a wave holds the rows of 64 tokens (two tiles) and multiplies every
// fragment with both, which halves the LDS traffic per MFMA.  To keep two workgroups per CU (256 registers per wave)
// next to the 2 * K / 8 operand registers, a column block is 64 wide (two accumulators per tile).  W is laid out for
// exactly this walk: [column block of 64][k-step][half g][column][16 k-bytes], so the units of a token tile are one
// contiguous stream.  Used for K = 256 and 512 when T is a multiple of 64; N is a run-time multiple of 64.
template <int K>
struct Plin2 {
    static constexpr int BN = 64, NTB = 2, TT = 2, KS = K / 32;
    static constexpr int KSU = KS < 8 ? KS : 8;                  // k-steps per unit
    static constexpr int UNITS_NB = KS / KSU;                    // units per column block
    static constexpr int UNIT = KSU * 2 * BN * 16;               // at most 16 KB
    static constexpr int NBUF = 3, AHEAD = 2;
    static constexpr int STAGE = TT * 32 * BN;                   // 4 KB: two int8 tiles, or one 32 x 32 int32 tile
    static int per_wave(int N) { return N * 4 + K; }
    static size_t total(int N) { return (size_t)NBUF * UNIT + EGG_WAVES * (size_t)(per_wave(N) + STAGE); }
};

__global__ void k_swizzle_cols64(const uint32_t *src, v4i *dst, int K, int N) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= K * N / 16) return;
    const int per_block = K / 16 * 64;
    const int nb = c / per_block, idx = c % per_block, pr = idx / 64, n = idx % 64;     // pr = 2 * k-step + g
    v4i v;
#pragma unroll
    for (int q = 0; q < 4; q++) v[q] = (int)src[(size_t)(4 * pr + q) * N + nb * 64 + n];
    dst[c] = v;
}

template <int K, bool OUT32, bool FUSE>
__global__ void __launch_bounds__(EGG_THREADS, 2) k_plinear2(PlinParams p) {
    typedef Plin2<K> P;
    typedef DmaPlan<2 * P::KSU, P::BN> Plan;
    constexpr int KS = P::KS, NTB = P::NTB, BN = P::BN, TT = P::TT;
    constexpr int STORES = OUT32 ? TT * NTB * 4 : TT * 2;        // global stores of one column block's results, per wave
    extern __shared__ __align__(16) int8_t smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const int N = p.N, nblk = N / BN;
    int8_t *tb = smem + P::NBUF * P::UNIT + wave * (N * 4 + K);
    int *At = reinterpret_cast<int *>(tb);
    int8_t *Bt = reinterpret_cast<int8_t *>(At + N);
    int8_t *stage = smem + P::NBUF * P::UNIT + EGG_WAVES * (N * 4 + K) + wave * P::STAGE;

    int member = blockIdx.x * EGG_WAVES + wave;
    if (member >= p.members) member = p.members - 1;
    // reference indexing: a pair shares one draw, the odd member takes it negated (mgpu.cu:864-871); own_noise: every
    // member its own draw, applied with ns = +1
    const int ns = (!p.own_noise && (member & 1)) ? -1 : 1;
    const uint32_t ps = p.seed + (uint32_t)(p.own_noise ? member : member / 2);

    const Plan plan = dma_plan<2 * P::KSU, P::BN>(BN);
    const int passes = p.T / 64, upp = nblk * P::UNITS_NB;      // units per pass: the whole of W, in stream order
    const int total_units = passes * upp;
    int issued = 0, next_u = 0;
    auto request = [&]() {
        if (issued < total_units) {
            dma_unit<2 * P::KSU, P::BN>(smem + (issued % P::NBUF) * P::UNIT, p.Wfrag + (size_t)next_u * P::UNIT, plan);
            issued++; next_u = next_u + 1 == upp ? 0 : next_u + 1;
        }
    };
    for (int i = 0; i < P::AHEAD; i++) request();
    if (!p.plain) {
        fill_noise_i32(At, ps + p.off_a, N, p.mask, ns, lane);
        fill_noise_i8(Bt, ps + p.off_b, K, p.mask, lane);
    }
    __syncthreads();

    int used = 0;
    v4i xop[TT][KS];
    auto load_rows = [&](int pass) {
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const int8_t *xr = p.X + ((size_t)member * p.T + pass * 64 + t * 32 + j) * K;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) xop[t][ks] = load_op(xr, ks, g);
        }
    };
    load_rows(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);            // nothing pending when the tile loop is entered
    for (int pass = 0; pass < passes; pass++) {
        int sb[TT];
#pragma unroll
        for (int t = 0; t < TT; t++) sb[t] = p.plain ? 0 : dot_noise<KS, true>(xop[t], Bt, 0, g);
#pragma unroll 1
        for (int nb = 0; nb < nblk; nb++) {
            v16i acc[TT][NTB];
#pragma unroll
            for (int t = 0; t < TT; t++) zero_acc<NTB>(acc[t]);
#pragma unroll
            for (int r = 0; r < P::UNITS_NB; r++) {
                // Unit `used` was requested two iterations ago.  What this wave issued after it may stay in flight: the
                // next unit and, once a column block has been finished, that block's result stores (the row loads of
                // the next token pair are not counted, which only makes the wait stricter; an overcount would let the
                // unit itself stay in flight).
                const int later = issued - used - 1;              // 0 or 1
                __builtin_amdgcn_sched_barrier(0);               // the counts rely on the program order of loads and stores
                if (r <= 1 && (nb > 0 || pass > 0)) wait_unit<Plan::PER, STORES>(later);
                else wait_unit<Plan::PER, 0>(later);
                __syncthreads();                 // also: every wave is done with the buffer the next request overwrites
                request();
                const int8_t *cur = smem + (used % P::NBUF) * P::UNIT;
                used++;
                v4i frag[2][NTB];
#pragma unroll
                for (int nt = 0; nt < NTB; nt++)
                    frag[0][nt] = *reinterpret_cast<const v4i *>(cur + ((size_t)g * BN + nt * 32 + j) * 16);
#pragma unroll
                for (int ks = 0; ks < P::KSU; ks++) {
                    const int slot = ks & 1;
                    if (ks + 1 < P::KSU) {
#pragma unroll
                        for (int nt = 0; nt < NTB; nt++)
                            frag[slot ^ 1][nt] = *reinterpret_cast<const v4i *>(cur + ((size_t)((ks + 1) * 2 + g) * BN + nt * 32 + j) * 16);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int nt = 0; nt < NTB; nt++)
#pragma unroll
                        for (int t = 0; t < TT; t++) {
                            acc[t][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[slot][nt], xop[t][r * P::KSU + ks], acc[t][nt], 0, 0, 0);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            const size_t row_base = (size_t)member * p.T + pass * 64;
            // after the last column block the operand registers are free: request the next pair's rows before the
            // epilogue so that they travel while it runs (reloading each k-step's rows in place as soon as it is
            // multiplied, a block earlier, costs 30-40 spilled registers and measured 8 % slower)
            if (nb == nblk - 1 && pass + 1 < passes) load_rows(pass + 1);
            auto finish_block = [&](auto plain_tag) {
                constexpr bool PLAIN = decltype(plain_tag)::value;
                if (OUT32) {
                    const int rr = lane >> 3, rc = lane & 7;
#pragma unroll
                    for (int t = 0; t < TT; t++)
#pragma unroll
                    for (int nt = 0; nt < NTB; nt++) {
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            const int n0 = nb * BN + 32 * nt + 8 * q + 4 * g;
                            v4i a4 = {0, 0, 0, 0}; if (!PLAIN) a4 = *reinterpret_cast<const v4i *>(At + n0);
                            v4i o4;
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                o4[e] = PLAIN ? (acc[t][nt][4 * q + e] >> p.shift) : perturbed<FUSE>(acc[t][nt][4 * q + e], sb[t], a4[e], p.sigma, p.shift);
                            *reinterpret_cast<v4i *>(stage + j * 128 + (((2 * q + g) ^ (j & 7)) * 16)) = o4;
                        }
                        wave_lds_fence();
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int r = rr + 8 * i;
                            v4i v = *reinterpret_cast<const v4i *>(stage + r * 128 + ((rc ^ (r & 7)) * 16));
                            *reinterpret_cast<v4i *>(p.Y32 + (row_base + 32 * t + r) * N + nb * BN + 32 * nt + 4 * rc) = v;
                        }
                        wave_lds_fence();
                    }
                } else {
                    // a row's 64 result bytes are four 16-byte chunks; rows 2i and 2i+1 share one 128-byte LDS line and
                    // chunk c of row r sits at position c ^ ((r >> 1) & 3) of its half, so eight lanes read one line
#pragma unroll
                    for (int t = 0; t < TT; t++)
#pragma unroll
                        for (int nt = 0; nt < NTB; nt++)
#pragma unroll
                            for (int q = 0; q < 4; q++) {
                                const int col = 32 * nt + 8 * q + 4 * g;
                                v4i a4 = {0, 0, 0, 0}; if (!PLAIN) a4 = *reinterpret_cast<const v4i *>(At + nb * BN + col);
                                int o[4];
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    o[e] = clip127(PLAIN ? (acc[t][nt][4 * q + e] >> p.shift) : perturbed<FUSE>(acc[t][nt][4 * q + e], sb[t], a4[e], p.sigma, p.shift));
                                *reinterpret_cast<int *>(stage + t * 2048 + (j >> 1) * 128 + (j & 1) * 64 + (((col >> 4) ^ ((j >> 1) & 3)) * 16) + (col & 15)) = pack4(o[0], o[1], o[2], o[3]);
                            }
                    wave_lds_fence();
                    const int rr = lane >> 2, rc = lane & 3;
#pragma unroll
                    for (int i = 0; i < TT * 2; i++) {
                        const int r = rr + 16 * i;             // row within the wave's 64 tokens
                        const int rl = r & 31;
                        v4i v = *reinterpret_cast<const v4i *>(stage + (r >> 5) * 2048 + (rl >> 1) * 128 + (rl & 1) * 64 + ((rc ^ ((rl >> 1) & 3)) * 16));
                        *reinterpret_cast<v4i *>(p.Y8 + (row_base + r) * N + nb * BN + 16 * rc) = v;
                    }
                    wave_lds_fence();
                }
            };
            if (p.plain) finish_block(std::true_type{}); else finish_block(std::false_type{});
        }
    }
}

template <int K, bool OUT32, bool FUSE>
static hipError_t launch_two(const PlinParams &p, hipStream_t s) {
    dim3 grid((p.members + EGG_WAVES - 1) / EGG_WAVES), block(EGG_THREADS);
    const size_t lds = Plin2<K>::total(p.N);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_plinear2<K, OUT32, FUSE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((k_plinear2<K, OUT32, FUSE>), grid, block, lds, s, p);
    return hipGetLastError();
}

template <int K, int N, bool OUT32, bool FUSE>
static hipError_t launch_one(const PlinParams &p, hipStream_t s) {
    dim3 grid((p.members + EGG_WAVES - 1) / EGG_WAVES), block(EGG_THREADS);
    const size_t lds = Plin<K, N>::TOTAL;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_plinear<K, N, OUT32, FUSE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((k_plinear<K, N, OUT32, FUSE>), grid, block, lds, s, p);
    return hipGetLastError();
}

template <int K, int N>
static hipError_t launch_kn(const PlinParams &p, hipStream_t s) {
    // the fused form needs |acc| * 2^sigma + |sb * a| < 2^31 for any int8 inputs: |acc| <= K * 128 * 128,
    // |sb| <= K * 128 * mask, |a| <= mask
    const long long mag = egg_noise_magnitude(p.mask);
    const long long bound = ((long long)K * 128 * 128 << p.sigma) + (long long)K * 128 * mag * mag;
    const bool fuse = p.sigma >= 0 && p.sigma <= 12 && p.sigma + p.shift < 32 && bound < (1LL << 31);
    // both outputs requested: two launches (the test hook asks for one at a time)
    hipError_t e = hipSuccess;
    if (p.Y32) e = fuse ? launch_one<K, N, true, true>(p, s) : launch_one<K, N, true, false>(p, s);
    if (e == hipSuccess && p.Y8) e = fuse ? launch_one<K, N, false, true>(p, s) : launch_one<K, N, false, false>(p, s);
    return e;
}

int egg_plinear_block(int K, int N) { int m = K < N ? K : N; return m < 128 ? m : 128; }

static bool one_tile_case(int K, int N) {
#define CASE(K_, N_) if (K == K_ && N == N_) return true;
    CASE(64, 64) CASE(64, 256) CASE(256, 64) CASE(128, 128) CASE(128, 512) CASE(512, 128)
    CASE(256, 256) CASE(256, 1024) CASE(1024, 256) CASE(512, 512)
#undef CASE
    return false;
}

// the two-tile kernel serves K = 256 / 512 with whole pairs of token tiles: whenever its tables fit next to a second
// workgroup's on the CU, and alone on the CU for the wide outputs the one-tile kernel has no instance for
static bool two_tile_shape(int T, int K, int N) {
    if (T % 64 || N % 64 || N < 64 || (K != 256 && K != 512)) return false;
    const size_t lds = K == 256 ? Plin2<256>::total(N) : Plin2<512>::total(N);
    return 2 * lds <= 160 * 1024 || (lds <= 160 * 1024 && !one_tile_case(K, N));
}

template <int K>
static hipError_t launch_two_k(const PlinParams &p, hipStream_t s) {
    const long long mag = egg_noise_magnitude(p.mask);
    const long long bound = ((long long)K * 128 * 128 << p.sigma) + (long long)K * 128 * mag * mag;
    const bool fuse = p.sigma >= 0 && p.sigma <= 12 && p.sigma + p.shift < 32 && bound < (1LL << 31);
    hipError_t e = hipSuccess;
    if (p.Y32) e = fuse ? launch_two<K, true, true>(p, s) : launch_two<K, true, false>(p, s);
    if (e == hipSuccess && p.Y8) e = fuse ? launch_two<K, false, true>(p, s) : launch_two<K, false, false>(p, s);
    return e;
}

hipError_t egg_launch_plinear_swizzle(const int8_t *W, int8_t *Wf, int T, int K, int N, hipStream_t s) {
    if (two_tile_shape(T, K, N)) {
        const int chunks = K * N / 16;
        hipLaunchKernelGGL(k_swizzle_cols64, dim3((chunks + 255) / 256), dim3(256), 0, s, reinterpret_cast<const uint32_t *>(W),
                           reinterpret_cast<v4i *>(Wf), K, N);
        return hipGetLastError();
    }
    const int PB = egg_plinear_block(K, N);
    if (K % PB || N % PB) return hipErrorInvalidValue;
    return egg_launch_swizzle(W, Wf, K, N, PB, 1, s);
}

hipError_t egg_launch_plinear(const PlinParams &p, hipStream_t s) {
    if (p.T % 32 || p.T < 32 || p.members < 1) return hipErrorInvalidValue;
    if (p.Wblocked && egg_plinear_ws_shape(p.K, p.N)) return egg_launch_plinear_ws(p, s);
    if (two_tile_shape(p.T, p.K, p.N)) return p.K == 256 ? launch_two_k<256>(p, s) : launch_two_k<512>(p, s);
#define CASE(K_, N_) if (p.K == K_ && p.N == N_) return launch_kn<K_, N_>(p, s);
    CASE(64, 64) CASE(64, 256) CASE(256, 64) CASE(128, 128) CASE(128, 512) CASE(512, 128)
    CASE(256, 256) CASE(256, 1024) CASE(1024, 256) CASE(512, 512)
#undef CASE
    return hipErrorInvalidValue;
}
