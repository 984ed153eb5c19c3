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
#include "egg_params.h"

// The float steps of the normalisations are single IEEE operations in the reference; a fused multiply-add in
// round_half_away(val * scale) changes results at exact .5 ties (e.g. max 6, value 3).  The build also passes
// -ffp-contract=off; this keeps the header right under any flags.
#pragma clang fp contract(off)

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
// `mask` is the magnitude mask (DEVICE_MASK) in its low byte; EGG_NOISE_GAUSSIAN (egg_params.h) on top of it selects the reference's
// DEVICE_GAUSSIAN form, the sum of three such fields taken from bits 0-5, 5-10 and 10-15 of the hash
__device__ __forceinline__ int noise_from_hash(uint32_t s, uint32_t idx, int mask) {
    uint32_t r = hash_rng(s, idx);
    const uint32_t m = (uint32_t)mask & 0xffu;
    int mag = (int)((r >> 1) & m);
    int n = (r & 1) ? mag : -mag;
    if (mask & EGG_NOISE_GAUSSIAN) {
        mag = (int)((r >> 6) & m); n += (r & 32) ? mag : -mag;
        mag = (int)((r >> 11) & m); n += (r & 1024) ? mag : -mag;
    }
    return n;
}

__device__ __forceinline__ int clip127(int a) { return min(127, max(-127, a)); }

// ---------------------------------------------------------------- lane helpers
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
// value held by the same token's lane in the other half
// A token's values sit in two lanes, 32 apart.  v_permlane32_swap on two copies of a register gives every lane the
// value of the lower half's lane (first result) and of the upper half's lane (second result): a reduction over the
// two halves is one swap and one operation, without the LDS crossbar or a lane index.
__device__ __forceinline__ int sum_halves(int v) {
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
    return (int)(r[0] + r[1]);
}
__device__ __forceinline__ int max_halves(int v) {
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
    return max((int)r[0], (int)r[1]);
}
__device__ __forceinline__ long long sum_halves64(long long v) {
    const auto lo = __builtin_amdgcn_permlane32_swap((unsigned)(v & 0xffffffffll), (unsigned)(v & 0xffffffffll), false, false);
    const auto hi = __builtin_amdgcn_permlane32_swap((unsigned)(v >> 32), (unsigned)(v >> 32), false, false);
    return (long long)(((unsigned long long)hi[0] << 32) | lo[0]) + (long long)(((unsigned long long)hi[1] << 32) | lo[1]);
}
// hidden index of accumulator register r of column group nt for lane half g
__device__ __forceinline__ int col_of(int nt, int r, int g) { return nt * 32 + ((r >> 2) << 3) + (g << 2) + (r & 3); }

__device__ __forceinline__ int sx8(int packed, int e) { return (int)(int8_t)(packed >> (8 * e)); }
// bytes 0 of four values side by side: two byte permutes and an or
__device__ __forceinline__ int pack4(int a, int b, int c, int d) {
    return (int)(__builtin_amdgcn_perm((unsigned)b, (unsigned)a, 0x0c0c0400u) | __builtin_amdgcn_perm((unsigned)d, (unsigned)c, 0x04000c0cu));
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
// x ^ 0x80 is x + 128 as an unsigned byte, so the byte-wise |(x + 128) - 128| of v_sad_u8 is |x|
__device__ __forceinline__ int sumabs4(int a, int c) {
    return (int)__builtin_amdgcn_sad_u8((unsigned)a ^ 0x80808080u, 0x80808080u, (unsigned)c);
}

// full-rate 24-bit multiply (both operands must fit in 24 signed bits, the product in 32)
__device__ __forceinline__ int mul24(int a, int b) { return __mul24(a, b); }

// C truncating division a / d for |a| <= 40000 and d in [1,127], with rcp = 1.0f / (float)d:
// trunc((a + copysign(0.5, a)) * rcp).  a/d is a multiple of 1/d, so (a +- 0.5)/d stays at least 0.5/d away
// from the next integer while the float error is below 0.007/d; checked exhaustively on the CPU.
__device__ __forceinline__ int div_trunc(int a, float rcp) {
    float af = (float)a;
    return (int)((af + __builtin_copysignf(0.5f, af)) * rcp);
}
// (int)roundf(x) (half away from zero) for |x| <= 4096: trunc(x + copysign(0.5 - 2^-25, x)); checked
// exhaustively on the CPU against roundf for every float in that range.
__device__ __forceinline__ int round_half_away(float x) {
    return (int)(x + __builtin_copysignf(0x1.fffffep-2f, x));
}

// ---------------------------------------------------------------- W block staging
// Weights are consumed from a "fragment-major" copy of each matrix (built by k_swizzle whenever the canonical
// blocked weights change): the matrix is cut into B x B blocks, B = min(hidden, 256); block (kb, nb) is stored
// contiguously at ((kb * (N/B)) + nb) * B*B as [B/16][B][16 bytes], where entry (p = 2*ks + g, n) holds the
// 16 k-bytes lane half g consumes in k-step ks for output column n: canonical dwords kq = 8ks + 2q + g (slot
// order) or 8ks + 4g + q (natural order), q = 0..3.  A block is therefore exactly its LDS image and staging
// is a straight 16-byte-per-lane copy with every load in flight before the first LDS write.
// A block is streamed in units of UK = min(B,128) k-rows (a contiguous slice of the block) through two LDS
// buffers with global_load_lds_dwordx4 (global -> LDS without passing through registers): while the waves run the
// MFMAs of unit i, the copy of unit i+1 is in flight.  One barrier per unit: it proves both that unit i has landed
// for every wave and that every wave is done with the buffer unit i+1 is about to overwrite.
template <int B>
struct WUnit {
    static constexpr int UK = B < 128 ? B : 128;
    static constexpr int BYTES = UK * B;
    static constexpr int PER_BLOCK = B / UK;
};
struct WStream {
    int8_t *fill;          // buffer the next prefetch writes
    int8_t *other;
};
__device__ __forceinline__ void wstream_init(WStream &s, int8_t *lds, int unit_bytes) { s.fill = lds; s.other = lds + unit_bytes; }

template <int B>
__device__ __forceinline__ void w_prefetch(WStream &s, const int8_t *unit);      // defined with the copy plans below

// wait for the unit prefetched last, make it visible to the workgroup, and hand it out
__device__ __forceinline__ const int8_t *w_acquire(WStream &s) {
    // s_waitcnt vmcnt(0) through the builtin (0x0F70 = vmcnt 0, expcnt/lgkmcnt untouched on gfx9) so that the compiler's
    // own counter bookkeeping sees it: it then knows none of its loads or stores is pending and does not add
    // vmcnt waits inside the phase, which would also wait for the copy issued right after this call
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    int8_t *p = s.fill;
    s.fill = s.other; s.other = p;
    return p;
}
template <int B>
__device__ __forceinline__ const int8_t *w_unit_ptr(const int8_t *Wf, int n_total, int k_off, int n_off, int unit) {
    const int kb = unit / WUnit<B>::PER_BLOCK, h = unit % WUnit<B>::PER_BLOCK;
    return Wf + ((size_t)(k_off / B + kb) * (n_total / B) + n_off / B) * (B * B) + (size_t)h * WUnit<B>::BYTES;
}

// acc[nt] += W_unit^T . xop for one staged unit; xop[ks] is the token operand of k-step ks of the unit.  The
// fragments of one k-step (at most 8) are read before its MFMAs so that one LDS latency is exposed per k-step.
template <int B>
__device__ __forceinline__ void mfma_unit(v16i *acc, const v4i *xop, const int8_t *lds, int lane) {
    const int i = lane & 31, g = lane >> 5;
    constexpr int NT = B / 32;
#pragma unroll
    for (int ks = 0; ks < WUnit<B>::UK / 32; ks++) {
        v4i a[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) a[nt] = *reinterpret_cast<const v4i *>(lds + ((size_t)(ks * 2 + g) * B + nt * 32 + i) * 16);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int nt = 0; nt < NT; nt++) acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[nt], xop[ks], acc[nt], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
    }
}

// Full GEMM for one tile: acc[NOUT/32] (+)= W[k_off.., n_off..]^T . xop[KTOT/32].  The first unit must already
// have been prefetched; `next` is the first unit of whatever GEMM follows (nullptr if none) and is prefetched while
// the last unit is consumed.  Every wave of the workgroup must call it (it synchronises).
template <int KTOT, int NOUT, int B>
__device__ __forceinline__ void gemm_stream(v16i *acc, const v4i *xop, const int8_t *Wf, int n_total,
                                            int k_off, int n_off, WStream &ws, const int8_t *next, int lane) {
    static_assert(KTOT % B == 0 && NOUT % B == 0, "block size must divide the GEMM");
    constexpr int UPB = WUnit<B>::PER_BLOCK, KU = (KTOT / B) * UPB;
#pragma unroll
    for (int nb = 0; nb < NOUT / B; nb++) {
#pragma unroll
        for (int u = 0; u < KU; u++) {
            const int8_t *cur = w_acquire(ws);
            const int8_t *nx = (u + 1 < KU) ? w_unit_ptr<B>(Wf, n_total, k_off, n_off + nb * B, u + 1)
                             : ((nb + 1 < NOUT / B) ? w_unit_ptr<B>(Wf, n_total, k_off, n_off + (nb + 1) * B, 0) : next);
            w_prefetch<B>(ws, nx);
            mfma_unit<B>(acc + nb * (B / 32), xop + u * (WUnit<B>::UK / 32), cur, lane);
        }
    }
}

// ---- units for the forward kernels: NP p-rows (p = 2*kstep + half) x COLS output columns of a fragment-major block
// whose rows hold src_cols columns.  LDS image: [NP][COLS][16 bytes], so 64-column segment number id (= pr * COLS/64
// + seg) lands at LDS byte id * 1024.  Wave w copies the PER consecutive segments w*PER .. w*PER + PER - 1 with one
// M0 / one SGPR base and the instruction offsets 0, 1024, ...; because that offset is added to the global address as
// well, each segment's per-lane global offset is precomputed once (DmaPlan) with the instruction offset taken out.
// Per unit this costs a handful of scalar instructions instead of a 64-bit address computation per segment.
template <int NP, int COLS>
struct DmaPlan {
    static_assert(COLS % 64 == 0, "a wave instruction copies 64 columns");
    static constexpr int SEG = COLS / 64, INSTR = NP * SEG, PER = INSTR / EGG_WAVES;
    static_assert(INSTR % EGG_WAVES == 0 && (PER == 1 || PER == 2 || PER == 4), "unit must split evenly over the waves");
    uint32_t voff[PER];      // lane * 16 + global byte offset of segment k of this wave - k * 1024
    uint32_t lds_off;        // first LDS byte of this wave inside the unit
};
template <int NP, int COLS>
__device__ __forceinline__ DmaPlan<NP, COLS> dma_plan(int src_cols) {
    typedef DmaPlan<NP, COLS> P;
    P pl;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane16 = (threadIdx.x & 63u) * 16u;
#pragma unroll
    for (int k = 0; k < P::PER; k++) {
        const int id = wave * P::PER + k, pr = id / P::SEG, seg = id % P::SEG;
        pl.voff[k] = lane16 + (uint32_t)(pr * src_cols + seg * 64) * 16u - (uint32_t)k * 1024u;
    }
    pl.lds_off = (uint32_t)wave * P::PER * 1024u;
    return pl;
}
// Start the copy of one unit to lds_dst (global -> LDS without passing through registers; lane l of segment k moves
// 16 bytes).  Written as inline assembly on purpose: for the compiler's own LDS-DMA intrinsic every later LDS read may
// alias the destination, so it waits for the copy (s_waitcnt vmcnt(0)) before the next table or fragment read and the
// copy no longer overlaps anything.  Here the ordering is explicit instead: w_acquire waits for vmcnt(0) and then
// barriers before anyone reads a unit, and a buffer is only overwritten after the barrier that follows its last
// reader.  src and lds_dst must be wave-uniform.
template <int NP, int COLS>
__device__ __forceinline__ void dma_unit(const int8_t *lds_dst, const int8_t *src, const DmaPlan<NP, COLS> &pl) {
    typedef DmaPlan<NP, COLS> P;
    const uint32_t m0v = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(size_t)(const __attribute__((address_space(3))) int8_t *)lds_dst) + pl.lds_off;
    const uint64_t b = (uint64_t)src;
    // readfirstlane returns a signed int: go through uint32_t so the low half is not sign-extended over the high half
    const uint32_t blo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b), bhi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    const uint64_t sb = ((uint64_t)bhi << 32) | blo;
    if (P::PER == 1)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     : : "s"(m0v), "v"(pl.voff[0]), "s"(sb) : "memory", "m0");
    else if (P::PER == 2)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %3\n\tglobal_load_lds_dwordx4 %2, %3 offset:1024"
                     : : "s"(m0v), "v"(pl.voff[0]), "v"(pl.voff[P::PER > 1 ? 1 : 0]), "s"(sb) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %5\n\tglobal_load_lds_dwordx4 %2, %5 offset:1024\n\t"
                     "global_load_lds_dwordx4 %3, %5 offset:2048\n\tglobal_load_lds_dwordx4 %4, %5 offset:3072"
                     : : "s"(m0v), "v"(pl.voff[0]), "v"(pl.voff[P::PER > 1 ? 1 : 0]), "v"(pl.voff[P::PER > 2 ? 2 : 0]),
                         "v"(pl.voff[P::PER > 3 ? 3 : 0]), "s"(sb) : "memory", "m0");
}
template <int NP, int COLS>
__device__ __forceinline__ void w_prefetch2(WStream &s, const int8_t *src, const DmaPlan<NP, COLS> &pl) {
    dma_unit<NP, COLS>(s.fill, src, pl);
}
// the same for a whole WUnit<B> (a contiguous slice of a block, so source and LDS image coincide); 32 KB units go as
// two halves
template <int B>
__device__ __forceinline__ void w_prefetch(WStream &s, const int8_t *unit) {
    if (unit == nullptr) return;
    constexpr int NP = WUnit<B>::UK / 16, HALVES = (NP * B * 16 > 16384) ? 2 : 1, NPH = NP / HALVES;
    const DmaPlan<NPH, B> pl = dma_plan<NPH, B>(B);
#pragma unroll
    for (int h = 0; h < HALVES; h++) dma_unit<NPH, B>(s.fill + h * (NPH * B * 16), unit + (size_t)h * (NPH * B * 16), pl);
}
// acc[nt] += unit^T . xop for a unit of KSU k-steps x NTU column groups
template <int KSU, int NTU>
__device__ __forceinline__ void mfma_unit2(v16i *acc, const v4i *xop, const int8_t *lds, int lane) {
    const int i = lane & 31, g = lane >> 5;
#pragma unroll
    for (int ks = 0; ks < KSU; ks++)
#pragma unroll
        for (int nt = 0; nt < NTU; nt++) {
            v4i a = *reinterpret_cast<const v4i *>(lds + ((size_t)(ks * 2 + g) * (NTU * 32) + nt * 32 + i) * 16);
            acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, xop[ks], acc[nt], 0, 0, 0);
        }
}

// acc[nt] += unit^T . xop for the NTW column groups starting at column `colbase` of a staged unit that is
// KSU k-steps deep and `cols` columns wide
// MAXF: fragments (four registers each) read ahead of their MFMAs
template <int KSU, int NTW, int MAXF = 8>
__device__ __forceinline__ void mfma_cols(v16i *acc, const v4i *xop, const int8_t *lds, int cols, int colbase, int lane) {
    const int i = lane & 31, g = lane >> 5;
    // all fragment reads of a batch are issued before its first MFMA, so one LDS latency is exposed per batch
    // instead of one per fragment pair
    constexpr int NB = NTW < MAXF ? NTW : MAXF;                                   // column groups per batch
    constexpr int BK = (KSU * NB <= MAXF) ? KSU : (MAXF / NB > 0 ? MAXF / NB : 1);   // k-steps per batch
    static_assert(NTW % NB == 0 && KSU % BK == 0, "batches must tile the unit");
#pragma unroll
    for (int n0 = 0; n0 < NTW; n0 += NB)
#pragma unroll
    for (int k0 = 0; k0 < KSU; k0 += BK) {
        v4i a[BK * NB];
#pragma unroll
        for (int ks = 0; ks < BK; ks++)
#pragma unroll
            for (int nt = 0; nt < NB; nt++)
                a[ks * NB + nt] = *reinterpret_cast<const v4i *>(lds + ((size_t)((k0 + ks) * 2 + g) * cols + colbase + (n0 + nt) * 32 + i) * 16);
        __builtin_amdgcn_sched_barrier(0);
        // a wave that has its fragments goes first: the matrix pipe is the unit other waves cannot substitute for
        // (measured: 1.8 % on the MLP kernel, nothing elsewhere)
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int ks = 0; ks < BK; ks++)
#pragma unroll
            for (int nt = 0; nt < NB; nt++)
                acc[n0 + nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks * NB + nt], xop[k0 + ks], acc[n0 + nt], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
    }
}

// Column split: for hidden sizes above 128 the H-wide accumulators of one 32-token tile do not fit one wave next to
// its operands, so CS = H/128 waves share a tile and each owns H/CS output columns (and 32*NTU of every sub-chunk
// of the MLP intermediate).  Per-token row statistics and the operands of the next GEMM are exchanged through LDS.
template <int H>
struct Shape {
    static constexpr int CS = H <= 128 ? 1 : H / 128;
    static constexpr int TPW = EGG_WAVES / CS;            // token tiles a workgroup covers per pass
    static constexpr int HS = H / CS, NTS = HS / 32, KS = H / 32;
};

// How the waves of a workgroup map to (member, tile, column slice) for a sequence of T tokens: with at least TPW
// tiles per member the whole workgroup serves one member (one shared set of noise tables) and walks its tiles in
// passes of TPW; with fewer it serves TPW / tiles members at once.
struct TileMap {
    int sets;        // members (= noise table sets) per workgroup
    int passes;
    int set;         // table set of this wave
    int mloc;        // member index within the chunk (may be >= n_members for a padding wave)
    int tile0;       // tile of this wave in pass 0; later passes add TPW
    int tslot;       // which of the workgroup's TPW tiles this wave works on
    int cs;          // column slice of this wave
};
template <int CS>
__device__ __forceinline__ TileMap tile_map(int T, int wave, int block) {
    constexpr int TPW = EGG_WAVES / CS;
    TileMap m; const int tpm = T / 32;
    m.tslot = wave / CS; m.cs = wave % CS;
    if (tpm >= TPW) { m.sets = 1; m.passes = tpm / TPW; m.set = 0; m.mloc = block; m.tile0 = m.tslot; }
    else { m.sets = TPW / tpm; m.passes = 1; m.set = m.tslot / tpm; m.mloc = block * m.sets + m.set; m.tile0 = m.tslot % tpm; }
    return m;
}
static inline int tile_map_sets(int T, int cs) { int tpm = T / 32, tpw = EGG_WAVES / cs; return tpm >= tpw ? 1 : tpw / tpm; }

// Combine a per-token value over the CS waves sharing a tile.  `site` is an LDS area of EGG_WAVES*64 ints that no
// other exchange uses until every wave has passed another barrier.  Every wave of the workgroup must call it.
template <int CS, bool IS_MAX>
__device__ __forceinline__ int xreduce(int v, int *site, const TileMap &tm, int lane) {
    if (CS == 1) return v;
    site[(tm.tslot * CS + tm.cs) * 64 + lane] = v;
    __syncthreads();
    int r = site[(tm.tslot * CS) * 64 + lane];
#pragma unroll
    for (int c = 1; c < CS; c++) { int o = site[(tm.tslot * CS + c) * 64 + lane]; r = IS_MAX ? max(r, o) : r + o; }
    return r;
}

template <int N>
__device__ __forceinline__ void zero_acc(v16i *acc) {
#pragma unroll
    for (int i = 0; i < N; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
}

// ---------------------------------------------------------------- per-member noise tables (one wave fills its own)
__device__ __forceinline__ void fill_noise_i8(int8_t *dst, uint32_t seed, int n, int mask, int lane, int nthr = 64, int mult = 1) {
    for (int i = lane; i < n; i += nthr) dst[i] = (int8_t)(noise_from_hash(seed, i, mask) * mult);
}
// dst[i] = noise(seed, i) * mult
__device__ __forceinline__ void fill_noise_i32(int *dst, uint32_t seed, int n, int mask, int mult, int lane, int nthr = 64) {
    for (int i = lane; i < n; i += nthr) dst[i] = noise_from_hash(seed, i, mask) * mult;
}
// dst[i] = base[i] + ((noise(seed_a,i) * noise(seed_b,i) * ns) >> shift)       (mgpu.cu:666-675, :733-735)
// (the result is stored shifted left by `lshift` where a kernel folds it into a GEMM accumulator)
__device__ __forceinline__ void fill_vec_i32(int *dst, const int8_t *base, uint32_t seed_a, uint32_t seed_b,
                                             int n, int mask, int ns, int shift, int lane, int nthr = 64, int lshift = 0, int add = 0) {
    for (int i = lane; i < n; i += nthr) {
        int v = base[i] + add;
        if (ns != 0) v += (noise_from_hash(seed_a, i, mask) * noise_from_hash(seed_b, i, mask) * ns) >> shift;
        dst[i] = v << lshift;
    }
}
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------- adaptive noise overlay (d-eggs)
// de/include/model/layers.cuh:12-53 (mode 1): an int8 overlay value ov scales a noise term by 0 (ov < 0), ov/64
// (ov < 64) or 1, in float, and the product is converted to int (toward zero).  All operands here are small enough
// for the float product to be exact, so the same value comes out of integer arithmetic: trunc(v * q / 64) with
// q = clamp(ov, 0, 64).  The kernels read q from a device blob laid out like the model blob (a vector tensor's values at
// the tensor's offset; a matrix's input-row values at its offset, its output-column values right behind them).
__device__ __forceinline__ int overlay_q(int ov) { return ov < 0 ? 0 : (ov > 64 ? 64 : ov); }
template <int BITS>
__device__ __forceinline__ int div_pow2_trunc(int t) { return (t + ((t >> 31) & ((1 << BITS) - 1))) >> BITS; }
__device__ __forceinline__ int overlay_scaled(int v, int q) { return div_pow2_trunc<6>(v * q); }
// the table fills above with the q values of the tensor's columns / elements applied
__device__ __forceinline__ void fill_noise_i8_ov(int8_t *dst, uint32_t seed, int n, int mask, int lane, int nthr, int mult, const int8_t *q) {
    for (int i = lane; i < n; i += nthr) dst[i] = (int8_t)(overlay_scaled(noise_from_hash(seed, i, mask), q[i]) * mult);
}
__device__ __forceinline__ void fill_noise_i32_ov(int *dst, uint32_t seed, int n, int mask, int mult, int lane, int nthr, const int8_t *q) {
    for (int i = lane; i < n; i += nthr) dst[i] = overlay_scaled(noise_from_hash(seed, i, mask), q[i]) * mult;
}
__device__ __forceinline__ void fill_vec_i32_ov(int *dst, const int8_t *base, uint32_t seed_a, uint32_t seed_b,
                                                int n, int mask, int ns, int shift, int lane, int nthr, int lshift, const int8_t *q, int add = 0) {
    for (int i = lane; i < n; i += nthr) {
        int v = base[i] + add;
        if (ns != 0) v += (overlay_scaled(noise_from_hash(seed_a, i, mask) * noise_from_hash(seed_b, i, mask), q[i]) * ns) >> shift;
        dst[i] = v << lshift;
    }
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
    return sum_halves(s);
}

// x . B under the overlay: every term x[k] * B[k] is scaled by the input row's factor and truncated before it is added
// (the reference converts each thread's term to int, de/include/model/layers.cuh:240).  qtab holds the rows' q values
// in the order of btab.
template <int KS, bool NAT>
__device__ __forceinline__ int dot_noise_ov(const v4i *xop, const int8_t *btab, const int8_t *qtab, int k_off, int g) {
    const int *b32 = reinterpret_cast<const int *>(btab + k_off);
    const int *q32 = reinterpret_cast<const int *>(qtab + k_off);
    int s = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int kd = NAT ? (8 * ks + 4 * g + q) : (8 * ks + 2 * q + g);
            const int xb = xop[ks][q], nb = b32[kd], qb = q32[kd];
#pragma unroll
            for (int e = 0; e < 4; e++) s += div_pow2_trunc<6>(mul24(mul24(sx8(xb, e), sx8(nb, e)), sx8(qb, e)));
        }
    return sum_halves(s);
}

// ---------------------------------------------------------------- norms on a token held as a packed operand
// apply_standard_norm (mgpu.cu:646-678) in two parts so that the row sum can be combined across waves:
// sum of |x| over N column groups (this lane's half only), then the scaling of N groups whose first column is col0.
// wt / bt are int32 tables already holding w + noise, b + noise.
template <int N>
__device__ __forceinline__ int sumabs_groups(const v4i *x) {
    int tot = 0;
#pragma unroll
    for (int ks = 0; ks < N; ks++)
#pragma unroll
        for (int q = 0; q < 4; q++) tot = sumabs4(x[ks][q], tot);
    return tot;
}
// wt holds 4 * (w + noise).  trunc(a / mn) for |a| <= 2^17 and 1 <= mn <= 127 is the high word of
// (4a) * (floor(2^30 / mn) + 1), plus one when a is negative (checked exhaustively on the CPU); the context refuses
// configurations whose gains could leave that range.
template <int N>
__device__ __forceinline__ void standard_scale(const v4i *x, v4i *out, int mn, const int *wt, const int *bt, int col0, int g) {
    const int M = (int)(1073741824.0 / (double)mn) + 1;       // exact: the quotient is an integer or at least 1/127 away from one
#pragma unroll
    for (int ks = 0; ks < N; ks++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int n0 = col0 + 32 * ks + 8 * q + 4 * g;
            v4i w4 = *reinterpret_cast<const v4i *>(wt + n0);
            v4i b4 = *reinterpret_cast<const v4i *>(bt + n0);
            int o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int a4 = mul24(sx8(x[ks][q], e), w4[e]);
                o[e] = clip127(__mulhi(a4, M) + (int)((unsigned)a4 >> 31) + b4[e]);
            }
            out[ks][q] = pack4(o[0], o[1], o[2], o[3]);
        }
}
template <int KS>
__device__ __forceinline__ void standard_norm(const v4i *x, v4i *out, const int *wt, const int *bt, int g) {
    int tot = sumabs_groups<KS>(x);
    tot = sum_halves(tot);
    int mn = tot / (32 * KS); if (!mn) mn = 1;
    standard_scale<KS>(x, out, mn, wt, bt, 0, g);
}

// adaptive_*_normalize (egg_adaptive_normalize.h:10-103), also in two parts: max |val| over NT column groups
// (both lane halves of the token combined), then the scaling.  The reference's final clamp to +-127 never binds:
// |val| <= mx, so (float)val * (127.0f / (float)mx) <= 127 * (1 + 2^-23) and rounds to at most 127.
template <int NT>
__device__ __forceinline__ int absmax_groups(const v16i *val) {
    int hi = 0, lo = 0;
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            hi = max(max(hi, val[nt][r]), val[nt][r + 1]);
            lo = min(min(lo, val[nt][r]), val[nt][r + 1]);
        }
    int mx = max(hi, -lo);
    return max_halves(mx);
}
template <int NT>
__device__ __forceinline__ void adaptive_scale(const v16i *val, int mx, v4i *out) {
    const float scale = 127.0f / ((float)mx + 1e-9f);
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = round_half_away((float)val[nt][4 * q + e] * scale);
            out[nt][q] = pack4(o[0], o[1], o[2], o[3]);
        }
}
template <int NT>
__device__ __forceinline__ void adaptive_norm(const v16i *val, v4i *out) {
    adaptive_scale<NT>(val, absmax_groups<NT>(val), out);
}

// The same two parts with the conversion to float first: (float) is monotonic, so the largest |(float)val| is the
// float of the largest |val| the reference converts, and |.| is an operand modifier of the float maximum (one
// three-operand maximum per two values instead of a maximum and a minimum).  The values are left as floats (bit
// patterns) for the scaling; the result is the maximum's bit pattern, which orders like the float since it is not negative.
template <int NT>
__device__ __forceinline__ int absmax_to_float_groups(v16i *val) {
    float m0 = 0.0f, m1 = 0.0f;
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int r = 0; r < 16; r += 4) {
            const float a = (float)val[nt][r], b = (float)val[nt][r + 1], c2 = (float)val[nt][r + 2], d = (float)val[nt][r + 3];
            m0 = fmaxf(fmaxf(m0, fabsf(a)), fabsf(b));
            m1 = fmaxf(fmaxf(m1, fabsf(c2)), fabsf(d));
            val[nt][r] = __float_as_int(a); val[nt][r + 1] = __float_as_int(b);
            val[nt][r + 2] = __float_as_int(c2); val[nt][r + 3] = __float_as_int(d);
        }
    return max_halves(__float_as_int(fmaxf(m0, m1)));
}
template <int NT>
__device__ __forceinline__ void adaptive_scale_floats(const v16i *valf, int mx_bits, v4i *out) {
    const float scale = 127.0f / (__int_as_float(mx_bits) + 1e-9f);
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = round_half_away(__int_as_float(valf[nt][4 * q + e]) * scale);
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
