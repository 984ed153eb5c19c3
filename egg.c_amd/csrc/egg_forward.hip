// egg_forward.hip -- Int8NativeFormer population forward on gfx950 (hand-written MFMA kernels).
//
// Reference: train_sequence_kernel and its device functions,
// full_cuda_train_transformer_adam_mgpu.cu:553-1029 ("mgpu.cu"), which runs one member per block,
// serially over tokens.  Here tokens are the GEMM's free dimension: a wave owns a tile of 32 tokens of
// one member, four waves share each W block staged in LDS, and a launch covers a chunk of members.
//   k_mlp<H,true>   embedding stage + initial MLP          (mgpu.cu:901-934, :708-759)
//   k_qkv<H,..>     LN1 + Q/K/V projections + RoPE + norms (mgpu.cu:769-784)
//   k_attn<HD,CT>   causal exp-LUT attention core          (mgpu.cu:787-825)
//   k_mlp<H,false>  O-projection + residual norm + MLP     (mgpu.cu:827-831, :708-759)
//   k_head<H>       final norm + tied head + loss          (mgpu.cu:955-1028)
#include <algorithm>
#include "egg_device.h"
#include "egg_params.h"
#include "egg_launch.h"

#pragma clang fp contract(off)

// stream position of a member's pair (mgpu.cu:864-870)
__device__ __forceinline__ int64_t stream_pos_of(const FwdCommon &c, int member) {
    int64_t pair = c.same_data ? 0 : member / 2;
    int64_t stride = c.data_len / (c.population / 2);
    return (*c.d_start_idx + pair * stride) % (c.data_len - c.T);
}

// token i of the stream: bytes, or uint32 where the vocabulary is larger than 256 (TokenType, de/include/config.h:26-28)
__device__ __forceinline__ int token_at(const FwdCommon &c, int64_t i) {
    return c.token_bytes == 4 ? (int)reinterpret_cast<const uint32_t *>(c.data)[i] : (int)c.data[i];
}

// acc[nt][r] += (sb * At[n]) >> sigma for NT column groups starting at table offset n_off
template <int NT>
__device__ __forceinline__ void add_perturb(v16i *acc, int sb, const int *At, int n_off, int sigma, int g) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            v4i a4 = *reinterpret_cast<const v4i *>(At + n_off + 32 * nt + 8 * q + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; e++) acc[nt][4 * q + e] += mul24(sb, a4[e]) >> sigma;
        }
}

// same with the output-side noise kept as int8, already multiplied by the member's sign
template <int NT>
__device__ __forceinline__ void add_perturb8(v16i *acc, int sb, const int8_t *At, int n_off, int sigma, int g) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int a4 = *reinterpret_cast<const int *>(At + n_off + 32 * nt + 8 * q + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; e++) acc[nt][4 * q + e] += mul24(sb, sx8(a4, e)) >> sigma;
        }
}

// (acc + ((sb * a) >> sigma)) >> shift.  With FUSE it is evaluated as ((acc << sigma) + sb * a) >> (sigma + shift):
// floor(floor(y / 2^sigma + acc) / 2^shift) == floor((y + acc * 2^sigma) / 2^(sigma + shift)) for integers, one
// instruction less.  The host selects FUSE only when |acc| * 2^sigma + |sb * a| < 2^31 for the GEMM depth in question.
template <bool FUSE>
__device__ __forceinline__ int perturb_shift(int acc, int sb, int a, int sigma, int shift) {
    // (measured: forcing the multiply apart from the add -- v_mul_i32_i24 with a byte operand select plus
    // v_lshl_add_u32, one instruction less per element -- runs 2 % slower than the multiply-add the compiler picks)
    if (FUSE) return (int)(((unsigned)acc << sigma) + (unsigned)mul24(sb, a)) >> (sigma + shift);
    return (acc + (mul24(sb, a) >> sigma)) >> shift;
}
// acc[nt][r] = perturb_shift(acc[nt][r], sb, At[n], ...) for NT column groups starting at table offset n_off
template <int NT, bool FUSE>
__device__ __forceinline__ void perturb_shift_groups(v16i *acc, int sb, const int8_t *At, int n_off, int sigma, int shift, int g) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            int a4 = *reinterpret_cast<const int *>(At + n_off + 32 * nt + 8 * q + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; e++) acc[nt][4 * q + e] = perturb_shift<FUSE>(acc[nt][4 * q + e], sb, sx8(a4, e), sigma, shift);
        }
}

// exchange of packed 32-column groups between the waves sharing a tile: group k of tile slot ts, 16 bytes per lane
__device__ __forceinline__ void xch_put(int8_t *xch, int groups, int ts, int k, int lane, v4i v) {
    *reinterpret_cast<v4i *>(xch + ((size_t)(ts * groups + k) * 64 + lane) * 16) = v;
}
__device__ __forceinline__ v4i xch_get(const int8_t *xch, int groups, int ts, int k, int lane) {
    return *reinterpret_cast<const v4i *>(xch + ((size_t)(ts * groups + k) * 64 + lane) * 16);
}

// Hand the packed groups of the normalised operand from the wave that computed them to every wave of the tile through
// the idle W buffer `buf` (`unit` bytes).  When the TPW tiles' operands exceed the buffer, the column slices take
// turns (ROUNDS rounds of SPR slices each).  Every wave of the workgroup must call it.
template <int CS, int NTS, int KS, int TPW, int UNIT_BYTES>
__device__ __forceinline__ void exchange_operand(int8_t *buf, const TileMap &tm, int lane, const v4i *mine, v4i *full) {
    constexpr int ROUNDS = (TPW * KS * 1024 + UNIT_BYTES - 1) / UNIT_BYTES, SPR = CS / ROUNDS, GR = SPR * NTS;
    static_assert(CS % ROUNDS == 0 && TPW * GR * 1024 <= UNIT_BYTES, "operand exchange does not fit the W buffer");
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        if (tm.cs / SPR == r)
#pragma unroll
            for (int nt = 0; nt < NTS; nt++) xch_put(buf, GR, tm.tslot, (tm.cs % SPR) * NTS + nt, lane, mine[nt]);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GR; k++) full[r * GR + k] = xch_get(buf, GR, tm.tslot, k, lane);
        if (r + 1 < ROUNDS) __syncthreads();
    }
}

// ============================================================================ MLP block
// The 4H-wide intermediate is produced SC columns at a time (up GEMM, GELU epilogue, immediately consumed as k-steps
// of the down GEMM), so only the down accumulator of the wave's column slice, the normalised input and one
// sub-chunk accumulator are live.  W streams through two LDS buffers in units of at most 16 KB.  The residual is
// parked in the x buffer and re-read at the end.
template <int H>
struct MlpCfg {
    typedef Shape<H> S;
    // hidden 512 runs the MLP with two column slices (not four): twice the MFMAs per staged unit and half the
    // exchanges outweigh the register spills of the 256-column accumulator
    static constexpr int CS = H == 512 ? 2 : S::CS;
    static constexpr int TPW = EGG_WAVES / CS, HS = H / CS, NTS = HS / 32, KS = H / 32;
    static constexpr int NTU = CS == 1 ? 2 : 1;          // up-GEMM column groups per wave and sub-chunk
    static constexpr int SC = 32 * CS * NTU;             // intermediate columns per sub-chunk
    static constexpr int NSUB = 4 * H / SC;
    static constexpr int cmin(int a, int b) { return a < b ? a : b; }
    static constexpr int cmax(int a, int b) { return a > b ? a : b; }
    // p-rows (16 k-bytes each, two per k-step) per staged unit and units per GEMM
    static constexpr int PRO = cmin(H / 16, 1024 / H), OU = (H / 16) / PRO;         // O projection  [H x H]
    static constexpr int PRUP = cmin(H / 16, 1024 / SC), UPU = (H / 16) / PRUP;     // up sub-chunk  [H x SC]
    static constexpr int PRDN = cmin(SC / 16, 1024 / H), DNU = (SC / 16) / PRDN;    // down sub-chunk [SC x H]
    static constexpr int UNIT = 16 * cmax(PRO * H, cmax(PRUP * SC, PRDN * H));
    static constexpr int WBYTES = 2 * UNIT;
    static constexpr int I32 = 9 * H;        // ex0[H] ex1[H] lnw[H] lnb[H] bup[4H] bdn[H]
    static constexpr int I8 = 11 * H;        // exB[H] upB[H] dnB[4H] upA[4H] dnA[H]   (A noise already times the sign)
    // The blocks behind the first one keep the up projection's output noise as int32 (UPA32): the GELU epilogue then
    // multiplies by a table word as it stands instead of extracting a byte per element.  The first block has no room
    // for it at three workgroups per CU (its value-rank tables take the space) and keeps the bytes.
    static constexpr int UPA32 = 3 * 4 * H;  // extra bytes of the int32 form: upA occupies 16H instead of 4H
    static constexpr int PER_SET = I32 * 4 + I8;
    // The normalised input is exchanged through whichever W buffer is idle at that point (TPW*32*H <= UNIT bytes);
    // the intermediate slices have their own small area because both W buffers are busy inside the sub-chunk loop.
    static constexpr int XCHG = CS > 1 ? TPW * 32 * SC : 0;
    static constexpr int SITE = EGG_WAVES * 64;                       // ints per reduction site
    static constexpr int RED = CS > 1 ? 2 * SITE * 4 : 0;             // two reduction sites used alternately
    static constexpr int OCC = H == 256 ? 3 : 2;                      // workgroups per CU the kernel is built for
    // first block only: rank of every byte value among the values present in the member's window [256], wave counts
    // [4 ints], and below hidden 256 the list of present values [256] (from hidden 256 on it lives in the table slot
    // of the O projection's noise, which the first block does not use)
    static constexpr int DEDUP = 256 + 16 + (H < 256 ? 256 : 0);
    static constexpr int ACT = 256;          // GELU table: entry v + 128 holds the activation of the int8 value v
    // (behind the first block ex1 does not exist: 4H bytes less.  At hidden 256 the total stays at 52 KB: the LDS is
    // handed out in granules, three workgroups of 53 KB no longer share a CU, and the kernel then runs 9 % slower.)
    static constexpr int per_set(bool first) { return PER_SET + (first ? 0 : UPA32 - 4 * H); }
    static int total(int sets, bool first) { return WBYTES + ACT + sets * per_set(first) + XCHG + RED + (first ? DEDUP : 0); }
};

// FUSE: the host has checked sigma <= 7 and |noise| <= 15, which bounds |acc| * 2^sigma + |sb * a| below 2^31 for
// GEMM depths up to 1024 (depth * 127 * 127 * 128 + depth * 127 * 225), and the same bound for the up accumulator
// with its bias seed (egg_mlp_up_acc_bound); the down projection (depth 4H) uses the fused form only for 4H <= 1024.
// ADAPT: the d-eggs adaptive noise overlay is on (de/include/model/layers.cuh:215-296, :432-438,
// de/src/kernels.cu:139-158); see k_qkv.  The down projection's input-side sum follows the reference thread of a
// hidden unit, which adds its four terms (k = unit, unit + H, ...) into an int one float addition at a time; the
// sub-chunks are therefore visited so that those four are consecutive.
template <int H, bool FIRST, bool FUSE, bool ADAPT>
__global__ void __launch_bounds__(EGG_THREADS, MlpCfg<H>::OCC) k_mlp(MlpParams p) {
    typedef MlpCfg<H> M;
    constexpr bool FUSE_DN = FUSE && 4 * H <= 1024;
    constexpr int CS = M::CS, KS = M::KS, NTS = M::NTS, HS = M::HS, NTU = M::NTU, SC = M::SC;
    // fragments read ahead of their MFMAs: at hidden 512 the accumulators and operands leave room for four
    constexpr int MAXF = H == 512 ? 4 : 8;
    extern __shared__ __align__(16) int8_t smem[];
    int8_t *act = smem + M::WBYTES;
    // The GELU table is read through an LDS address formed from the index itself plus a constant offset, which assumes
    // that the dynamic LDS block starts at LDS address 0 (the kernel declares no static LDS); built from the `act`
    // pointer instead, every read carries an extra add of that (zero) base.
    typedef const __attribute__((address_space(3))) uint8_t *lds_u8_ptr;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const FwdCommon &c = p.c;
    const int T = c.T;
    const TileMap tm = tile_map<CS>(c.tn, wave, blockIdx.x);
    const int col0 = tm.cs * HS;                      // first output column of this wave's slice
    constexpr int PSET = M::per_set(FIRST);
    constexpr bool UPA32 = !FIRST;
    int8_t *tb = act + M::ACT + tm.set * PSET;
    int *ex0 = reinterpret_cast<int *>(tb);           // FIRST: emb_bias + noise   | else: O-proj A noise * ns as int8
    int *ex1 = ex0 + H;                               // FIRST: b_dim noise * ns    | else: absent
    int *lnw = ex1 + (FIRST ? H : 0), *lnb = lnw + H, *bup = lnb + H, *bdn = bup + 4 * H;
    int8_t *exB = reinterpret_cast<int8_t *>(bdn + H);   // O-proj B noise
    int8_t *upB = exB + H, *dnB = upB + H, *upA = dnB + 4 * H, *dnA = upA + (UPA32 ? 16 : 4) * H;
    const int8_t *oA = reinterpret_cast<const int8_t *>(ex0);
    int8_t *xch = act + M::ACT + tm.sets * PSET;
    int *red = reinterpret_cast<int *>(xch + M::XCHG);
    int rsite = 0;          // the two reduction sites take turns, call by call (the same sequence in every wave)
    auto next_site = [&]() { rsite ^= 1; return red + rsite * M::SITE; };

    WStream ws; wstream_init(ws, smem, M::UNIT);
    // unit sources inside the fragment-major copies (block size == H)
    const DmaPlan<M::PRUP, SC> plan_up = dma_plan<M::PRUP, SC>(H);
    const DmaPlan<M::PRDN, H> plan_dn = dma_plan<M::PRDN, H>(H);
    const DmaPlan<M::PRO, H> plan_o = dma_plan<M::PRO, H>(H);
    auto pf_up = [&](int s, int ku) {
        const int n = s * SC;
        w_prefetch2<M::PRUP, SC>(ws, p.w_up + (size_t)(n / H) * H * H + ((size_t)ku * M::PRUP * H + n % H) * 16, plan_up);
    };
    auto pf_dn = [&](int s, int du) {
        const int k = s * SC;
        w_prefetch2<M::PRDN, H>(ws, p.w_dn + (size_t)(k / H) * H * H + (size_t)((k % H) / 16 + du * M::PRDN) * H * 16, plan_dn);
    };
    // (the unit index passes through an empty asm so that the four unit addresses are formed where they are used:
    // precomputed in front of the pass loop they overflow the scalar registers and are spilled through scratch)
    auto pf_o = [&](int u) {
        asm volatile("" : "+s"(u));
        w_prefetch2<M::PRO, H>(ws, p.w_o + (size_t)(unsigned)u * (M::PRO * H * 16), plan_o);
    };
    auto pf_pass_first = [&]() { if (FIRST) pf_up(0, 0); else pf_o(0); };
    pf_pass_first();

    for (int i = threadIdx.x; i < 256; i += EGG_THREADS)      // act_lut is indexed by the value's two's-complement byte
        act[(i + 128) & 255] = c.act_lut[i];
    for (int ss = 0; ss < tm.sets; ss++) {
        int ml = blockIdx.x * tm.sets + ss; if (ml >= c.n_members) ml = c.n_members - 1;
        const int mem = c.pop_offset + ml, nsx = (mem & 1) ? -1 : 1;
        const uint32_t pseed = *c.d_step_seed + (uint32_t)(mem / 2), sbx = pseed + (uint32_t)p.seed_base;
        int8_t *t2 = act + M::ACT + ss * PSET;
        int *e0 = reinterpret_cast<int *>(t2), *e1 = e0 + H, *lw = e1 + (FIRST ? H : 0), *lb = lw + H, *bu = lb + H, *bd = bu + 4 * H;
        int8_t *eB = reinterpret_cast<int8_t *>(bd + H), *uB = eB + H, *dB = uB + H, *uA = dB + 4 * H, *dA = uA + (UPA32 ? 16 : 4) * H;
        const int tid = threadIdx.x;
        if (ADAPT) {
            if (FIRST) {
                fill_vec_i32_ov(e0, p.emb_bias, pseed + OFF_EMB_BIAS_A, pseed + OFF_EMB_BIAS_B, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 0, p.q_emb_bias);
                // b_dim * q(hidden) * ns, not yet divided: the token's factor joins before the truncation
                for (int i = tid; i < H; i += EGG_THREADS) e1[i] = noise_from_hash(pseed + OFF_EMB + H, i, c.mask) * p.q_emb[i] * nsx;
            } else {
                fill_noise_i8_ov(reinterpret_cast<int8_t *>(e0), sbx + OFF_O_A, H, c.mask, tid, EGG_THREADS, nsx, p.q_o + H);
                fill_noise_i8(eB, sbx + OFF_O_B, H, c.mask, tid, EGG_THREADS);
            }
            fill_vec_i32_ov(lw, p.ln_w, sbx + p.off_ln_a, sbx + p.off_ln_b, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 2, p.q_ln_w);
            fill_vec_i32_ov(lb, p.ln_b, sbx + p.off_lnb_a, sbx + p.off_lnb_b, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 0, p.q_ln_b);
            if (UPA32) fill_noise_i32_ov(reinterpret_cast<int *>(uA), sbx + p.off_up_a, 4 * H, c.mask, nsx, tid, EGG_THREADS, p.q_up + H);
            else fill_noise_i8_ov(uA, sbx + p.off_up_a, 4 * H, c.mask, tid, EGG_THREADS, nsx, p.q_up + H);
            fill_vec_i32_ov(bu, p.b_up, sbx + p.off_bup_a, sbx + p.off_bup_b, 4 * H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, c.shift_mlp_up, p.q_b_up, 128);
            fill_noise_i8_ov(dA, sbx + p.off_dn_a, H, c.mask, tid, EGG_THREADS, nsx, p.q_dn + 4 * H);
            fill_vec_i32_ov(bd, p.b_dn, sbx + p.off_bdn_a, sbx + p.off_bdn_b, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 0, p.q_b_dn);
            fill_noise_i8(uB, sbx + p.off_up_b, H, c.mask, tid, EGG_THREADS);
            fill_noise_i8(dB, sbx + p.off_dn_b, 4 * H, c.mask, tid, EGG_THREADS);
            continue;
        }
        if (FIRST) {
            fill_vec_i32(e0, p.emb_bias, pseed + OFF_EMB_BIAS_A, pseed + OFF_EMB_BIAS_B, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS);
            fill_noise_i32(e1, pseed + OFF_EMB + H, H, c.mask, nsx, tid, EGG_THREADS);
        } else {
            fill_noise_i8(reinterpret_cast<int8_t *>(e0), sbx + OFF_O_A, H, c.mask, tid, EGG_THREADS, nsx);
            fill_noise_i8(eB, sbx + OFF_O_B, H, c.mask, tid, EGG_THREADS);
        }
        fill_vec_i32(lw, p.ln_w, sbx + p.off_ln_a, sbx + p.off_ln_b, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 2);     // 4 * gain, see standard_scale
        fill_vec_i32(lb, p.ln_b, sbx + p.off_lnb_a, sbx + p.off_lnb_b, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS);
        if (UPA32) fill_noise_i32(reinterpret_cast<int *>(uA), sbx + p.off_up_a, 4 * H, c.mask, nsx, tid, EGG_THREADS);
        else fill_noise_i8(uA, sbx + p.off_up_a, 4 * H, c.mask, tid, EGG_THREADS, nsx);
        // the up bias is stored as (b + 128) << shift_mlp_up and seeds the up accumulator: ((a + (b << s)) >> s) == (a >> s) + b;
        // the 128 makes the clamped result (1..255) the GELU table's index
        fill_vec_i32(bu, p.b_up, sbx + p.off_bup_a, sbx + p.off_bup_b, 4 * H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, c.shift_mlp_up, 128);
        fill_noise_i8(dA, sbx + p.off_dn_a, H, c.mask, tid, EGG_THREADS, nsx);
        fill_vec_i32(bd, p.b_dn, sbx + p.off_bdn_a, sbx + p.off_bdn_b, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS);
        fill_noise_i8(uB, sbx + p.off_up_b, H, c.mask, tid, EGG_THREADS);
        fill_noise_i8(dB, sbx + p.off_dn_b, 4 * H, c.mask, tid, EGG_THREADS);
    }
    __syncthreads();

    int mloc = tm.mloc;
    const bool valid = mloc < c.n_members;
    if (!valid) mloc = c.n_members - 1;
    const int member = c.pop_offset + mloc;
    const uint32_t pair_seed = *c.d_step_seed + (uint32_t)(member / 2);
    const int64_t spos = FIRST ? stream_pos_of(c, member) : 0;

    // The first block (embedding, norm, MLP, residual, adaptive norm) has no attention in front of it: its result is a
    // function of the member and the byte value alone.  It is therefore evaluated once per distinct byte value of the
    // member's window -- row r of `p.tab` belongs to the r-th smallest value present -- and copied to every position
    // that holds the value at the end.  (A workgroup that serves several members keeps the per-position form.)
    const bool dedup = FIRST && p.tab != nullptr && tm.sets == 1;
    uint8_t *rnk = reinterpret_cast<uint8_t *>(red) + M::RED;
    int *wcnt = reinterpret_cast<int *>(rnk + 256);
    uint8_t *uniq = H < 256 ? rnk + 272 : reinterpret_cast<uint8_t *>(exB);
    int npass = tm.passes, nrows = T;
    if (FIRST && dedup) {
        static_assert(EGG_THREADS == 256, "one thread per byte value");
        rnk[threadIdx.x] = 0;
        __syncthreads();
        for (int t = threadIdx.x; t < T; t += EGG_THREADS) rnk[c.data[spos + t]] = 1;
        __syncthreads();
        const bool present = rnk[threadIdx.x] != 0;
        const unsigned long long bal = __ballot(present);
        if (lane == 0) wcnt[wave] = __popcll(bal);
        __syncthreads();
        int below = 0;
        nrows = 0;
#pragma unroll
        for (int w = 0; w < EGG_WAVES; w++) { const int n = wcnt[w]; if (w < wave) below += n; nrows += n; }
        const int r = below + __popcll(bal & ((1ull << lane) - 1ull));
        if (present) { rnk[threadIdx.x] = (uint8_t)r; uniq[r] = (uint8_t)threadIdx.x; }
        __syncthreads();
        npass = (nrows + 32 * M::TPW - 1) / (32 * M::TPW);
    }

    for (int pass = 0; pass < npass; pass++) {
        // The lane index is re-read behind an empty asm at the top of a pass and again behind the sub-chunk loop: the
        // table and exchange addresses of the code around the loop are then formed where they are used instead of
        // being computed once in front of the pass loop and held (or spilled) across the sub-chunk loop.
        int laneA = lane;
        asm volatile("" : "+v"(laneA));
        const int gA = laneA >> 5, jA = laneA & 31;
        const int t = c.t0 + (tm.tile0 + M::TPW * pass) * 32 + jA;     // token position; with dedup, row of the table
        const size_t row = ((size_t)mloc * T + t) * H;
        int8_t *xrow = (FIRST && dedup ? p.tab : p.x) + row + col0;   // this wave's slice of the residual row
        v4i xs[NTS];

        if (FIRST) {
            // embedding stage (mgpu.cu:901-931)
            const int tok = dedup ? uniq[min(t, nrows - 1)] : token_at(c, spos + t);
            int a_tok = noise_from_hash(pair_seed + OFF_EMB, (uint32_t)tok, c.mask);
            if (ADAPT) a_tok *= p.q_emb[H + tok];        // a_tok * q(token); the table holds b_dim * q(hidden) * ns
            const uint32_t *E32 = reinterpret_cast<const uint32_t *>(p.embedding);
#pragma unroll
            for (int nt = 0; nt < NTS; nt++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int n0 = col0 + 32 * nt + 8 * q + 4 * gA;
                    int e4 = (int)E32[(size_t)(n0 >> 2) * c.vocab + tok];
                    v4i b4 = *reinterpret_cast<const v4i *>(ex0 + n0);
                    v4i d4 = *reinterpret_cast<const v4i *>(ex1 + n0);
                    int o[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        int pp = mul24(a_tok, d4[e]);
                        if (ADAPT) pp = div_pow2_trunc<12>(pp);      // (int)(a * b * f(token) * f(hidden)), both factors x/64
                        o[e] = clip127(sx8(e4, e) + b4[e] + (pp >> c.sigma));
                    }
                    xs[nt][q] = pack4(o[0], o[1], o[2], o[3]);
                }
        } else {
            // attention output projection + residual + adaptive norm (mgpu.cu:827-831)
            v16i acc[NTS];
            zero_acc<NTS>(acc);
            int sbo;
            {
                v4i aop[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ks++) aop[ks] = load_op(p.ao + row, ks, gA);
                sbo = ADAPT ? dot_noise_ov<KS, false>(aop, exB, p.q_o, 0, gA) : dot_noise<KS, false>(aop, exB, 0, gA);
#pragma unroll
                for (int u = 0; u < M::OU; u++) {
                    const int8_t *cur = w_acquire(ws);
                    if (u + 1 < M::OU) pf_o(u + 1); else pf_up(0, 0);
                    mfma_cols<M::PRO / 2, NTS, MAXF>(acc, aop + u * (M::PRO / 2), cur, H, col0, laneA);
                }
            }
            perturb_shift_groups<NTS, FUSE>(acc, sbo, oA, col0, c.sigma, c.shift_out, gA);
#pragma unroll
            for (int nt = 0; nt < NTS; nt++) {
                v4i xr = load_op(xrow, nt, gA);
#pragma unroll
                for (int r = 0; r < 16; r++) acc[nt][r] += sx8(xr[r >> 2], r & 3);
            }
            const int mx = xreduce<CS, true>(absmax_to_float_groups<NTS>(acc), next_site(), tm, laneA);
            adaptive_scale_floats<NTS>(acc, mx, xs);
            if (p.x_mid && valid)
#pragma unroll
                for (int nt = 0; nt < NTS; nt++) store_op(p.x_mid + row + col0, nt, gA, xs[nt]);
        }
        // park the residual (this wave owns the slice; invalid padding waves only recompute, and so do the rows of the
        // value table beyond the number of distinct values: nothing reads them, so nothing of them is written)
        const bool keep = valid && (!(FIRST && dedup) || t < nrows);
        if (keep)
#pragma unroll
            for (int nt = 0; nt < NTS; nt++) store_op(xrow, nt, gA, xs[nt]);

        // MLP (mgpu.cu:708-759)
        v4i nrm[KS];
        {
            int tot = sumabs_groups<NTS>(xs);
            tot = sum_halves(tot);
            tot = xreduce<CS, false>(tot, next_site(), tm, laneA);
            int mn = tot / H; if (!mn) mn = 1;
            if constexpr (CS == 1) standard_scale<NTS>(xs, nrm, mn, lnw, lnb, 0, gA);
            else {
                // ws.other holds the unit consumed last; every wave has passed a barrier since reading it, and the
                // next prefetch into it is issued only after the barrier of the next w_acquire
                v4i mine[NTS];
                standard_scale<NTS>(xs, mine, mn, lnw, lnb, col0, gA);
                exchange_operand<CS, NTS, KS, M::TPW, M::UNIT>(ws.other, tm, laneA, mine, nrm);
            }
        }
        const int sbu = ADAPT ? dot_noise_ov<KS, false>(nrm, upB, p.q_up, 0, gA) : dot_noise<KS, false>(nrm, upB, 0, gA);
        v16i accd[NTS];
        zero_acc<NTS>(accd);
        int sbd = 0;
        int pb[ADAPT ? NTU * 16 : 1];           // ADAPT: running sums of the reference threads this laneA stands in for
        // ADAPT: iteration it visits sub-chunk (it % 4) * NSUB/4 + it / 4, so four consecutive iterations cover the
        // intermediate columns unit, unit + H, unit + 2H, unit + 3H of the same hidden units
        auto sub_chunk = [](int it) { return ADAPT ? (it & 3) * (M::NSUB / 4) + (it >> 2) : it; };
        int laneL = lane;
        asm volatile("" : "+v"(laneL));
        const int gL = laneL >> 5;
#pragma unroll 1
        for (int it = 0; it < M::NSUB; it++) {
            const int s = sub_chunk(it);
            v16i au[NTU];
#pragma unroll
            for (int nt = 0; nt < NTU; nt++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    v4i b4 = *reinterpret_cast<const v4i *>(bup + s * SC + tm.cs * 32 * NTU + 32 * nt + 8 * q + 4 * gL);
#pragma unroll
                    for (int e = 0; e < 4; e++) au[nt][4 * q + e] = b4[e];
                }
#pragma unroll
            for (int ku = 0; ku < M::UPU; ku++) {
                const int8_t *cur = w_acquire(ws);
                if (ku + 1 < M::UPU) pf_up(s, ku + 1); else pf_dn(s, 0);
                mfma_cols<M::PRUP / 2, NTU, MAXF>(au, nrm + ku * (M::PRUP / 2), cur, SC, tm.cs * 32 * NTU, laneL);
            }
            v4i mid[CS * NTU];
            {
                const int nb = s * SC + tm.cs * 32 * NTU;            // first intermediate column of this wave
                const int *dnb32 = reinterpret_cast<const int *>(dnB + nb);
                v4i mine[NTU];
#pragma unroll
                for (int nt = 0; nt < NTU; nt++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        int n0 = nb + 32 * nt + 8 * q + 4 * gL;
                        int a4 = 0; v4i a32 = {0, 0, 0, 0};
                        if (UPA32) a32 = *reinterpret_cast<const v4i *>(reinterpret_cast<const int *>(upA) + n0);
                        else a4 = *reinterpret_cast<const int *>(upA + n0);
                        uint32_t r4[4];          // the activation of element e as an unsigned byte
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            // the accumulator carries + 128 (see the bias table): clamping to 1..255 is the clamp to +-127,
                            // and the result is the table index as it stands
                            const int idx = min(255, max(1, perturb_shift<FUSE>(au[nt][4 * q + e], sbu, UPA32 ? a32[e] : sx8(a4, e), c.sigma, c.shift_mlp_up)));
                            r4[e] = reinterpret_cast<lds_u8_ptr>((uintptr_t)(uint32_t)idx)[M::WBYTES];
                        }
                        // bytes 0 of the four results side by side: two byte permutes and an or
                        mine[nt][q] = (int)(__builtin_amdgcn_perm(r4[1], r4[0], 0x0c0c0400u) | __builtin_amdgcn_perm(r4[3], r4[2], 0x04000c0cu));
                        if (!ADAPT) sbd = dot4(mine[nt][q], dnb32[8 * nt + 2 * q + gL], sbd);
                        else {
                            const int nz4 = dnb32[8 * nt + 2 * q + gL], q4 = *reinterpret_cast<const int *>(p.q_dn + n0);
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                const int idx = ADAPT ? (nt * 4 + q) * 4 + e : 0;
                                const int prev = (it & 3) ? pb[idx] : 0;
                                // (int)((float)pb + x * n * q / 64): every value is a multiple of 1/64 below 2^24
                                pb[idx] = div_pow2_trunc<6>((prev << 6) + mul24(mul24(sx8((int)r4[e], 0), sx8(nz4, e)), sx8(q4, e)));
                            }
                        }
                    }
                if (ADAPT && (it & 3) == 3) {
#pragma unroll
                    for (int i2 = 0; i2 < (ADAPT ? NTU * 16 : 1); i2++) sbd += pb[i2];
                }
                if (CS == 1) {
#pragma unroll
                    for (int nt = 0; nt < NTU; nt++) mid[nt] = mine[nt];
                } else {
#pragma unroll
                    for (int nt = 0; nt < NTU; nt++) xch_put(xch, CS * NTU, tm.tslot, tm.cs * NTU + nt, laneL, mine[nt]);
                }
            }
#pragma unroll
            for (int du = 0; du < M::DNU; du++) {
                const int8_t *cur = w_acquire(ws);        // its barrier also publishes the intermediate slices
                if (CS > 1 && du == 0)
#pragma unroll
                    for (int k = 0; k < CS * NTU; k++) mid[k] = xch_get(xch, CS * NTU, tm.tslot, k, laneL);
                if (du + 1 < M::DNU) pf_dn(s, du + 1);
                else if (it + 1 < M::NSUB) pf_up(sub_chunk(it + 1), 0);
                else if (pass + 1 < npass) pf_pass_first();
                mfma_cols<M::PRDN / 2, NTS, MAXF>(accd, mid + du * (M::PRDN / 2), cur, H, col0, laneL);
            }
        }
        int laneB = lane;
        asm volatile("" : "+v"(laneB));
        const int gB = laneB >> 5;
        sbd = sum_halves(sbd);
        sbd = xreduce<CS, false>(sbd, next_site(), tm, laneB);
        perturb_shift_groups<NTS, FUSE_DN>(accd, sbd, dnA, col0, c.sigma, c.shift_mlp_down, gB);
#pragma unroll
        for (int nt = 0; nt < NTS; nt++) {
            v4i xr = load_op(xrow, nt, gB);          // the parked residual (for a padding wave: someone else's row, unused)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                v4i b4 = *reinterpret_cast<const v4i *>(bdn + col0 + 32 * nt + 8 * q + 4 * gB);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    accd[nt][4 * q + e] += sx8(xr[q], e) + b4[e];
            }
        }
        v4i xnew[NTS];
        const int mx2 = xreduce<CS, true>(absmax_to_float_groups<NTS>(accd), next_site(), tm, laneB);
        adaptive_scale_floats<NTS>(accd, mx2, xnew);
        if (keep)
#pragma unroll
            for (int nt = 0; nt < NTS; nt++) store_op(xrow, nt, gB, xnew[nt]);
    }
    if (FIRST && dedup) {
        // every position takes the row of its byte value (16 bytes per thread and step)
        __syncthreads();
        constexpr int PARTS = H / 16;
        for (int i = threadIdx.x; i < T * PARTS; i += EGG_THREADS) {
            const int t = i / PARTS, part = i % PARTS;
            const int r = rnk[c.data[spos + t]];
            const v4i v = *reinterpret_cast<const v4i *>(p.tab + ((size_t)mloc * T + r) * H + part * 16);
            *reinterpret_cast<v4i *>(p.x + ((size_t)mloc * T + t) * H + part * 16) = v;
        }
    }
}

// ============================================================================ QKV
template <int H>
struct QkvCfg {
    typedef Shape<H> S;
    // hidden 512: two column slices, as in the MLP (2.05 -> 1.57 ms per 2048 members x 512 tokens against four)
    static constexpr int CS = H == 512 ? 2 : S::CS;
    static constexpr int TPW = EGG_WAVES / CS, HS = H / CS, NTS = HS / 32, KS = S::KS;
    static constexpr int PR = (H / 16) < (1024 / H) ? (H / 16) : (1024 / H), NU = (H / 16) / PR;   // p-rows per unit, units per matrix
    static constexpr int UNIT = 16 * PR * H;
    static constexpr int WBYTES = 2 * UNIT;
    // lnw lnb (int32) | qA kA vA (int32, times the sign: an operand of the multiply without a byte extraction) | qB kB vB (int8)
    static constexpr int PER_SET = 5 * H * 4 + 3 * H;
    static constexpr int XCHG = 0;             // the normalised input is exchanged through the idle W buffer
    static constexpr int SITE = EGG_WAVES * 64;
    static constexpr int RED = CS > 1 ? 2 * SITE * 4 : 0;       // two reduction sites used alternately
    static constexpr int OCC = H == 256 ? 3 : 2;               // workgroups per CU the kernel is built for
    static int total(int sets) { return WBYTES + sets * PER_SET + XCHG + RED; }
};

// apply_rope_integer (mgpu.cu:624-644) on the raw accumulators of one token.  The (cos, sin) pairs repeat every
// head, so a lane needs only the head_dim/32 * 8 pairs of its own slots.
// The reference evaluates (ve*c -+ vo*s + 2^(bit-1)) >> bit in int64, and so does this code: 64-bit multiply-adds
// (v_mad_i64_i32, full rate on gfx950); the shifted result fits 32 bits like the reference's AccumType.
// The NT column groups must start at a head boundary.  The
// pairs are read where they are used (one 16-byte load per two pairs, cache hits): holding a token's 16 pairs in
// registers across the three projections costs the 32 registers that separate two from three workgroups per CU.
template <int NT>
__device__ __forceinline__ void rope_inplace(v16i *acc, const int32_t *rope_row, int head_dim, int g, int bit) {
    const int hdt = head_dim >> 5;
    const long long half = 1ll << (bit - 1);
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int n = 32 * (hdt == 2 ? (nt & 1) : 0) + 8 * q + 4 * g;
            const v4i cs = *reinterpret_cast<const v4i *>(rope_row + n);        // c0 s0 c1 s1
#pragma unroll
            for (int ep = 0; ep < 2; ep++) {
                const int cc = cs[2 * ep], ss = cs[2 * ep + 1];
                const int ve = acc[nt][4 * q + 2 * ep], vo = acc[nt][4 * q + 2 * ep + 1], nvo = -vo;
                const long long re = (long long)nvo * ss + ((long long)ve * cc + half);
                const long long ro = (long long)vo * cc + ((long long)ve * ss + half);
                acc[nt][4 * q + 2 * ep] = (int)__builtin_amdgcn_alignbit((unsigned)(re >> 32), (unsigned)re, (unsigned)bit);
                acc[nt][4 * q + 2 * ep + 1] = (int)__builtin_amdgcn_alignbit((unsigned)(ro >> 32), (unsigned)ro, (unsigned)bit);
            }
        }
}

// ADAPT: the d-eggs adaptive noise overlay is on (de/include/model/layers.cuh:313-351): output-side noise and vector
// noise are scaled when the per-member tables are filled, the input-side sums take the slow term-by-term form.
template <int H, bool ADAPT>
__global__ void __launch_bounds__(EGG_THREADS, ADAPT ? 2 : QkvCfg<H>::OCC) k_qkv(QkvParams p) {
    typedef QkvCfg<H> Q;
    constexpr int CS = Q::CS, KS = Q::KS, NTS = Q::NTS, HS = Q::HS;
    extern __shared__ __align__(16) int8_t smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const FwdCommon &c = p.c;
    const int T = c.T;
    const TileMap tm = tile_map<CS>(c.tn, wave, blockIdx.x);
    const int col0 = tm.cs * HS;
    int8_t *tb = smem + Q::WBYTES + tm.set * Q::PER_SET;
    int *lnw = reinterpret_cast<int *>(tb), *lnb = lnw + H;
    int *qA = lnb + H, *kA = qA + H, *vA = kA + H;
    int8_t *qB = reinterpret_cast<int8_t *>(vA + H), *kB = qB + H, *vB = kB + H;
    int8_t *xch = smem + Q::WBYTES + tm.sets * Q::PER_SET;
    int *red = reinterpret_cast<int *>(xch + Q::XCHG);

    WStream ws; wstream_init(ws, smem, Q::UNIT);
    const DmaPlan<Q::PR, H> plan = dma_plan<Q::PR, H>(H);
    auto pf = [&](const int8_t *W, int u) { w_prefetch2<Q::PR, H>(ws, W + (size_t)u * Q::PR * H * 16, plan); };
    pf(p.w_q, 0);

    for (int ss = 0; ss < tm.sets; ss++) {
        int ml = blockIdx.x * tm.sets + ss; if (ml >= c.n_members) ml = c.n_members - 1;
        const int mem = c.pop_offset + ml, nsx = (mem & 1) ? -1 : 1;
        const uint32_t sbx = *c.d_step_seed + (uint32_t)(mem / 2) + (uint32_t)p.seed_base;
        int8_t *t2 = smem + Q::WBYTES + ss * Q::PER_SET;
        int *lw = reinterpret_cast<int *>(t2), *lb = lw + H;
        int *a0 = lb + H, *a1 = a0 + H, *a2 = a1 + H;
        int8_t *b0 = reinterpret_cast<int8_t *>(a2 + H), *b1 = b0 + H, *b2 = b1 + H;
        const int tid = threadIdx.x;
        if (ADAPT) {
            fill_vec_i32_ov(lw, p.ln_w, sbx + OFF_LN_1_A, sbx + OFF_LN_1_B, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 2, p.q_ln_w);
            fill_vec_i32_ov(lb, p.ln_b, sbx + OFF_LN_1_BIAS_A, sbx + OFF_LN_1_BIAS_B, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 0, p.q_ln_b);
            fill_noise_i32_ov(a0, sbx + OFF_Q_A, H, c.mask, nsx, tid, EGG_THREADS, p.q_wq + H);
            fill_noise_i32_ov(a1, sbx + OFF_K_A, H, c.mask, nsx, tid, EGG_THREADS, p.q_wk + H);
            fill_noise_i32_ov(a2, sbx + OFF_V_A, H, c.mask, nsx, tid, EGG_THREADS, p.q_wv + H);
        } else {
            fill_vec_i32(lw, p.ln_w, sbx + OFF_LN_1_A, sbx + OFF_LN_1_B, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS, 2);     // 4 * gain, see standard_scale
            fill_vec_i32(lb, p.ln_b, sbx + OFF_LN_1_BIAS_A, sbx + OFF_LN_1_BIAS_B, H, c.mask, nsx, c.sigma_vec, tid, EGG_THREADS);
            fill_noise_i32(a0, sbx + OFF_Q_A, H, c.mask, nsx, tid, EGG_THREADS);
            fill_noise_i32(a1, sbx + OFF_K_A, H, c.mask, nsx, tid, EGG_THREADS);
            fill_noise_i32(a2, sbx + OFF_V_A, H, c.mask, nsx, tid, EGG_THREADS);
        }
        fill_noise_i8(b0, sbx + OFF_Q_B, H, c.mask, tid, EGG_THREADS);
        fill_noise_i8(b1, sbx + OFF_K_B, H, c.mask, tid, EGG_THREADS);
        fill_noise_i8(b2, sbx + OFF_V_B, H, c.mask, tid, EGG_THREADS);
    }
    __syncthreads();

    int mloc = tm.mloc;
    const bool valid = mloc < c.n_members;
    if (!valid) mloc = c.n_members - 1;

    for (int pass = 0; pass < tm.passes; pass++) {
        const int t = c.t0 + (tm.tile0 + Q::TPW * pass) * 32 + j;
        const size_t row = ((size_t)mloc * T + t) * H;
        v4i nrm[KS];
        {
            v4i x[NTS];
#pragma unroll
            for (int nt = 0; nt < NTS; nt++) x[nt] = load_op(p.x + row + col0, nt, g);
            int tot = sumabs_groups<NTS>(x);
            tot = sum_halves(tot);
            tot = xreduce<CS, false>(tot, red, tm, lane);        // sites alternate 0,1,0,1 through the pass
            int mn = tot / H; if (!mn) mn = 1;
            if constexpr (CS == 1) standard_scale<NTS>(x, nrm, mn, lnw, lnb, 0, g);
            else {
                v4i mine[NTS];
                standard_scale<NTS>(x, mine, mn, lnw, lnb, col0, g);
                exchange_operand<CS, NTS, KS, Q::TPW, Q::UNIT>(ws.other, tm, lane, mine, nrm);
            }
        }
#pragma unroll 1
        for (int which = 0; which < 3; which++) {
            const int8_t *W = which == 0 ? p.w_q : (which == 1 ? p.w_k : p.w_v);
            const int8_t *nw = which == 0 ? p.w_k : (which == 1 ? p.w_v : ((pass + 1 < tm.passes) ? p.w_q : nullptr));
            const int8_t *Bn = which == 0 ? qB : (which == 1 ? kB : vB);
            const int *An = which == 0 ? qA : (which == 1 ? kA : vA);
            int8_t *dst = which == 0 ? p.q : (which == 1 ? p.k : p.v);
            const int sb = ADAPT ? dot_noise_ov<KS, false>(nrm, Bn, which == 0 ? p.q_wq : (which == 1 ? p.q_wk : p.q_wv), 0, g)
                                 : dot_noise<KS, false>(nrm, Bn, 0, g);
            v16i acc[NTS];
            zero_acc<NTS>(acc);
#pragma unroll
            for (int u = 0; u < Q::NU; u++) {
                const int8_t *cur = w_acquire(ws);
                if (u + 1 < Q::NU) pf(W, u + 1);
                else if (nw) pf(nw, 0);
                mfma_cols<Q::PR / 2, NTS>(acc, nrm + u * (Q::PR / 2), cur, H, col0, lane);
            }
            add_perturb<NTS>(acc, sb, An, col0, c.sigma, g);
            if (which < 2) rope_inplace<NTS>(acc, c.rope_lut + (size_t)t * c.head_dim, c.head_dim, g, c.rope_scale_bit);
            const int mx = xreduce<CS, true>(absmax_to_float_groups<NTS>(acc), red + ((1 + which) & 1) * Q::SITE, tm, lane);
            v4i o[NTS];
            adaptive_scale_floats<NTS>(acc, mx, o);
            if (valid)
#pragma unroll
                for (int nt = 0; nt < NTS; nt++) store_op(dst + row + col0, nt, g, o[nt]);
        }
    }
}

// ============================================================================ attention core
// One wave per (member, head).  S^T = K.Q^T per 32x32 tile (lane = query token), two passes over the
// causal context (row max, then LUT weights), O^T = V^T.P^T with the 19-bit weights split into three
// 7-bit planes so the weighted sum stays exact on the int8 MFMA.  The LDS table holds, per exp-LUT index,
// the three planes packed as bytes (4-byte entries: the gathers are what loads the LDS pipe), so the planes of four
// context positions are regrouped with byte permutes instead of shifts and masks; the sum of the weights is rebuilt
// from per-plane byte sums.  Only the diagonal tile needs the causal mask.
// den[pl] accumulates the plane sums; the sum of the weights is den[0] + 128 den[1] + 16384 den[2] (attn_den).
// Workgroups go to the eight XCDs (each with an L2 of its own) in turn: block b runs on XCD b % 8.  The heads of a member
// read 64-byte (or 32-byte) pieces of the same 128-byte lines of its Q, K and V rows, so they should meet in one L2: the
// blocks of one XCD, in launch order, take consecutive (member, head) units.  Needs a grid that is a multiple of eight;
// any other grid keeps the plain order.
__device__ __forceinline__ int xcd_contiguous_unit(int block, int nblocks) {
    if (nblocks & 7) return block;
    return (block & 7) * (nblocks >> 3) + (block >> 3);
}
// `last4` is four times the last table index a lookup may use: the index of the first entry from which the table is zero to
// its end (255 if the last entry is not zero).  Indices beyond it would read zeros anyway, and sending them all to one
// entry turns most of a wave's gather into a broadcast instead of a spread over the LDS banks.  `mxs4` is four times
// the shifted maximum: the byte offset 4 * (mxs - (s >> shift)) is one 24-bit multiply-add away from the shifted score.
__device__ __forceinline__ int attn_lut_last4(const int32_t *exp_lut, int *spare, int wave, int lane) {
    // last nonzero entry over the 256 threads of the workgroup (every thread looks at its own entry)
    const unsigned long long nz = __ballot(exp_lut[threadIdx.x & 255] != 0);
    if (lane == 0) spare[wave] = nz ? 64 * wave + 63 - __builtin_clzll(nz) : -1;
    __syncthreads();
    int last = -1;
#pragma unroll
    for (int w = 0; w < EGG_WAVES; w++) last = max(last, spare[w]);
    return 4 * min(last + 1, 255);
}
__device__ __forceinline__ void attn_weights(const v16i &s, const int *lut, int mxs4, int last4, int shift, bool diag, int ct, int t, int g,
                                             v4i *pw, int *den) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
        int pk[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            // spelt out: the compiler turns the multiply into a shift and a subtraction and the clamp into two instructions
            int off;
            asm("v_mad_i32_i24 %0, %1, -4, %2\n\tv_med3_i32 %0, %0, 0, %3" : "=&v"(off) : "v"(s[4 * q + e] >> shift), "v"(mxs4), "v"(last4));
            pk[e] = *reinterpret_cast<const int *>(reinterpret_cast<const int8_t *>(lut) + off);
            // on the diagonal tile (ct == t / 32) the position 32 ct + 8q + 4g + e lies behind the query's when 8q + 4g + e > t % 32,
            // which depends on the lane and the register only
            if (diag && (8 * q + 4 * g + e) > (t & 31)) pk[e] = 0;
        }
        // bytes of pk[e]: plane0, plane1, plane2, 0  ->  one dword per plane holding the four positions
        const int ab_lo = __builtin_amdgcn_perm(pk[1], pk[0], 0x05010400);   // a0 b0 a1 b1
        const int cd_lo = __builtin_amdgcn_perm(pk[3], pk[2], 0x05010400);
        const int ab_hi = __builtin_amdgcn_perm(pk[1], pk[0], 0x07030602);   // a2 b2 a3 b3
        const int cd_hi = __builtin_amdgcn_perm(pk[3], pk[2], 0x07030602);
        pw[0][q] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100);
        pw[1][q] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302);
        pw[2][q] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100);
#pragma unroll
        for (int pl = 0; pl < 3; pl++) den[pl] = dot4(pw[pl][q], 0x01010101, den[pl]);
    }
}
__device__ __forceinline__ int attn_den(const int *den) { return den[0] + (den[1] << 7) + (den[2] << 14); }

template <int HD, int CT>
__global__ void __launch_bounds__(EGG_THREADS, (CT > 8 ? 1 : 2)) k_attn(AttnParams p) {
    constexpr int KS = HD / 32, DT = HD / 32;
    constexpr int T = CT * 32;
    extern __shared__ __align__(16) int8_t smem[];
    int *lut = reinterpret_cast<int *>(smem);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    int8_t *vl = smem + 2048 + (size_t)wave * 2 * T * HD;      // per wave: rows (V, then K) | Q rows
    int8_t *ql = vl + T * HD;

    const FwdCommon &c = p.c;
    const int H = c.H, NH = H / HD;
    int unit = blockIdx.x * EGG_WAVES + wave;
    const bool valid = unit < c.n_members * NH;
    if (!valid) unit = c.n_members * NH - 1;
    const int mloc = unit / NH, h = unit % NH;
    const size_t base = (size_t)mloc * T * H + (size_t)h * HD;

    for (int i = threadIdx.x; i < 256; i += EGG_THREADS) {
        const int w = c.exp_lut[i];
        lut[i] = (w & 127) | (((w >> 7) & 127) << 8) | ((w >> 14) << 16);
    }
    const int last4 = attn_lut_last4(c.exp_lut, lut + 256, wave, lane);
    // All three row sets of this (member, head) are requested at once, so the wave waits for global memory once: the K
    // rows stay in registers until the V rows have left the row area, the Q rows go to LDS in the K rows' layout
    // (chunk c of row r at c ^ ((r / RPL) % CH), see below), the V rows to LDS rows [ctx][HD].
    constexpr int CH = HD / 16, RPL = 128 / HD, PER = T * CH / 64;
    v4i kreg[PER];
    {
        v4i qreg[PER], vreg[PER];
#pragma unroll
        for (int n = 0; n < PER; n++) {
            const int i = lane + n * 64, cx = i / CH, part = i % CH;
            kreg[n] = *reinterpret_cast<const v4i *>(p.k + base + (size_t)cx * H + part * 16);
            qreg[n] = *reinterpret_cast<const v4i *>(p.q + base + (size_t)cx * H + part * 16);
            vreg[n] = *reinterpret_cast<const v4i *>(p.v + base + (size_t)cx * H + part * 16);
        }
#pragma unroll
        for (int n = 0; n < PER; n++) {
            const int i = lane + n * 64, cx = i / CH, part = i % CH;
            *reinterpret_cast<v4i *>(vl + (size_t)cx * HD + part * 16) = vreg[n];
            *reinterpret_cast<v4i *>(ql + (size_t)cx * HD + ((part ^ ((cx / RPL) % CH)) * 16)) = qreg[n];
        }
    }
    __syncthreads();
    // V^T fragments: A-operand row i = natural head dim d = 32dt + i, stored at slot position 16g'+4q'+e'
    v4i vt[CT][DT];
    {
        const int pos = ((j >> 2) & 1) * 16 + (j >> 3) * 4 + (j & 3);
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int b[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) b[e] = vl[(size_t)(32 * ct + 8 * q + 4 * g + e) * HD + 32 * dt + pos];
                    vt[ct][dt][q] = pack4(b[0], b[1], b[2], b[3]);
                }
    }

    // the V rows are no longer needed once their transposed fragments sit in registers: the wave's LDS region now
    // takes the K rows of this (member, head), which every query tile re-reads twice per context tile
    // Rows are HD bytes apart, so the 16-byte chunk a lane reads (row = its context position) would hit the same few
    // banks for every row; chunk c of row r is therefore kept at position c ^ ((r / RPL) % CH), which spreads eight
    // consecutive rows over all banks.
    wave_lds_fence();
#pragma unroll
    for (int n = 0; n < PER; n++) {
        const int i = lane + n * 64, cx = i / CH, part = i % CH;
        *reinterpret_cast<v4i *>(vl + (size_t)cx * HD + ((part ^ ((cx / RPL) % CH)) * 16)) = kreg[n];
    }
    wave_lds_fence();
    const int8_t *kl = vl;
    auto k_frag = [&](int ct, int ks) {
        const int r = 32 * ct + j;
        return *reinterpret_cast<const v4i *>(kl + (size_t)r * HD + (((ks * 2 + g) ^ ((r / RPL) % CH)) * 16));
    };

#pragma unroll 1
    for (int qt = c.t0 >> 5; qt < ((c.t0 + c.tn) >> 5); qt++) {
        const int t = qt * 32 + j;
        v4i qop[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            qop[ks] = *reinterpret_cast<const v4i *>(ql + (size_t)t * HD + (((ks * 2 + g) ^ ((t / RPL) % CH)) * 16));
        // pass 1: per-head maximum score over ctx <= t (mgpu.cu:795-802)
        int mx = INT_MIN;
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
            if (ct <= qt) {
                v16i s;
#pragma unroll
                for (int r = 0; r < 16; r++) s[r] = 0;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    v4i kf = k_frag(ct, ks);
                    s = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qop[ks], s, 0, 0, 0);
                }
                if (ct == qt) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        int cx = 32 * ct + ((r >> 2) << 3) + (g << 2) + (r & 3);
                        if (cx <= t) mx = max(mx, s[r]);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r += 2) mx = max(max(mx, s[r]), s[r + 1]);
                }
            }
        }
        mx = max_halves(mx);
        const int mxs = mx >> c.shift_attn;
        // pass 2: weights and weighted V sum (mgpu.cu:810-824)
        v16i o[3][DT];
#pragma unroll
        for (int pl = 0; pl < 3; pl++) zero_acc<DT>(o[pl]);
        int dpl[3] = {0, 0, 0};
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
            if (ct <= qt) {
                v16i s;
#pragma unroll
                for (int r = 0; r < 16; r++) s[r] = 0;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    v4i kf = k_frag(ct, ks);
                    s = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qop[ks], s, 0, 0, 0);
                }
                v4i pw[3];
                if (ct == qt) attn_weights(s, lut, 4 * mxs, last4, c.shift_attn, true, ct, t, g, pw, dpl);
                else attn_weights(s, lut, 4 * mxs, last4, c.shift_attn, false, ct, t, g, pw, dpl);
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int pl = 0; pl < 3; pl++)
                        o[pl][dt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vt[ct][dt], pw[pl], o[pl][dt], 0, 0, 0);
            }
        }
        int den = attn_den(dpl);
        den = sum_halves(den);
        // Truncating quotient num / den with one reciprocal per token.  num and den are integers below 2^53, the
        // quotient is at most 127 in magnitude, and a non-integer quotient is at least 1/den >= 2^-27 away from
        // the next integer.  Scaling the reciprocal by (1 + 2^-40) pushes an exactly integer quotient k to
        // k(1 + 2^-40 +- 2^-51), which truncates to k, and moves any other quotient by less than 2^-32.
        const double rden = (1.0 + 0x1p-40) / (double)(den ? den : 1);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            v4i outp;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int ov[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int r = 4 * q + e;
                    // planes 0 and 1 combine in int32 (127*127*T + 127*127*T*128 < 2^31 for T <= 512)
                    const int lo = o[0][dt][r] + (o[1][dt][r] << 7);
                    double num = __builtin_fma((double)o[2][dt][r], 16384.0, (double)lo);
                    ov[e] = clip127((int)(num * rden));
                }
                outp[q] = pack4(ov[0], ov[1], ov[2], ov[3]);
            }
            if (valid) store_op(p.ao + base + (size_t)t * H, dt, g, outp);
        }
    }
}

// The same attention for long sequences (at least 8 tiles): one workgroup per (member, head).  The K rows and the
// transposed V fragments are built once in LDS and shared by the four waves, which split the query tiles so that
// the causal work is balanced (wave w takes tiles w and 7 - w of every group of eight).  Keeping the V fragments in
// LDS instead of registers leaves room for more resident waves.
template <int HD, int CT>
struct AttnWg {
    static constexpr int T = CT * 32, ROWS = T * HD;               // bytes of one K or V head tile
    // The Q rows of all query tiles go through LDS as well when three workgroups per CU still fit; otherwise (sequence
    // 512) every query tile loads its operand from global memory and two workgroups share a CU.
    static constexpr bool QLDS = 3 * (2048 + 3 * ROWS) <= 160 * 1024;
    static constexpr int LDS = 2048 + (QLDS ? 3 : 2) * ROWS;       // LUT | rows (V, then K) | V^T fragments | Q rows
    static constexpr int OCC = QLDS ? 3 : (2 * LDS <= 160 * 1024 ? 2 : 1);    // workgroups per CU the kernel is built for
};
template <int HD, int CT>
__global__ void __launch_bounds__(EGG_THREADS, (AttnWg<HD, CT>::OCC)) k_attn_wg(AttnParams p) {
    constexpr int KS = HD / 32, DT = HD / 32, T = CT * 32, CH = HD / 16, RPL = 128 / HD;
    static_assert(CT % 8 == 0, "query tiles are dealt in groups of eight");
    extern __shared__ __align__(16) int8_t smem[];
    int *lut = reinterpret_cast<int *>(smem);
    int8_t *rows = smem + 2048;
    int8_t *vfrag = rows + AttnWg<HD, CT>::ROWS;
    int8_t *qrows = vfrag + AttnWg<HD, CT>::ROWS;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    const FwdCommon &c = p.c;
    const int H = c.H, NH = H / HD;
    const int unit = xcd_contiguous_unit(blockIdx.x, gridDim.x);   // grid = n_members * heads exactly
    const int mloc = unit / NH, h = unit % NH;
    const size_t base = (size_t)mloc * T * H + (size_t)h * HD;

    for (int i = threadIdx.x; i < 256; i += EGG_THREADS) {
        const int w = c.exp_lut[i];
        lut[i] = (w & 127) | (((w >> 7) & 127) << 8) | ((w >> 14) << 16);
    }
    const int last4 = attn_lut_last4(c.exp_lut, lut + 256, wave, lane);
    // the K rows are requested now and held in registers until the V rows have left the shared row area, so that their
    // latency overlaps the V stage instead of following it
    constexpr int PER = T * CH / EGG_THREADS;
    static_assert(T * CH % EGG_THREADS == 0, "row chunks are dealt evenly to the threads");
    v4i kreg[PER];
#pragma unroll
    for (int n = 0; n < PER; n++) {
        const int i = threadIdx.x + n * EGG_THREADS, cx = i / CH, part = i % CH;
        kreg[n] = *reinterpret_cast<const v4i *>(p.k + base + (size_t)cx * H + part * 16);
    }
    // Q rows -> LDS in the K rows' layout (every wave reads its query tiles from there: one round of global latency
    // for the whole workgroup instead of one per query tile), V rows of this (member, head) -> LDS [ctx][HD]
    {
        constexpr bool QLDS = AttnWg<HD, CT>::QLDS;
        v4i qreg[QLDS ? PER : 1], vreg[PER];
#pragma unroll
        for (int n = 0; n < PER; n++) {
            const int i = threadIdx.x + n * EGG_THREADS, cx = i / CH, part = i % CH;
            if constexpr (QLDS) qreg[n] = *reinterpret_cast<const v4i *>(p.q + base + (size_t)cx * H + part * 16);
            vreg[n] = *reinterpret_cast<const v4i *>(p.v + base + (size_t)cx * H + part * 16);
        }
#pragma unroll
        for (int n = 0; n < PER; n++) {
            const int i = threadIdx.x + n * EGG_THREADS, cx = i / CH, part = i % CH;
            *reinterpret_cast<v4i *>(rows + (size_t)cx * HD + part * 16) = vreg[n];
            if constexpr (QLDS) *reinterpret_cast<v4i *>(qrows + (size_t)cx * HD + ((part ^ ((cx / RPL) % CH)) * 16)) = qreg[n];
        }
    }
    __syncthreads();
    // V^T fragments: A-operand row i = natural head dim d = 32dt + i, stored at slot position 16g'+4q'+e'
    {
        const int pos = ((j >> 2) & 1) * 16 + (j >> 3) * 4 + (j & 3);
        for (int f = wave; f < CT * DT; f += EGG_WAVES) {
            const int ct = f / DT, dt = f % DT;
            v4i frag;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int b[4];
#pragma unroll
                for (int e = 0; e < 4; e++) b[e] = rows[(size_t)(32 * ct + 8 * q + 4 * g + e) * HD + 32 * dt + pos];
                frag[q] = pack4(b[0], b[1], b[2], b[3]);
            }
            *reinterpret_cast<v4i *>(vfrag + ((size_t)f * 64 + lane) * 16) = frag;
        }
    }
    __syncthreads();
    // K rows take the place of the V rows; chunk c of row r sits at c ^ ((r / RPL) % CH) to spread the banks
#pragma unroll
    for (int n = 0; n < PER; n++) {
        const int i = threadIdx.x + n * EGG_THREADS, cx = i / CH, part = i % CH;
        *reinterpret_cast<v4i *>(rows + (size_t)cx * HD + ((part ^ ((cx / RPL) % CH)) * 16)) = kreg[n];
    }
    __syncthreads();
    auto score_tile = [&](int ct, const v4i *qop) {
        v16i s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0;
        const int r = 32 * ct + j;
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            v4i kf = *reinterpret_cast<const v4i *>(rows + (size_t)r * HD + (((ks * 2 + g) ^ ((r / RPL) % CH)) * 16));
            s = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qop[ks], s, 0, 0, 0);
        }
        __builtin_amdgcn_s_setprio(0);
        return s;
    };

#pragma unroll 1
    for (int qi = 0; qi < CT / 4; qi++) {
        const int qt = (qi >> 1) * 8 + ((qi & 1) ? 7 - wave : wave);
        if (qt * 32 < c.t0 || qt * 32 >= c.t0 + c.tn) continue;      // (wave-uniform; the loop holds no barrier)
        const int t = qt * 32 + j;
        v4i qop[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            if constexpr (AttnWg<HD, CT>::QLDS)
                qop[ks] = *reinterpret_cast<const v4i *>(qrows + (size_t)t * HD + (((ks * 2 + g) ^ ((t / RPL) % CH)) * 16));
            else qop[ks] = load_op(p.q + base + (size_t)t * H, ks, g);
        }
        // pass 1: per-head maximum score over ctx <= t (mgpu.cu:795-802)
        // (both passes issue the score MFMAs of the next context tile before they work on the current one)
        int mx = INT_MIN;
        {
            v16i s = score_tile(0, qop);
#pragma unroll 2
            for (int ct = 0; ct < qt; ct++) {
                const v16i sn = score_tile(ct + 1, qop);
#pragma unroll
                for (int r = 0; r < 16; r += 2) mx = max(max(mx, s[r]), s[r + 1]);
                s = sn;
            }
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int cx = ((r >> 2) << 3) + (g << 2) + (r & 3);      // position within the diagonal tile
                if (cx <= j) mx = max(mx, s[r]);
            }
        }
        mx = max_halves(mx);
        const int mxs = mx >> c.shift_attn;
        // pass 2: weights and weighted V sum (mgpu.cu:810-824).  The first tile weighed starts the accumulators (a zero C
        // operand instead of 96 cleared registers); the scores of the next tile are in flight while a tile is weighed.
        v16i o[3][DT];
        int dpl[3] = {0, 0, 0};
        const int mxs4 = 4 * mxs;
        auto weigh_tile = [&](const v16i &s, int ct, bool diag, bool first) {      // diag and first are constants at every call
            v4i pw[3];
            attn_weights(s, lut, mxs4, last4, c.shift_attn, diag, ct, t, g, pw, dpl);
            v16i z;
#pragma unroll
            for (int r = 0; r < 16; r++) z[r] = 0;
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                const v4i vt = *reinterpret_cast<const v4i *>(vfrag + ((size_t)(ct * DT + dt) * 64 + lane) * 16);
#pragma unroll
                for (int pl = 0; pl < 3; pl++) o[pl][dt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vt, pw[pl], first ? z : o[pl][dt], 0, 0, 0);
            }
            __builtin_amdgcn_s_setprio(0);
        };
        {
            // integer sums do not depend on the order: the diagonal tile goes first and starts the accumulators
            v16i s = score_tile(qt, qop);
            v16i sn = score_tile(0, qop);
            weigh_tile(s, qt, true, true);
            s = sn;
#pragma unroll 1
            for (int ct = 0; ct < qt; ct++) {
                sn = score_tile(ct + 1 < qt ? ct + 1 : ct, qop);       // (the last one is not used)
                weigh_tile(s, ct, false, false);
                s = sn;
            }
        }
        int den = attn_den(dpl);
        den = sum_halves(den);
        // truncating quotient with one reciprocal per token, see k_attn
        const double rden = (1.0 + 0x1p-40) / (double)(den ? den : 1);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            v4i outp;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int ov[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int r = 4 * q + e;
                    const int lo = o[0][dt][r] + (o[1][dt][r] << 7);
                    double num = __builtin_fma((double)o[2][dt][r], 16384.0, (double)lo);
                    ov[e] = clip127((int)(num * rden));
                }
                outp[q] = pack4(ov[0], ov[1], ov[2], ov[3]);
            }
            store_op(p.ao + base + (size_t)t * H, dt, g, outp);
        }
    }
}

// ============================================================================ head + loss
template <int H>
struct HeadLds {
    static constexpr int PER_WAVE = (2 * H + 256) * 4 + H;   // lnw lnb hA[256] + hB[H]
    static constexpr int WBLOCK = 2 * WUnit<(H < 256 ? H : 256)>::BYTES;   // double-buffered W units
    static constexpr int TOTAL = WBLOCK + 1024 + EGG_WAVES * PER_WAVE;
};

// ADAPT: adaptive noise overlay; the tied head takes the embedding's per-hidden q values on its input side and the
// per-token values on its output side (de/src/kernels.cu:200-240)
// BIG: a vocabulary of more than 256 entries
template <int H, bool ADAPT, bool BIG>
__global__ void __launch_bounds__(EGG_THREADS, (H > 256 ? 1 : 2)) k_head(HeadParams p) {
    constexpr int KS = H / 32, NV = 256 / 32, BLK = H < 256 ? H : 256;
    extern __shared__ __align__(16) int8_t smem[];
    int8_t *wlds = smem;
    int *lut = reinterpret_cast<int *>(smem + HeadLds<H>::WBLOCK);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    int8_t *tb = smem + HeadLds<H>::WBLOCK + 1024 + wave * HeadLds<H>::PER_WAVE;
    int *lnw = reinterpret_cast<int *>(tb), *lnb = lnw + H, *hA = lnb + H;
    int8_t *hB = reinterpret_cast<int8_t *>(hA + 256);

    const FwdCommon &c = p.c;
    const int T = c.T;
    int mloc = blockIdx.x * EGG_WAVES + wave;
    const bool valid = mloc < c.n_members;
    if (!valid) mloc = c.n_members - 1;
    const int member = c.pop_offset + mloc;
    const int ns = (member & 1) ? -1 : 1;
    const uint32_t pair_seed = *c.d_step_seed + (uint32_t)(member / 2);

    // The vocabulary is taken in blocks of 256 columns.  One block (the byte-level model): the logits stay in registers
    // between the maximum and the sum.  More: like the reference (de/src/kernels.cu:233-272) the projection runs twice,
    // first for the maximum, then for the sum of the table weights and the target's logit; the output-side noise of a
    // block is rebuilt in front of it (noise(seed, 256 b + i) is the hash of seed + 256 b * 0x9e3779b9 at index i).
    const int V = BIG ? c.vocab : 256, nvb = BIG ? V >> 8 : 1;
    constexpr bool single = !BIG;
    WStream ws; wstream_init(ws, wlds, WUnit<BLK>::BYTES);
    w_prefetch<BLK>(ws, w_unit_ptr<BLK>(p.embedding_frag, V, 0, 0, 0));
    for (int i = threadIdx.x; i < 256; i += EGG_THREADS) lut[i] = c.exp_lut[i];
    if (ADAPT) {
        fill_vec_i32_ov(lnw, p.ln_w, pair_seed + OFF_LN_F_A, pair_seed + OFF_LN_F_B, H, c.mask, ns, c.sigma_vec, lane, 64, 2, p.q_ln_w);
        fill_vec_i32_ov(lnb, p.ln_b, pair_seed + OFF_LN_F_BIAS_A, pair_seed + OFF_LN_F_BIAS_B, H, c.mask, ns, c.sigma_vec, lane, 64, 0, p.q_ln_b);
    } else {
        fill_vec_i32(lnw, p.ln_w, pair_seed + OFF_LN_F_A, pair_seed + OFF_LN_F_B, H, c.mask, ns, c.sigma_vec, lane, 64, 2);   // 4 * gain, see standard_scale
        fill_vec_i32(lnb, p.ln_b, pair_seed + OFF_LN_F_BIAS_A, pair_seed + OFF_LN_F_BIAS_B, H, c.mask, ns, c.sigma_vec, lane);
    }
    if (single) {
        if (ADAPT) fill_noise_i32_ov(hA, pair_seed + OFF_EMB, 256, c.mask, ns, lane, 64, p.q_emb + H);
        else fill_noise_i32(hA, pair_seed + OFF_EMB, 256, c.mask, ns, lane);
    }
    fill_noise_i8(hB, pair_seed + OFF_EMB + H, H, c.mask, lane);
    __syncthreads();

    const int64_t spos = stream_pos_of(c, member);
    long long wave_loss = 0;
    const int pass_end = (c.t0 + c.tn) >> 5;
    for (int pass = c.t0 >> 5; pass < pass_end; pass++) {
        const int t = pass * 32 + j;
        const size_t row = ((size_t)mloc * T + t) * H;
        v4i x[KS], nf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) x[ks] = load_op(p.x + row, ks, g);
        standard_norm<KS>(x, nf, lnw, lnb, g);
        const int sbh = ADAPT ? dot_noise_ov<KS, false>(nf, hB, p.q_emb, 0, g) : dot_noise<KS, false>(nf, hB, 0, g);
        int gmax = INT_MIN, target;
        long long sum_ex; int tl;
        // two-pass softmax statistics (mgpu.cu:969-1009)
        if constexpr (single) {
            v16i acc[NV];
            zero_acc<NV>(acc);
            gemm_stream<H, 256, BLK>(acc, nf, p.embedding_frag, 256, 0, 0, ws, (pass + 1 < pass_end) ? w_unit_ptr<BLK>(p.embedding_frag, 256, 0, 0, 0) : nullptr, lane);
            add_perturb<NV>(acc, sbh, hA, 0, c.sigma, g);
#pragma unroll
            for (int nt = 0; nt < NV; nt++)
#pragma unroll
                for (int r = 0; r < 16; r++) { acc[nt][r] >>= c.shift_logit; gmax = max(gmax, acc[nt][r]); }
            gmax = max_halves(gmax);
            target = c.data[spos + t + 1];
            sum_ex = 0; tl = 0;
#pragma unroll
            for (int nt = 0; nt < NV; nt++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    int idx = min(255, max(0, gmax - acc[nt][r]));
                    sum_ex += lut[idx];
                    if (col_of(nt, r, g) == target) tl = acc[nt][r];
                }
            sum_ex = sum_halves64(sum_ex);
            tl = sum_halves(tl);
            if (p.logits_tap && valid)
#pragma unroll
                for (int nt = 0; nt < NV; nt++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        v4i o4;
#pragma unroll
                        for (int e = 0; e < 4; e++) o4[e] = acc[nt][4 * q + e];
                        *reinterpret_cast<v4i *>(p.logits_tap + ((size_t)mloc * T + t) * 256 + 32 * nt + 8 * q + 4 * g) = o4;
                    }
        } else {
            target = token_at(c, spos + t + 1);
            sum_ex = 0; tl = 0;
#pragma unroll 1
            for (int phase = 0; phase < 2; phase++) {
#pragma unroll 1
                for (int vb = 0; vb < nvb; vb++) {
                    {                                   // read behind the barriers of the product below, by this wave only
                        const uint32_t seed = pair_seed + OFF_EMB + (uint32_t)(vb * 256) * 0x9e3779b9u;
                        if (ADAPT) fill_noise_i32_ov(hA, seed, 256, c.mask, ns, lane, 64, p.q_emb + H + vb * 256);
                        else fill_noise_i32(hA, seed, 256, c.mask, ns, lane);
                    }
                    const bool last = vb + 1 == nvb && phase == 1;
                    const int8_t *next = !last ? w_unit_ptr<BLK>(p.embedding_frag, V, 0, (vb + 1 == nvb ? 0 : vb + 1) * 256, 0)
                                               : ((pass + 1 < pass_end) ? w_unit_ptr<BLK>(p.embedding_frag, V, 0, 0, 0) : nullptr);
                    v16i acc[NV];
                    zero_acc<NV>(acc);
                    gemm_stream<H, 256, BLK>(acc, nf, p.embedding_frag, V, 0, vb * 256, ws, next, lane);
                    add_perturb<NV>(acc, sbh, hA, 0, c.sigma, g);
                    if (phase == 0) {
#pragma unroll
                        for (int nt = 0; nt < NV; nt++)
#pragma unroll
                            for (int r = 0; r < 16; r++) { acc[nt][r] >>= c.shift_logit; gmax = max(gmax, acc[nt][r]); }
                        if (p.logits_tap && valid)
#pragma unroll
                            for (int nt = 0; nt < NV; nt++)
#pragma unroll
                                for (int q = 0; q < 4; q++) {
                                    v4i o4;
#pragma unroll
                                    for (int e = 0; e < 4; e++) o4[e] = acc[nt][4 * q + e];
                                    *reinterpret_cast<v4i *>(p.logits_tap + ((size_t)mloc * T + t) * V + vb * 256 + 32 * nt + 8 * q + 4 * g) = o4;
                                }
                    } else {
#pragma unroll
                        for (int nt = 0; nt < NV; nt++)
#pragma unroll
                            for (int r = 0; r < 16; r++) {
                                const int lg = acc[nt][r] >> c.shift_logit;
                                sum_ex += lut[min(255, max(0, gmax - lg))];
                                if (vb * 256 + col_of(nt, r, g) == target) tl = lg;
                            }
                    }
                }
                if (phase == 0) gmax = max_halves(gmax);
            }
        }
        if constexpr (!single) { sum_ex = sum_halves64(sum_ex); tl = sum_halves(tl); }
        // loss (mgpu.cu:1012-1024)
        long long log_sum = 0;
        if (sum_ex > 0) {
            int pos = 63 - __clzll((unsigned long long)sum_ex);      // floor(log2), same as the reference's shift ladder
            log_sum = ((long long)pos << 4) - ((long long)c.softmax_scale_bit << 4);
        }
        long long lt = (log_sum >> 1) + gmax - tl;
        if (g == 0) wave_loss += lt;
    }
    // sum over the wave's 32 tokens (lanes of half 0), then one atomic per member
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {
        int lo = __shfl_xor((int)(wave_loss & 0xffffffffll), off, 64);
        int hi = __shfl_xor((int)(wave_loss >> 32), off, 64);
        wave_loss += ((long long)hi << 32) | (unsigned int)lo;
    }
    if (lane == 0 && valid) atomicAdd(p.loss_acc + member, (unsigned long long)wave_loss);
}

// ============================================================================ host launchers
template <int H>
static hipError_t launch_mlp_h(const MlpParams &p, bool first, hipStream_t s) {
    const int sets = tile_map_sets(p.c.tn, MlpCfg<H>::CS);
    dim3 grid((p.c.n_members + sets - 1) / sets), block(EGG_THREADS);
    size_t lds = MlpCfg<H>::total(sets, first);
    // The up accumulator is seeded with (bias + 128 + noise) << shift_mlp_up (see the bias table), so its range is the
    // GEMM's plus that seed; the fused perturb-and-shift needs |acc| * 2^sigma + |sb * a| below 2^31 for it as well.
    const long long mag = egg_noise_magnitude(p.c.mask);
    const long long up_acc = egg_mlp_up_acc_bound(H, p.c.mask, p.c.sigma_vec, p.c.shift_mlp_up);
    const bool up_fits = p.c.sigma >= 0 && p.c.sigma < 31 && (up_acc << p.c.sigma) + (long long)H * 127 * mag * mag < (1LL << 31);
    const bool fuse = p.c.sigma <= 7 && mag <= 15 && up_fits;
    if (up_acc >= (1LL << 31)) return hipErrorInvalidValue;      // egg_ctx_create refuses such shifts
    if (p.q_ln_w) {      // adaptive noise overlay: one (unfused) variant
        if (first) hipLaunchKernelGGL((k_mlp<H, true, false, true>), grid, block, lds, s, p);
        else hipLaunchKernelGGL((k_mlp<H, false, false, true>), grid, block, lds, s, p);
        return hipGetLastError();
    }
    if (first) { if (fuse) hipLaunchKernelGGL((k_mlp<H, true, true, false>), grid, block, lds, s, p); else hipLaunchKernelGGL((k_mlp<H, true, false, false>), grid, block, lds, s, p); }
    else { if (fuse) hipLaunchKernelGGL((k_mlp<H, false, true, false>), grid, block, lds, s, p); else hipLaunchKernelGGL((k_mlp<H, false, false, false>), grid, block, lds, s, p); }
    return hipGetLastError();
}
hipError_t egg_launch_mlp(const MlpParams &p, bool first, hipStream_t s) {
    switch (p.c.H) {
        case 64: return launch_mlp_h<64>(p, first, s);
        case 128: return launch_mlp_h<128>(p, first, s);
        case 256: return launch_mlp_h<256>(p, first, s);
        case 512: return launch_mlp_h<512>(p, first, s);
        default: return hipErrorInvalidValue;
    }
}

template <int H>
static hipError_t launch_qkv_h(const QkvParams &p, hipStream_t s) {
    const int sets = tile_map_sets(p.c.tn, QkvCfg<H>::CS);
    dim3 grid((p.c.n_members + sets - 1) / sets), block(EGG_THREADS);
    size_t lds = QkvCfg<H>::total(sets);
    if (p.q_ln_w) hipLaunchKernelGGL((k_qkv<H, true>), grid, block, lds, s, p);
    else hipLaunchKernelGGL((k_qkv<H, false>), grid, block, lds, s, p);
    return hipGetLastError();
}
hipError_t egg_launch_qkv(const QkvParams &p, hipStream_t s) {
    switch (p.c.H) {
        case 64: return launch_qkv_h<64>(p, s);
        case 128: return launch_qkv_h<128>(p, s);
        case 256: return launch_qkv_h<256>(p, s);
        case 512: return launch_qkv_h<512>(p, s);
        default: return hipErrorInvalidValue;
    }
}

template <int HD, int CT>
static hipError_t launch_attn_t(const AttnParams &p, hipStream_t s) {
    int units = p.c.n_members * (p.c.H / HD);
    if constexpr (CT % 8 == 0) {
        const size_t lds_wg = AttnWg<HD, CT>::LDS;
        hipLaunchKernelGGL((k_attn_wg<HD, CT>), dim3(units), dim3(EGG_THREADS), lds_wg, s, p);
    } else {
        dim3 grid((units + EGG_WAVES - 1) / EGG_WAVES), block(EGG_THREADS);
        size_t lds = 2048 + (size_t)EGG_WAVES * 2 * CT * 32 * HD;
        hipLaunchKernelGGL((k_attn<HD, CT>), grid, block, lds, s, p);
    }
    return hipGetLastError();
}
template <int HD>
static hipError_t launch_attn_hd(const AttnParams &p, hipStream_t s) {
    switch (p.c.T / 32) {
        case 1: return launch_attn_t<HD, 1>(p, s);
        case 2: return launch_attn_t<HD, 2>(p, s);
        case 4: return launch_attn_t<HD, 4>(p, s);
        case 8: return launch_attn_t<HD, 8>(p, s);
        case 16: return launch_attn_t<HD, 16>(p, s);
        default: return hipErrorInvalidValue;
    }
}
hipError_t egg_launch_attn(const AttnParams &p, hipStream_t s) {
    switch (p.c.head_dim) {
        case 32: return launch_attn_hd<32>(p, s);
        case 64: return launch_attn_hd<64>(p, s);
        default: return hipErrorInvalidValue;
    }
}

template <int H>
static hipError_t launch_head_h(const HeadParams &p, hipStream_t s) {
    dim3 grid((p.c.n_members + EGG_WAVES - 1) / EGG_WAVES), block(EGG_THREADS);
    size_t lds = HeadLds<H>::TOTAL;
    if (p.c.vocab < 256 || p.c.vocab % 256) return hipErrorInvalidValue;
    if (p.c.vocab > 256) {
        if (p.q_ln_w) hipLaunchKernelGGL((k_head<H, true, true>), grid, block, lds, s, p);
        else hipLaunchKernelGGL((k_head<H, false, true>), grid, block, lds, s, p);
    } else if (p.q_ln_w) hipLaunchKernelGGL((k_head<H, true, false>), grid, block, lds, s, p);
    else hipLaunchKernelGGL((k_head<H, false, false>), grid, block, lds, s, p);
    return hipGetLastError();
}
hipError_t egg_launch_head(const HeadParams &p, hipStream_t s) {
    switch (p.c.H) {
        case 64: return launch_head_h<64>(p, s);
        case 128: return launch_head_h<128>(p, s);
        case 256: return launch_head_h<256>(p, s);
        case 512: return launch_head_h<512>(p, s);
        default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------- one-time LDS opt-in (not a stream operation,
// so it is done at context creation and never while a stream is capturing)
#define SET_LDS(kern, bytes) do { hipError_t e_ = hipFuncSetAttribute(reinterpret_cast<const void *>(&kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)); if (e_ != hipSuccess) return e_; } while (0)
// k_mlp reads its GELU table through LDS addresses that assume the dynamic LDS block starts at address 0, i.e. that the
// kernel has no static LDS in front of it; refuse to run if a build ever gives it some
template <typename K>
static hipError_t no_static_lds(K kern) {
    hipFuncAttributes a;
    hipError_t e = hipFuncGetAttributes(&a, reinterpret_cast<const void *>(kern));
    if (e != hipSuccess) return e;
    return a.sharedSizeBytes == 0 ? hipSuccess : hipErrorInvalidConfiguration;
}
template <int H>
static hipError_t prepare_h(int T) {
    // table sets per workgroup: the whole window's, or a single tile's (egg_generate evaluates one tile per new token)
    const int sets = std::max(tile_map_sets(T, QkvCfg<H>::CS), tile_map_sets(32, QkvCfg<H>::CS));
    const int msets = std::max(tile_map_sets(T, MlpCfg<H>::CS), tile_map_sets(32, MlpCfg<H>::CS));
    for (hipError_t e : {no_static_lds(&k_mlp<H, true, true, false>), no_static_lds(&k_mlp<H, false, true, false>),
                         no_static_lds(&k_mlp<H, true, false, false>), no_static_lds(&k_mlp<H, false, false, false>),
                         no_static_lds(&k_mlp<H, true, false, true>), no_static_lds(&k_mlp<H, false, false, true>)})
        if (e != hipSuccess) return e;
    SET_LDS((k_mlp<H, true, true, false>), MlpCfg<H>::total(msets, true));
    SET_LDS((k_mlp<H, false, true, false>), MlpCfg<H>::total(msets, false));
    SET_LDS((k_mlp<H, true, false, false>), MlpCfg<H>::total(msets, true));
    SET_LDS((k_mlp<H, false, false, false>), MlpCfg<H>::total(msets, false));
    SET_LDS((k_mlp<H, true, false, true>), MlpCfg<H>::total(msets, true));
    SET_LDS((k_mlp<H, false, false, true>), MlpCfg<H>::total(msets, false));
    SET_LDS((k_qkv<H, false>), QkvCfg<H>::total(sets));
    SET_LDS((k_qkv<H, true>), QkvCfg<H>::total(sets));
    SET_LDS((k_head<H, false, false>), HeadLds<H>::TOTAL);
    SET_LDS((k_head<H, true, false>), HeadLds<H>::TOTAL);
    SET_LDS((k_head<H, false, true>), HeadLds<H>::TOTAL);
    SET_LDS((k_head<H, true, true>), HeadLds<H>::TOTAL);
    return hipSuccess;
}
template <int HD, int CT>
static hipError_t prepare_attn() {
    if constexpr (CT % 8 == 0) SET_LDS((k_attn_wg<HD, CT>), (AttnWg<HD, CT>::LDS));
    else SET_LDS((k_attn<HD, CT>), 2048 + (size_t)EGG_WAVES * 2 * CT * 32 * HD);
    return hipSuccess;
}
template <int HD>
static hipError_t prepare_attn_hd(int ct) {
    switch (ct) {
        case 1: return prepare_attn<HD, 1>();
        case 2: return prepare_attn<HD, 2>();
        case 4: return prepare_attn<HD, 4>();
        case 8: return prepare_attn<HD, 8>();
        case 16: return prepare_attn<HD, 16>();
        default: return hipErrorInvalidValue;
    }
}
hipError_t egg_prepare_forward(int H, int head_dim, int T) {
    hipError_t e;
    switch (H) {
        case 64: e = prepare_h<64>(T); break;
        case 128: e = prepare_h<128>(T); break;
        case 256: e = prepare_h<256>(T); break;
        case 512: e = prepare_h<512>(T); break;
        default: return hipErrorInvalidValue;
    }
    if (e != hipSuccess) return e;
    return head_dim == 32 ? prepare_attn_hd<32>(T / 32) : (head_dim == 64 ? prepare_attn_hd<64>(T / 32) : hipErrorInvalidValue);
}
