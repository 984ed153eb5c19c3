// egg_linear_ws.hip -- the perturbed int8 linear layer (compute_linear_projection,
// full_cuda_train_transformer_adam_mgpu.cu:553-572) with W stationary in registers.
//
// One persistent workgroup per CU, one wave per SIMD, each wave with the whole register file (512 registers).  Wave w
// keeps the MFMA fragments of output columns [w*N/4, (w+1)*N/4) for all of K in registers (K * N / 4 bytes: 256 registers
// at K = N = 512), loaded once from the canonical blocked matrix; after that W costs no LDS and no L2 traffic.  Token
// tiles (32 rows of K bytes) stream HBM -> LDS through a ring of NSLOT slots with global_load_lds_dwordx4, NSLOT - 2
// tiles ahead of their use; all four waves read every fragment of a tile from LDS and a fragment read feeds N/128
// MFMAs.  The columns of W are dealt to the MFMA rows so that a lane's 16 int8 results of a column tile are 16
// consecutive columns of its token: they leave as one 16-byte store, without a transpose (the int32 form goes through a
// per-wave LDS transpose and leaves as full 128-byte lines).
//
// The loop is software-pipelined inside the wave: while the MFMAs of tile t run, the vector unit finishes tile t - 1
// (shift, rank-1 term, clip, pack, transpose) one slice per k-step, so the two accumulator sets alternate roles and the
// tile loop is unrolled twice.  The only workgroup barrier of a tile sits in the middle of its k-loop: it publishes tile
// t + 1 (whose copy was waited for just before), frees the slot of tile t - 1 for the next copy, and publishes the
// per-token noise dots of tile t; the first fragments of tile t + 1 are read before tile t's last MFMAs.
//
// LDS image of a tile: 1 KB blocks [row group rg = row/8][128-byte column block cb]; inside a block the 16-byte chunk
// (row r = row%8, chunk c = 2h + g: h = k-step within the block, g = lane half) sits at position r*8 + pp with
// pp = (2*(h ^ (r&3)) + (g ^ (r>>2))) ^ 2*((rg>>1)&1).  A copy instruction of wave w moves the eight 128-byte lines of
// rows 8w..8w+7 of one column block (fully coalesced).  A 128-bit LDS read serves 16 lanes per clock over 64 banks, in
// the groups (0-3, 12-15, 20-23, 24-27), (4-7, 8-11, 16-19, 28-31) and the same plus 32; in each group the two lanes
// that share r differ in (rg>>1)&1, so a fragment read (lane = row j, half g) touches 16 different 16-byte bank groups.
//
// Built with -mllvm -amdgpu-mfma-vgpr-form so that the accumulators live in the arch registers the vector unit reads
// and the resident W takes the 256 accumulation registers.
#include <type_traits>
#include "egg_device.h"
#include "egg_launch.h"

template <int K, int N>
struct PlinWS {
    static constexpr int KS = K / 32, NW = N / EGG_WAVES, NCT = NW / 32, CB = K / 128;
    static constexpr int TILE = 32 * K;
    static constexpr int NSLOT = K <= 256 ? 12 : 8;
    static constexpr int PF = 4;                                  // fragments read ahead of their MFMAs
    static constexpr int SLICES = NCT * 4;                        // epilogue slices of a tile: (column tile, q)
    static constexpr int NTAB = 3;                                // noise-table sets in rotation (member % 3)
    static constexpr int STAGE = 32 * 128;                        // per wave: 32 rows x 128 bytes
    static constexpr int OFF_B = NSLOT * TILE;                    // B noise, int8 [NTAB][K]
    static constexpr int OFF_A = OFF_B + NTAB * K;                // A noise * sign, int32 [wave][NTAB][NW]
    static constexpr int OFF_SB = OFF_A + NTAB * N * 4;           // partial noise dots, int32 [tile parity][wave][32 tokens]
    static constexpr int OFF_STAGE = OFF_SB + 2 * EGG_WAVES * 32 * 4;
    static constexpr int TOTAL = OFF_STAGE + EGG_WAVES * STAGE;
    static_assert(NW % 32 == 0 && K % 128 == 0 && KS % EGG_WAVES == 0, "shape");
    static_assert(K * NW <= 65536, "a wave's slice of W must fit 256 registers");
    static_assert(SLICES % KS == 0 || KS % SLICES == 0, "slices spread evenly over the k-steps");
    static_assert(TOTAL <= 160 * 1024, "LDS");
};

// (acc + ((sb * a) >> sigma)) >> shift; FUSE evaluates it as ((acc << sigma) + sb * a) >> (sigma + shift), the same
// value with one instruction less (the host selects it only when the sum cannot leave 32 bits)
template <bool FUSE>
__device__ __forceinline__ int ws_perturbed(int acc, int sb, int a, int sigma, int shift) {
    if (FUSE) return (int)(((unsigned)acc << sigma) + (unsigned)mul24(sb, a)) >> (sigma + shift);
    return (acc + (mul24(sb, a) >> sigma)) >> shift;
}
// bytes 0 of four values side by side
__device__ __forceinline__ int pack_bytes(int a, int b, int c, int d) {
    return (int)(__builtin_amdgcn_perm((unsigned)b, (unsigned)a, 0x0c0c0400u) | __builtin_amdgcn_perm((unsigned)d, (unsigned)c, 0x04000c0cu));
}

// bytes 1 of four values side by side
__device__ __forceinline__ int pack_bytes1(int a, int b, int c, int d) {
    return (int)(__builtin_amdgcn_perm((unsigned)b, (unsigned)a, 0x0c0c0501u) | __builtin_amdgcn_perm((unsigned)d, (unsigned)c, 0x05010c0cu));
}

// s_waitcnt vmcnt(n) for a run-time n (wave-uniform), n <= 63
__device__ __forceinline__ void wait_vmcnt_upto(int n) {
#define W_(c) case c: __builtin_amdgcn_s_waitcnt(0x0F70 | ((c) & 15) | (((c) >> 4) << 14)); break;
    switch (n) {
        W_(0) W_(1) W_(2) W_(3) W_(4) W_(5) W_(6) W_(7) W_(8) W_(9) W_(10) W_(11) W_(12) W_(13) W_(14) W_(15)
        W_(16) W_(17) W_(18) W_(19) W_(20) W_(21) W_(22) W_(23) W_(24) W_(25) W_(26) W_(27) W_(28) W_(29) W_(30) W_(31)
        W_(32) W_(33) W_(34) W_(35) W_(36) W_(37) W_(38) W_(39) W_(40) W_(41) W_(42) W_(43) W_(44) W_(45) W_(46) W_(47)
        W_(48) W_(49) W_(50) W_(51) W_(52) W_(53) W_(54) W_(55) W_(56) W_(57) W_(58) W_(59) W_(60) W_(61) W_(62)
        default: __builtin_amdgcn_s_waitcnt(0x0F70 | 15 | (3 << 14)); break;
    }
#undef W_
}

// MODE: 0 = the shared-weight product alone (no rank-1 term), 1 = perturbed, 2 = perturbed with the fused shift,
// 3 = the shared-weight product alone with int8 results and a shift of exactly 8: the accumulator is clamped where it
// stands (to [-127 * 256, 127 * 256 + 255]) and the result is its second byte, which the pack's byte permute picks,
// so the shift costs no instruction
template <int K, int N, bool OUT32, int MODE>
__global__ void __launch_bounds__(EGG_THREADS, 1) k_plinear_ws(PlinParams p) {
    typedef PlinWS<K, N> P;
    constexpr bool PLAIN = MODE == 0 || MODE == 3, FUSE = MODE == 2, BYTE1 = MODE == 3;
    static_assert(!(BYTE1 && OUT32), "the byte-pick form packs int8 results");
    constexpr int KS = P::KS, NCT = P::NCT, NW = P::NW, CB = P::CB, NSLOT = P::NSLOT, PF = P::PF, NTAB = P::NTAB;
    constexpr int STORES = OUT32 ? NCT * 4 : NCT;                 // global store instructions per tile and wave
    constexpr int MID = KS / 2;                                   // k-step in front of which the tile's barrier sits
    constexpr int QS = KS / EGG_WAVES;                            // k-steps of a tile whose x.B share a wave computes
    static_assert(QS <= MID && PF <= KS - MID && NCT == 4 && KS % PF == 0 && CB <= NCT && MID + 1 < KS, "pipeline shape");
    extern __shared__ __align__(16) int8_t smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, g = lane >> 5, j = lane & 31;
    int8_t *Btab = smem + P::OFF_B;
    int *Atab = reinterpret_cast<int *>(smem + P::OFF_A) + wave * NTAB * NW;
    int *sbx = reinterpret_cast<int *>(smem + P::OFF_SB);          // [tile parity][token][wave]
    int8_t *stage = smem + P::OFF_STAGE + wave * P::STAGE;

    // Workgroup b takes members b, b + grid, b + 2 grid, ...: at any time the workgroups of the grid read and write one
    // contiguous stretch of rows (ranges a power of two apart per workgroup would all fall on the same memory channels).
    // Local tile t is tile t % tpm of the workgroup's member number t / tpm.
    const int tpm = p.T / 32;                                      // tiles per member
    const int grid = gridDim.x, b0 = blockIdx.x;
    if (b0 >= p.members) return;
    const int n_local = ((p.members - b0 + grid - 1) / grid) * tpm;

    // ---- the activation stream
    // copy side: lane (r = lane / 8, pp = lane % 8) of wave w moves chunk 2h + gg of row 8w + r of each column block
    const uint32_t lds_ring = (uint32_t)(size_t)(const __attribute__((address_space(3))) int8_t *)smem;
    uint32_t voff[CB];
    {
        const int r = lane >> 3, pp = (lane & 7) ^ (2 * ((wave >> 1) & 1)), h = (pp >> 1) ^ (r & 3), gg = (pp & 1) ^ (r >> 2);
#pragma unroll
        for (int cb = 0; cb < CB; cb++) voff[cb] = (uint32_t)((8 * wave + r) * K + cb * 128 + (2 * h + gg) * 16);
    }
    // next tile to request: local index, position inside its member, source pointer, LDS slot; the stream advances by one
    // tile, and by the rows of grid - 1 members more when it leaves a member
    int rq_t = 0, rq_tin = 0;
    uint64_t rq_src = (uint64_t)(p.X + (size_t)b0 * tpm * P::TILE);
    const uint64_t member_jump = (uint64_t)(grid - 1) * tpm * P::TILE;
    uint32_t rq_slot = 0;
    uint32_t rq_m0 = 0; uint64_t rq_base = 0; bool rq_go = false;        // the request being issued
    // A request is a few scalar instructions and CB copy instructions.  With one wave per SIMD every instruction of
    // the wave takes an issue slot of four clocks, so the parts are dealt out behind different MFMAs.
    auto request_prepare = [&]() {
        rq_go = rq_t < n_local;
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)rq_src), hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(rq_src >> 32));
        rq_base = ((uint64_t)hi << 32) | lo;
        rq_m0 = lds_ring + rq_slot + (uint32_t)(wave * CB * 1024);
        rq_t++;
        rq_src += P::TILE;
        if (++rq_tin == tpm) { rq_tin = 0; rq_src += member_jump; }
        rq_slot += P::TILE; if (rq_slot == (uint32_t)(NSLOT * P::TILE)) rq_slot = 0;
    };
    auto request_part = [&](int cb) {       // cb is a compile-time constant at every call site
        if (rq_go)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         : : "s"(rq_m0 + cb * 1024), "v"(voff[cb]), "s"(rq_base) : "memory", "m0");
    };
    auto request_next = [&]() {
        request_prepare();
#pragma unroll
        for (int cb = 0; cb < CB; cb++) request_part(cb);
    };
    // read side: lane (row j, half g), k-step ks = 4 cb + h
    uint32_t roff[4];
    {
        const int rg = j >> 3, r = j & 7;
#pragma unroll
        for (int h = 0; h < 4; h++) roff[h] = (uint32_t)(((rg * CB) * 64 + r * 8 + ((2 * (h ^ (r & 3)) + (g ^ (r >> 2))) ^ (2 * ((rg >> 1) & 1)))) * 16);
    }
    auto frag = [&](int slot_byte, int ks) -> v4i {      // ks is a compile-time constant at every call site
        return *reinterpret_cast<const v4i *>(smem + slot_byte + roff[ks & 3] + (ks >> 2) * 1024);
    };
    // the k-steps whose share of x.B this wave computes: kk = wave * QS + i; their fragment and B-table offsets
    uint32_t sb_xoff[QS], sb_boff[QS];
#pragma unroll
    for (int i = 0; i < QS; i++) {
        const int kk = wave * QS + i, h = kk & 3;
        uint32_t ro = roff[0];
#pragma unroll
        for (int hh = 1; hh < 4; hh++) ro = (h == hh) ? roff[hh] : ro;
        sb_xoff[i] = ro + (uint32_t)((kk >> 2) * 1024);
        sb_boff[i] = (uint32_t)(32 * kk + 16 * g);
    }
#pragma unroll 1
    for (int t = 0; t < NSLOT - 1; t++) request_next();

    // ---- resident W: lane (column j of column tile ct, half g) holds k = 32 ks + 16 g + 0..15 of its column, i.e. the
    // canonical blocked dwords kq = 8 ks + 4 g + q of column n
    // Which column goes to which MFMA row is free: row i = 8q + 4g' + e of a column tile takes column 16g' + 4q + e, so
    // that the 16 results a lane (token j, half g) holds per column tile are the 16 consecutive columns 32ct + 16g + 0..15
    // and leave as one 16-byte store (int8) without a transpose.
    const int pj = 16 * ((j >> 2) & 1) + 4 * (j >> 3) + (j & 3);
    v4i w[NCT][KS];
    {
        const uint32_t *Wb = reinterpret_cast<const uint32_t *>(p.Wblocked);
#pragma unroll
        for (int ct = 0; ct < NCT; ct++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
#pragma unroll
                for (int q = 0; q < 4; q++) w[ct][ks][q] = (int)Wb[(size_t)(8 * ks + 4 * g + q) * N + wave * NW + 32 * ct + pj];
    }

    // noise tables of a member, in set member % NTAB: this wave's columns of A (times the member's sign), and its
    // quarter of B for everyone
    auto fill_tables = [&](int member) {
        const int set = (member / grid) % NTAB;            // consecutive members of this workgroup rotate through the sets
        const int ns = (!p.own_noise && (member & 1)) ? -1 : 1;
        const uint32_t ps = p.seed + (uint32_t)(p.own_noise ? member : member / 2);
        for (int i = lane; i < NW; i += 64) Atab[set * NW + i] = noise_from_hash(ps + p.off_a, wave * NW + i, p.mask) * ns;
        for (int i = lane; i < K / EGG_WAVES; i += 64)
            Btab[set * K + wave * (K / EGG_WAVES) + i] = (int8_t)noise_from_hash(ps + p.off_b, wave * (K / EGG_WAVES) + i, p.mask);
    };
    // members (and tile positions inside them) of tiles t - 1, t, t + 1, kept incrementally; past either end they repeat
    // the first / last tile
    int m_prev = b0, m_cur = b0, m_next = b0, tin_next = 0;
    size_t row_prev = (size_t)b0 * tpm * 32, row_cur = row_prev, row_next = row_prev;       // first rows of those tiles
    if (n_local > 1) {
        if (tpm > 1) { tin_next = 1; row_next += 32; } else { m_next = b0 + grid; row_next += (size_t)grid * 32; }
    }
    if (!PLAIN) { fill_tables(m_cur); if (m_next != m_cur) fill_tables(m_next); }
    __builtin_amdgcn_s_waitcnt(0x0F70);       // the W loads and the first NSLOT - 1 tiles have landed: nothing is pending
    __syncthreads();

    // stage addressing (int32 only): one 32 x 32 tile at a time, 128 bytes per row, 16-byte chunk c of row r at c ^ (r & 7)
    const int rr8 = lane >> 3, rc8 = lane & 7;

    // One slice (column tile ct, q) of a finished tile is four results per lane: ep_value finishes one of them (shift,
    // rank-1 term, clip for int8), ep_emit packs the four into the stage; the int32 form stores a 32 x 32 tile after
    // its fourth slice.
    auto ep_value = [&](int accv, int a, int sbv) -> int {
        if (BYTE1) return min(127 * 256 + 255, max(-127 * 256, accv));
        const int o = PLAIN ? (accv >> p.shift) : ws_perturbed<FUSE>(accv, sbv, a, p.sigma, p.shift);
        return OUT32 ? o : clip127(o);
    };
    int o8[4];                                   // int8: the packed results of the slices of one column tile
    auto ep_emit = [&](int s, const int (&o)[4], size_t row0) {
        const int ct = s >> 2, q = s & 3;
        if (OUT32) {
            // lane (row j) holds int32 columns 16g + 4q + e of the 32 x 32 tile: chunk 4g + q of its 128-byte row
            v4i o4 = {o[0], o[1], o[2], o[3]};
            *reinterpret_cast<v4i *>(stage + j * 128 + (((4 * g + q) ^ (j & 7)) * 16)) = o4;
            if (q == 3) {
                wave_lds_fence();
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = rr8 + 8 * i;
                    v4i v = *reinterpret_cast<const v4i *>(stage + r * 128 + ((rc8 ^ (r & 7)) * 16));
                    *reinterpret_cast<v4i *>(p.Y32 + (row0 + r) * N + wave * NW + 32 * ct + 4 * rc8) = v;
                }
                wave_lds_fence();
            }
        } else {
            o8[q] = BYTE1 ? pack_bytes1(o[0], o[1], o[2], o[3]) : pack_bytes(o[0], o[1], o[2], o[3]);
            if (q == 3) {
                const v4i v = {o8[0], o8[1], o8[2], o8[3]};
                *reinterpret_cast<v4i *>(p.Y8 + (row0 + j) * N + wave * NW + 32 * ct + 16 * g) = v;
            }
        }
    };
    auto ep_slice = [&](v16i (&acc)[NCT], int s, const int *Aset, int sbv, size_t row0) {
        const int ct = s >> 2, q = s & 3;
        v4i a4 = {0, 0, 0, 0};
        if (!PLAIN) a4 = *reinterpret_cast<const v4i *>(Aset + 32 * ct + 16 * g + 4 * q);
        int o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = ep_value(acc[ct][4 * q + e], a4[e], sbv);
        ep_emit(s, o, row0);
    };
    v4i xq[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) xq[i] = frag(0, i);      // (the last of them is read again by the first k-step; harmless)
    int sb_prev = 0;                           // x.B of this lane's token in the previous tile
    uint32_t slot_cur = 0;                     // LDS byte offset of the current tile's slot

    // One tile: MFMAs of tile t into `cur`, epilogue of tile t - 1 from `prev`.
    auto step = [&](v16i (&cur)[NCT], v16i (&prev)[NCT], int t) {
        const int slot = (int)slot_cur, slot_next = (slot + P::TILE == NSLOT * P::TILE) ? 0 : slot + P::TILE;
        // for t = 0 the epilogue processes zeros and stores them to tile 0's rows, which the real epilogue of tile 0
        // overwrites later from the same wave
        const size_t prow0 = row_prev;
        const int *Aprev = Atab + (PLAIN ? 0 : ((m_prev / grid) % NTAB) * NW);
        const int8_t *Bcur = Btab + (PLAIN ? 0 : ((m_cur / grid) % NTAB) * K);
        int sbp = 0, sb_next = 0;
        constexpr int SPK = P::SLICES >= KS ? P::SLICES / KS : 1;           // epilogue slices per k-step
        constexpr int KPS = P::SLICES >= KS ? 1 : KS / P::SLICES;           // k-steps per slice
        v4i pre_a[SPK], pre_xs = {0, 0, 0, 0}, pre_b = {0, 0, 0, 0};
#pragma unroll
        for (int si = 0; si < SPK; si++) pre_a[si] = v4i{0, 0, 0, 0};
        auto load_small = [&](int ks) {          // A noise of the slices finished in k-step ks; fragment and B noise of the x.B share
            if (ks >= KS) return;
            if (!PLAIN && ks % KPS == 0) {
#pragma unroll
                for (int si = 0; si < SPK; si++) {
                    const int sl = (ks / KPS) * SPK + si;
                    pre_a[si] = *reinterpret_cast<const v4i *>(Aprev + 32 * (sl >> 2) + 16 * g + 4 * (sl & 3));
                }
            }
            if (!PLAIN && ks < QS) {
                pre_xs = *reinterpret_cast<const v4i *>(smem + slot + sb_xoff[ks < QS ? ks : 0]);
                pre_b = *reinterpret_cast<const v4i *>(Bcur + sb_boff[ks < QS ? ks : 0]);
            }
        };
        load_small(0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            if (ks == MID) {
                // Tile t + 1 was requested NSLOT - 2 tiles ago, at this point of that tile's loop; every tile issues CB
                // copies here (while tiles remain) and STORES stores.  Operations complete in issue order, so once at
                // most the later ones are outstanding, tile t + 1 has landed.  The first NSLOT - 2 tiles were waited
                // for before the loop.
                // (No store is issued between this wait and the copies of the same tile -- the stores of a k-step follow its
                // last MFMA, the copies sit behind the first MFMAs of k-step MID + 1 -- so "later" counts whole tiles.)
                static_assert(P::SLICES >= KS ? (KS / 4 <= 2 || (MID % 4 != 3 && (MID + 1) % 4 != 3)) : true, "no store between the wait and the copies");
                __builtin_amdgcn_sched_barrier(0);
                if (t >= NSLOT - 2) {
                    constexpr int steady = (NSLOT - 2) * STORES + (NSLOT - 3) * CB;
                    if (t + NSLOT - 1 <= n_local) {                // NSLOT - 3 or more requests followed tile t + 1's
                        constexpr int cnt = steady < 63 ? steady : 63;
                        __builtin_amdgcn_s_waitcnt(0x0F70 | (cnt & 15) | ((cnt >> 4) << 14));
                    } else {
                        int reqs = n_local - t - 2;                // fewer near the end
                        reqs = reqs < 0 ? 0 : reqs;
                        wait_vmcnt_upto((NSLOT - 2) * STORES + reqs * CB);
                    }
                }
                __syncthreads();
                // the request of tile t + NSLOT - 1 (into the slot of tile t - 1, which every wave has left) follows behind
                // the MFMAs of this k-step and the next
                __builtin_amdgcn_sched_barrier(0);
            }
            // The wave issues in order and a second MFMA cannot start while the first one occupies the matrix pipe, so the
            // vector work of this k-step is dealt out behind the individual MFMAs: each runs in the shadow of the one
            // in front of it.  The scheduling barriers keep that order.
            const bool ep_here = ks % KPS == 0;
            static_assert((SPK * 4) % NCT == 0, "epilogue values per MFMA");
            constexpr int EPM = SPK * 4 / NCT;                                  // epilogue values behind each MFMA
            const v4i xf = xq[ks % PF];
            int o[SPK][4];
            // the small table reads of this k-step were issued a k-step earlier (pre_*), those of the next one go out
            // behind the first MFMA
            v4i a4[SPK], xs = {0, 0, 0, 0}, b4 = {0, 0, 0, 0};
#pragma unroll
            for (int si = 0; si < SPK; si++) a4[si] = pre_a[si];
            if (!PLAIN && ks < QS) { xs = pre_xs; b4 = pre_b; }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) {
                if (ks == 0) {
                    v16i z;
#pragma unroll
                    for (int r = 0; r < 16; r++) z[r] = 0;
                    cur[ct] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[ct][ks], xf, z, 0, 0, 0);
                } else cur[ct] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[ct][ks], xf, cur[ct], 0, 0, 0);
                if (ks == MID && ct == NCT - 1) request_prepare();
                if (ks == MID + 1 && ct < CB) request_part(ct);
                if (ct == 0) {
                    // The fragment registers of the previous k-step are free only now: an MFMA keeps reading its operands
                    // while it runs, so a write to them right behind the MFMA that used them last (a vector temporary, or
                    // the issue of this read) would wait for it.  The empty asm keeps the compiler from giving them away
                    // earlier.  The read fetches the fragment PF - 1 steps ahead: of this tile, or (after the barrier) of
                    // the next one.
                    const int pq = (ks + PF - 1) % PF, pk = ks - 1 + PF;
                    asm volatile("" : : "v"(xq[pq]));
                    xq[pq] = (pk < KS) ? frag(slot, pk) : frag(slot_next, pk - KS);
                    load_small(ks + 1);
                }
                if (ep_here) {
#pragma unroll
                    for (int i = 0; i < EPM; i++) {
                        const int v = ct * EPM + i, si = v >> 2, e = v & 3, sl = (ks / KPS) * SPK + si;
                        o[si][e] = ep_value(prev[sl >> 2][4 * (sl & 3) + e], a4[si][e], sb_prev);
                    }
                }
                if (!PLAIN && ks < QS) sbp = dot4(xs[ct & 3], b4[ct & 3], sbp);
                if (ct == NCT - 1) {
                    if (ep_here) {
#pragma unroll
                        for (int si = 0; si < SPK; si++) ep_emit((ks / KPS) * SPK + si, o[si], prow0);
                    }
                    if (!PLAIN) {
                        if (ks == QS) {
                            sbp = sum_halves(sbp);
                            sbx[(((t & 1) * 32 + j) << 2) + wave] = sbp;
                        }
                        if (ks == MID + 1) {
                            const v4i parts = *reinterpret_cast<const v4i *>(sbx + (((t & 1) * 32 + j) << 2));
                            sb_next = parts[0] + parts[1] + parts[2] + parts[3];
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        sb_prev = sb_next;
        slot_cur = (uint32_t)slot_next;
        // members of the next step; the tables of tile t + 2's member are filled now and published by the barrier of
        // tile t + 1, one tile ahead of their first use (three sets in rotation: those of tiles t and t + 1 stay intact)
        m_prev = m_cur; m_cur = m_next; row_prev = row_cur; row_cur = row_next;
        if (t + 2 < n_local) {
            row_next += 32;
            if (++tin_next == tpm) { tin_next = 0; m_next += grid; row_next += (size_t)(grid - 1) * tpm * 32; if (!PLAIN) fill_tables(m_next); }
        }
    };

    v16i accA[NCT], accB[NCT];
    zero_acc<NCT>(accB);
    int t = 0;
#pragma unroll 1
    for (; t + 1 < n_local; t += 2) { step(accA, accB, t); step(accB, accA, t + 1); }
    // after the last step (m_prev, row_prev) is the last tile
    if (t < n_local) step(accA, accB, t);
    const size_t lrow0 = row_prev;
    const int *Alast = Atab + (PLAIN ? 0 : ((m_prev / grid) % NTAB) * NW);
    if (t < n_local) {
#pragma unroll
        for (int s = 0; s < P::SLICES; s++) ep_slice(accA, s, Alast, sb_prev, lrow0);
    } else {
#pragma unroll
        for (int s = 0; s < P::SLICES; s++) ep_slice(accB, s, Alast, sb_prev, lrow0);
    }
}

static int egg_cu_count() {
    static int n = 0;
    if (!n) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) n = v;
        else n = 256;
    }
    return n;
}

template <int K, int N, bool OUT32, int MODE>
static hipError_t launch_ws(const PlinParams &p, hipStream_t s) {
    typedef PlinWS<K, N> P;
    int grid = egg_cu_count(); if (grid > p.members) grid = p.members;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_plinear_ws<K, N, OUT32, MODE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)P::TOTAL);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((k_plinear_ws<K, N, OUT32, MODE>), dim3(grid), dim3(EGG_THREADS), P::TOTAL, s, p);
    return hipGetLastError();
}
template <int K, int N>
static hipError_t launch_ws_kn(const PlinParams &p, hipStream_t s) {
    const long long mag = egg_noise_magnitude(p.mask);
    const long long bound = ((long long)K * 128 * 128 << p.sigma) + (long long)K * 128 * mag * mag;
    const bool fuse = p.sigma >= 0 && p.sigma <= 12 && p.sigma + p.shift < 32 && bound < (1LL << 31);
    const int mode = p.plain ? 0 : (fuse ? 2 : 1);
    hipError_t e = hipSuccess;
    if (p.Y32) e = mode == 0 ? launch_ws<K, N, true, 0>(p, s) : (mode == 1 ? launch_ws<K, N, true, 1>(p, s) : launch_ws<K, N, true, 2>(p, s));
    if (e == hipSuccess && p.Y8) e = mode == 0 ? (p.shift == 8 ? launch_ws<K, N, false, 3>(p, s) : launch_ws<K, N, false, 0>(p, s))
                                               : (mode == 1 ? launch_ws<K, N, false, 1>(p, s) : launch_ws<K, N, false, 2>(p, s));
    return e;
}
// shapes the W-stationary kernel is built for
bool egg_plinear_ws_shape(int K, int N) { return (K == 512 && N == 512) || (K == 256 && N == 512); }
hipError_t egg_launch_plinear_ws(const PlinParams &p, hipStream_t s) {
    if (!p.Wblocked || p.T % 32 || p.T < 32 || p.members < 1) return hipErrorInvalidValue;
    if (p.K == 512 && p.N == 512) return launch_ws_kn<512, 512>(p, s);
    if (p.K == 256 && p.N == 512) return launch_ws_kn<256, 512>(p, s);
    return hipErrorInvalidValue;
}
