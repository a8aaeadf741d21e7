// gemm_mfma16_kernel.hpp -- gfx950 GEMM kernels built on v_mfma_f32_16x16x32_{bf16,f16}:
// the default tiled kernel of the library (aligned and predicated variants) and a ring variant.
//
//   C[M,N] = A[M,K] . B[N,K]^T
//   aligned variant:    M % BM == 0, N % BN == 0, K % 128 == 0, 16-byte aligned pointers
//   predicated variant: any M, N, K >= 1, any (2-byte) alignment
//
// Why this MFMA shape: on random bf16 data the chip is power limited, and an MFMA-only loop
// of 16x16x32 instructions sustains ~1.9-2.05 PFLOP/s where 32x32x16 sustains ~1.75 (the
// 16x16 instruction moves half as many accumulator registers per flop).  One wave per SIMD
// issues it back to back (16.4 cycles per MFMA measured), so the kernel runs four waves with
// a 128 x 128 wave tile (64 accumulator tiles, 256 AGPRs per lane) -- the least LDS traffic
// per flop -- or eight waves with 64 x 128.
//
// Everything else follows gemm_kernel.hpp: two LDS stages of one 64-deep K slab each,
// 128-byte rows with the 16-byte chunks stored at chunk ^ ((row >> 1) & 7), direct-to-LDS
// buffer loads (inline asm, explicit waits), XCD-aware tile order, C tile transposed through
// LDS and written 16 bytes per lane.  A K step is two 32-deep slices: slice 0 multiplies
// while the fragments of slice 1 are fetched; after the mid-step barrier slice 1 multiplies
// while slice 0 of the next slab is fetched.  The loads of the slab after next either go out
// during slice 1 (DRAIN = 0) or, after an early second barrier that frees the current
// stage, are spread over nearly the whole step (DRAIN > 0, see Mfma16Config).
//
// Fragment layout of the 16x16x32 MFMA: lane l holds row (l & 15), k chunk (l >> 4) of the
// 32-deep slice (8 elements, 16 bytes); result register e of lane l is
// D[4*(l >> 4) + e][l & 15].  Operands are swapped (B rows as the MFMA "A" matrix) so that a
// lane holds 4 consecutive n of one m.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "gemm_kernel.hpp"

namespace mi {

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// KG = 2: eight waves as two groups of WM x WN, each multiplying one half of K of the same tile
// in LDS stages of its own; the groups share the barriers (same trip count: K % 256 == 0) and
// the second hands its accumulators to the first through LDS at the end.  For tiles that are
// alone on their CU (a lone 128x128 workgroup of the two-per-CU kernel runs at ~62 % of its
// paired rate: two waves per SIMD hide each other's LDS and load latency).
template <int BM_, int BN_, int WM_, int WN_, int GROUP_, int DT_, int DRAIN_ = 0, bool EDGE_ = false, int OCC_ = 1,
          int KG_ = 1>
struct Mfma16Config {
    static constexpr int BM = BM_, BN = BN_, BK = 64;
    static constexpr int WM = WM_, WN = WN_, GROUP = GROUP_, DT = DT_;
    static constexpr bool DRAIN = DRAIN_ != 0;
    static constexpr bool EDGE = EDGE_;                  // predicated variant: any M, N, K, any alignment
    static constexpr int KG = KG_;                       // groups of waves that split K
    static constexpr int NW = WM * WN, NT = NW * KG * 64;
    static constexpr int TM = BM / WM, TN = BN / WN;
    static constexpr int MI = TM / 16, NI = TN / 16;
    static constexpr int RPP = NW * 8;                   // tile rows one pass of a group's threads loads
    static constexpr int LA = BM / RPP, LB = BN / RPP;   // load instructions per wave per slab
    static constexpr int A_STAGE = BM * 128, B_STAGE = BN * 128;
    static constexpr int LDS_GROUP = 2 * (A_STAGE + B_STAGE);
    static constexpr int LDS_BYTES = KG * LDS_GROUP;
    static constexpr int OCC = OCC_;                     // workgroups per CU the register / LDS budget is sized for
    static_assert(KG == 1 || (KG == 2 && BM * BN * 4 <= LDS_GROUP), "the second group's accumulators pass through its stages");
    static constexpr int WAVES_PER_EU = NT / 256 * OCC;
    static constexpr int NMMA = MI * NI, NFR = MI + NI;
    static_assert(NT == 256 || NT == 512, "one or two waves per SIMD");
    static_assert(OCC >= 1 && LDS_BYTES * OCC <= 160 * 1024, "LDS budget of one CU");
    static_assert(TM % 16 == 0 && TN % 16 == 0, "wave tile must be a multiple of 16x16");
    static_assert(BM % RPP == 0 && BN % RPP == 0 && RPP % 16 == 0, "tile rows divide over the threads");
    static constexpr int DSP = (NMMA - NFR) / (LA + LB);   // MFMA slots between two load instructions
    static_assert(DSP >= 1, "reads and loads each get an MFMA slot");
    // DRAIN > 0: a second barrier early in slice 0 (slot SA = NFR + 4*DRAIN, once every wave has fetched the
    // slice-1 fragments) frees the current stage, so the loads of the slab after next are
    // dealt out over the rest of slice 0 and all of slice 1 (slots SA+1 + d*DSPD of the
    // step) and have a whole K step to land; D0 of them are issued before the mid-step wait.
    static constexpr int SA = NFR + 4 * DRAIN_;
    static constexpr int DSPD = (2 * NMMA - 5 - SA) / (LA + LB);
    static constexpr int D0 = DSPD > 0 ? (NMMA - SA - 1 + DSPD - 1) / DSPD : 0;
    static_assert(!DRAIN || (DSPD >= 1 && SA + 1 < NMMA && D0 <= LA + LB), "drain schedule");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
    static_assert(BM * BN * 2 <= LDS_GROUP, "the epilogue stages the C tile in the stage buffers");
};

template <int DT>
__device__ __forceinline__ f32x4_t mfma_16x16x32(u32x4_t a, u32x4_t b, f32x4_t c) {
    if constexpr (DT == DT_BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                      __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                     __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
}

// SPLITK: the workgroup multiplies one piece of the K range of its tile (blockIdx.y) and
// leaves an fp32 partial tile in the workspace instead of C.  A separate instantiation, so
// that the plain kernel's registers and epilogue are untouched by it (a run-time branch to a
// third epilogue made the 256-accumulator kernel spill in its last K step and epilogue).
//
// Only when the header is compiled with -DMI_GEMM_ABLATE (harness/gemm_power.hip does, the
// library does not) the kernel takes a fourth parameter ABLATE that compiles parts of the K
// loop out, so that their share of cycles and of power can be read off -- bit 0: no global ->
// LDS loads after the prologue, bit 1: no LDS fragment reads in the loop, bit 2: no barriers,
// bit 3: no epilogue (C is not written).  The results of such a kernel are meaningless.  In the library's build MI_ABLATED is `false`.
#ifdef MI_GEMM_ABLATE
#define MI_ABLATED(bits) ((ABLATE & (bits)) != 0)
template <class Cfg, bool TRACE = false, bool SPLITK = false, int ABLATE = 0>
#else
#define MI_ABLATED(bits) false
template <class Cfg, bool TRACE = false, bool SPLITK = false>
#endif
__global__ void __launch_bounds__(Cfg::NT)
__attribute__((amdgpu_waves_per_eu(Cfg::WAVES_PER_EU, Cfg::WAVES_PER_EU)))
gemm_mfma16_kernel(const GemmArgs p) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, WN = Cfg::WN;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, LA = Cfg::LA, LB = Cfg::LB, RPP = Cfg::RPP;
    constexpr int A_STAGE = Cfg::A_STAGE, B_STAGE = Cfg::B_STAGE;
    constexpr int NMMA = Cfg::NMMA, NFR = Cfg::NFR, DT = Cfg::DT;
    constexpr int TM = Cfg::TM, TN = Cfg::TN;

    // [A stage 0][A stage 1][B stage 0][B stage 1], once per K group
    __shared__ __attribute__((aligned(128))) unsigned char lds_all[Cfg::LDS_BYTES];
    static_assert(!(SPLITK && Cfg::KG > 1), "K is split either over workgroups or over the groups of one");

    long long tr_wait = 0, tr_t0 = 0, tr_loop = 0;
    int tr_cnt = 0;
    auto tr_now = [&]() __attribute__((always_inline)) { return (long long)__builtin_readcyclecounter(); };
    if constexpr (TRACE) tr_loop = tr_now();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = Cfg::KG > 1 ? wave_all / Cfg::NW : 0;        // K group of this wave
    const int wave = Cfg::KG > 1 ? wave_all % Cfg::NW : wave_all;   // its number inside the group
    const int wm = wave / WN, wn = wave % WN;
    // (the array itself when there is one group: a pointer variable in its place costs the
    // 256-accumulator kernels registers, and they have none to spare)
    decltype(auto) lds = [&]() -> decltype(auto) {
        if constexpr (Cfg::KG == 1) return (lds_all);
        else return lds_all + kg * Cfg::LDS_GROUP;
    }();

    int tm, tn;
    tile_of_block<Cfg::GROUP>(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
    const int row0 = tm * BM, col0 = tn * BN;
    constexpr bool EDGE = Cfg::EDGE;
    // Split-K: this workgroup multiplies the K range [k0, k0 + K) of its tile; k_per_split is a
    // multiple of 128, so only the last piece can have a K tail.  Everything below works on
    // the local range.
    // K groups: group g multiplies [g * K / KG, (g + 1) * K / KG); the launcher's caller makes
    // sure K is a multiple of 128 * KG, so the groups run the same number of steps.
    const int k0 = SPLITK ? (int)blockIdx.y * p.k_per_split : kg * (p.K / Cfg::KG);
    const int M = p.M, N = p.N;
    const int K = SPLITK ? ((p.K - k0) < p.k_per_split ? (p.K - k0) : p.k_per_split) : p.K / Cfg::KG;
    // K steps: an even number.  The aligned variant is only launched with K % 128 == 0; the
    // predicated one rounds up and the surplus (part of a) slab is zeroed in LDS (a slab that
    // lies past K altogether is still loaded and zeroed, but its step is not run).
    const int KT = EDGE ? ((K + 2 * BK - 1) / (2 * BK)) * 2 : K / BK;

    // Descriptors end exactly at the last element of the tile's last valid row: nothing past
    // the end of a matrix is ever touched, and rows past M / N read as zeros.
    const int rowsA = (M - row0) < BM ? (M - row0) : BM;
    const int rowsB = (N - col0) < BN ? (N - col0) : BN;
    const unsigned char* Ab = (const unsigned char*)p.A + ((size_t)row0 * p.lda + k0) * 2;
    const unsigned char* Bb = (const unsigned char*)p.B + ((size_t)col0 * p.ldb + k0) * 2;
    // (split-K: up to the true end of the last row, so that a piece that ends inside the row
    // does not lose its last element to the dword-granular range check; K - k0 == K_local in
    // the last piece, where the K-tail logic needs exactly that)
    const int Kdesc = p.K - k0;
    const uint32_t bytesA = (uint32_t)((rowsA - 1) * p.lda + Kdesc) * 2u;
    const uint32_t bytesB = (uint32_t)((rowsB - 1) * p.ldb + Kdesc) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);

    auto swz = [](int row) __attribute__((always_inline)) { return (row >> 1) & 7; };
    // direct-to-LDS loads: one instruction fills 8 rows x 128 bytes; lane l lands on chunk
    // position l & 7 of row l >> 3 and fetches logical chunk (l & 7) ^ swz(row)
    const int lr = lane >> 3, lc = lane & 7;
    const int drow = wave * 8 + lr;
    const int dchunk = lc ^ swz(drow);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const uint32_t dlds = lds_base + (uint32_t)wave * 1024u;
    // GROUPED (aligned variant): wave w loads the contiguous rows w*LA*8 .. of A (and likewise
    // of B), load d covering rows d*8 .. d*8+7 of that range, so that up to four consecutive
    // loads land 1 KB apart in LDS: they share one M0 value and differ in the instruction's
    // immediate offset.  The immediate is added to the global address as well, so it is
    // subtracted from the lane offset beforehand (never below zero: the rows of load d start
    // at least 8*d rows = 8*d*K*2 >= 2048*d bytes into the panel, K >= 128 here).  Four M0
    // writes (and the wait state each needs before the load that reads it) per K step instead
    // of sixteen: 2368 -> 2314 cycles per K step at 256x256.  M0 stays live from one asm
    // statement to the next; the compiler has no use for it in this kernel (LDS instructions
    // need no M0 on gfx9), which tests/test_isa_invariants.py checks on the generated code.
    // Predicated variant: load d covers rows d*RPP + w*8 .. (the lane's chunk is then the same
    // for all its loads, which the K-tail fix-up relies on), one M0 value per load.
    constexpr bool GROUPED = !EDGE;
    constexpr int GA = LA % 4 == 0 ? 4 : LA % 3 == 0 ? 3 : LA % 2 == 0 ? 2 : 1;
    constexpr int GB = LB % 4 == 0 ? 4 : LB % 3 == 0 ? 3 : LB % 2 == 0 ? 2 : 1;
    uint32_t voffs[LA + LB];
    if constexpr (GROUPED) {
#pragma unroll
        for (int d = 0; d < LA; ++d) {
            const int row = wave * (LA * 8) + d * 8 + lr;
            voffs[d] = (uint32_t)(row * p.lda + (lc ^ swz(row)) * 8) * 2u - (uint32_t)((d % GA) * 1024);
        }
#pragma unroll
        for (int d = 0; d < LB; ++d) {
            const int row = wave * (LB * 8) + d * 8 + lr;
            voffs[LA + d] = (uint32_t)(row * p.ldb + (lc ^ swz(row)) * 8) * 2u - (uint32_t)((d % GB) * 1024);
        }
    } else {
        const uint32_t dvoffA = (uint32_t)(drow * p.lda + dchunk * 8) * 2u;
        const uint32_t dvoffB = (uint32_t)(drow * p.ldb + dchunk * 8) * 2u;
        const uint32_t passA = (uint32_t)(RPP * p.lda) * 2u;
        const uint32_t passB = (uint32_t)(RPP * p.ldb) * 2u;
#pragma unroll
        for (int d = 0; d < LA; ++d) voffs[d] = dvoffA + d * passA;
#pragma unroll
        for (int d = 0; d < LB; ++d) voffs[LA + d] = dvoffB + d * passB;
    }
    auto dma = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
    };
    // same M0 as the previous load of this wave, LDS (and global) address advanced by IMM bytes
    auto dma_next = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, auto imm_c) __attribute__((always_inline)) {
        asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 lds"
                     :: "v"(voff), "s"(rsrc), "s"(soff), "n"(decltype(imm_c)::value) : "memory");
    };
    auto dma_one = [&](int kt, int stage, int d) __attribute__((always_inline)) {
        if constexpr (MI_ABLATED(1)) { if (kt >= 2) return; }
        const uint32_t kb = (uint32_t)kt * (BK * 2);
        if constexpr (GROUPED) {
            if (d < LA) {
                const uint32_t dst = lds_base + stage * A_STAGE + (wave * LA + (d / GA) * GA) * 1024;
                if (d % GA == 0) dma(rsrcA, voffs[d], kb, dst);
                else if (d % GA == 1) dma_next(rsrcA, voffs[d], kb, std::integral_constant<int, 1024>{});
                else if (d % GA == 2) dma_next(rsrcA, voffs[d], kb, std::integral_constant<int, 2048>{});
                else dma_next(rsrcA, voffs[d], kb, std::integral_constant<int, 3072>{});
            } else {
                const int e = d - LA;
                const uint32_t dst = lds_base + 2 * A_STAGE + stage * B_STAGE + (wave * LB + (e / GB) * GB) * 1024;
                if (e % GB == 0) dma(rsrcB, voffs[d], kb, dst);
                else if (e % GB == 1) dma_next(rsrcB, voffs[d], kb, std::integral_constant<int, 1024>{});
                else if (e % GB == 2) dma_next(rsrcB, voffs[d], kb, std::integral_constant<int, 2048>{});
                else dma_next(rsrcB, voffs[d], kb, std::integral_constant<int, 3072>{});
            }
        } else {
            if (d < LA)
                dma(rsrcA, voffs[d], kb, dlds + stage * A_STAGE + d * (RPP * 128));
            else
                dma(rsrcB, voffs[d], kb, dlds + 2 * A_STAGE + stage * B_STAGE + (d - LA) * (RPP * 128));
        }
    };

    // K tail (predicated variant).  A direct-to-LDS load of the chunk at k..k+7 of a row runs
    // into the next row of the matrix when k+7 >= K (or returns zeros past the descriptor), so
    // once its own loads of a slab have landed, each lane zeroes what it fetched at k >= K, in
    // LDS, before the barrier that publishes the slab.  The range check works on whole
    // dwords: the dword holding the last element (k = K-1) of the tile's last row is dropped
    // whenever its other half lies past the descriptor's end, so that one element per operand
    // is fetched by a 2-byte load up front (tailA / tailB) and put back here.  This lane's
    // logical chunk is the same for all its loads (the swizzle repeats every 16 rows).
    uint32_t tailA = 0, tailB = 0;
    if constexpr (EDGE) {
        tailA = __builtin_amdgcn_readfirstlane(__builtin_amdgcn_raw_buffer_load_b16(rsrcA, bytesA - 2u, 0, 0));
        tailB = __builtin_amdgcn_readfirstlane(__builtin_amdgcn_raw_buffer_load_b16(rsrcB, bytesB - 2u, 0, 0));
    }
    auto fix_tail = [&](int kt, int stage) __attribute__((always_inline)) {
        const int nvalid = K - (kt * BK + dchunk * 8);   // elements of this lane's chunk that lie inside K
        if (nvalid >= 8) return;
        const int kl = nvalid - 1;                       // where k = K-1 sits in this chunk
        const bool mine = kl >= 0;
        uint32_t m[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int n = nvalid - 2 * d;
            m[d] = n >= 2 ? 0xffffffffu : (n == 1 ? 0x0000ffffu : 0u);
        }
        // rolled loops: this runs for the last two slabs only and must not cost registers
        auto fix_rows = [&](unsigned char* ptr, int passes, int last_row, uint32_t e) __attribute__((always_inline)) {
#pragma clang loop unroll(disable)
            for (int d = 0; d < passes; ++d, ptr += RPP * 128) {
                u32x4_t v = *(const u32x4_t*)ptr;
                const bool hit = mine && d * RPP + drow == last_row;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t old = v[w];
                    const uint32_t pv = (kl & 1) ? ((old & 0x0000ffffu) | (e << 16)) : ((old & 0xffff0000u) | e);
                    v[w] = ((hit && (kl >> 1) == w) ? pv : old) & m[w];
                }
                *(u32x4_t*)ptr = v;
            }
        };
        fix_rows(lds + stage * A_STAGE + wave * 1024 + lane * 16, LA, rowsA - 1, tailA);
        fix_rows(lds + 2 * A_STAGE + stage * B_STAGE + wave * 1024 + lane * 16, LB, rowsB - 1, tailB);
    };

    // fragment reads: lane holds row (lane & 15), k chunk 4*ks + (lane >> 4) of the slab
    const int l16 = lane & 15, q = lane >> 4;
    int rd_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) rd_off[ks] = l16 * 128 + ((((ks << 2) | q) ^ swz(l16)) << 4);
    const int a_wave = wm * TM * 128;
    const int b_wave = 2 * A_STAGE + wn * TN * 128;

    u32x4_t fa[2][MI], fb[2][NI];
    f32x4_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.0f;

    auto mma_one = [&](int buf, int idx) __attribute__((always_inline)) {
        // rows of accumulator tiles in turn, columns back and forth: srcB (the A fragment) stays
        // for a whole row and srcA (the B fragment) is kept across the turn, so every MFMA
        // changes one operand only.  The chip is power limited and operand changes cost power:
        // same cycle count, 0.3-1 % less time than always starting a row at column 0 (and the
        // column-major order, srcB changing every time, measured 8 % slower).
        const int i = idx / NI, j = (i & 1) ? NI - 1 - idx % NI : idx % NI;
        acc[i][j] = mfma_16x16x32<DT>(fb[buf][j], fa[buf][i], acc[i][j]);
    };
    // fragment r of a slice in the order the MFMAs first need them: A0, B0..B(NI-1), A1..
    [[maybe_unused]] bool in_loop = false;      // (ablation bit 1: fragment reads only before the K loop)
    auto read_one = [&](int stage, int ks, int buf, int r) __attribute__((always_inline)) {
        if constexpr (MI_ABLATED(2)) { if (in_loop) return; }
        if (r == 0 || r > NI) {
            const int i = r == 0 ? 0 : r - NI;
            fa[buf][i] = *(const u32x4_t*)(lds + stage * A_STAGE + a_wave + i * 2048 + rd_off[ks]);
        } else {
            const int j = r - 1;
            fb[buf][j] = *(const u32x4_t*)(lds + stage * B_STAGE + b_wave + j * 2048 + rd_off[ks]);
        }
    };

    // ---- prologue: slab 0 -> stage 0, slab 1 -> stage 1 ----
#pragma unroll
    for (int d = 0; d < LA + LB; ++d) dma_one(0, 0, d);
#pragma unroll
    for (int d = 0; d < LA + LB; ++d) dma_one(1, 1, d);
    // Pin the zeroing of the accumulators here, while the first slabs are on their way: left
    // alone, the compiler zeroes every accumulator register twice, after the wait for slab 0.
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) asm volatile("" : "+a"(acc[i][j]));
    if constexpr (EDGE) {
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"(LA + LB) : "memory");            // own loads of slab 0 are in
        if (BK > K) fix_tail(0, 0);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(LA + LB) : "memory");    // slab 0 is in
    }
#pragma unroll
    for (int r = 0; r < NFR; ++r) read_one(0, 0, 0, r);

    // load instruction slots of slice 1: spread evenly over the MFMAs that follow the fragment reads
    auto kstep = [&](int kt, auto cur_c, auto has1_c, auto has2_c, auto fix_c) __attribute__((always_inline)) {
        constexpr int cur = decltype(cur_c)::value;
        constexpr int nxt = cur ^ 1;
        constexpr bool has1 = decltype(has1_c)::value;
        constexpr bool has2 = decltype(has2_c)::value;
        constexpr bool fix = decltype(fix_c)::value;       // slab kt+1 may cross K (predicated variant)
        // load d of slab kt+2 goes out at slot g of the step (slice 0: g < NMMA)
        auto dma_slot = [&](int g) __attribute__((always_inline)) {
            if constexpr (has2) {
                if constexpr (Cfg::DRAIN) {
                    const int d = g - (Cfg::SA + 1);
                    if (d >= 0 && d % Cfg::DSPD == 0 && d / Cfg::DSPD < LA + LB) dma_one(kt + 2, cur, d / Cfg::DSPD);
                } else {
                    const int d = g - NMMA - NFR;
                    if (d >= 0 && d % Cfg::DSP == 0 && d / Cfg::DSP < LA + LB) dma_one(kt + 2, cur, d / Cfg::DSP);
                }
            }
        };
#pragma unroll
        for (int idx = 0; idx < NMMA; ++idx) {
            mma_one(0, idx);
            if (idx < NFR) read_one(cur, 1, 1, idx);
            if constexpr (Cfg::DRAIN && has2) {
                // every wave holds its slice-1 fragments: stage `cur` may be overwritten
                if (idx == Cfg::SA) {
                    if constexpr (MI_ABLATED(4)) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    else asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                }
            }
            dma_slot(idx);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (has1) {
            if constexpr (TRACE) tr_t0 = tr_now();
            // slab kt+1 has landed (the D0 younger loads of slab kt+2 may still be in flight)
            if constexpr (fix) {
                if constexpr (Cfg::DRAIN && has2)
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" :: "n"(Cfg::D0) : "memory");
                else
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                fix_tail(kt + 1, nxt);
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            } else if constexpr (MI_ABLATED(4)) {
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            } else if constexpr (Cfg::DRAIN && has2) {
                asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(Cfg::D0) : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            }
            if constexpr (TRACE) { tr_wait += tr_now() - tr_t0; ++tr_cnt; }
        }
#pragma unroll
        for (int idx = 0; idx < NMMA; ++idx) {
            mma_one(1, idx);
            if constexpr (has1) {
                if (idx < NFR) read_one(nxt, 0, 0, idx);
            }
            dma_slot(NMMA + idx);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if constexpr (MI_ABLATED(2)) {      // both fragment buffers hold real operand data
#pragma unroll
        for (int r = 0; r < NFR; ++r) read_one(0, 1, 1, r);
    }
    in_loop = true;
    using T = std::true_type;
    using F = std::false_type;
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    int kt = 0;
    if constexpr (!EDGE) {
        for (; kt + 2 < KT; kt += 2) {
            kstep(kt, S0{}, T{}, T{}, F{});
            kstep(kt + 1, S1{}, T{}, T{}, F{});
        }
        kstep(kt, S0{}, T{}, F{}, F{});
        kstep(kt + 1, S1{}, F{}, F{}, F{});
    } else {
        // Only the last two slabs can cross K (KT is rounded up to even); the steps that
        // publish them are peeled off so that the steady-state loop carries no fix-up code.
        if (KT >= 4) {
            for (; kt + 4 < KT; kt += 2) {
                kstep(kt, S0{}, T{}, T{}, F{});
                kstep(kt + 1, S1{}, T{}, T{}, F{});
            }
            kstep(kt, S0{}, T{}, T{}, F{});
            kstep(kt + 1, S1{}, T{}, T{}, T{});
            kt += 2;
        }
        kstep(kt, S0{}, T{}, F{}, T{});
        // the surplus slab of an odd number of 64-deep slabs is all zeros: its step is skipped
        if ((kt + 1) * BK < K) kstep(kt + 1, S1{}, F{}, F{}, F{});
    }

    long long tr_store = 0;
    if constexpr (TRACE) {
        tr_store = tr_now();
        tr_loop = tr_store - tr_loop;
    }
    // ---- K groups: the second group's accumulators pass through its (drained) stages, 16
    //      bytes per lane and tile, to the wave of the first group that owns the same sub-tile;
    //      the sum is (first half of K) + (second half), a fixed order ----
    if constexpr (Cfg::KG > 1) {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");     // every wave is done with the last stage
        f32x4_t* hand = (f32x4_t*)(lds_all + Cfg::LDS_GROUP) + (wave * (MI * NI)) * 64 + lane;
        if (kg == 1) {
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) hand[(i * NI + j) * 64] = acc[i][j];
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (kg == 1) return;            // (waves that have ended no longer count at the barriers below)
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const f32x4_t v = hand[(i * NI + j) * 64];
                acc[i][j][0] += v[0]; acc[i][j][1] += v[1]; acc[i][j][2] += v[2]; acc[i][j][3] += v[3];
            }
    }
    // ---- epilogue: C tile -> storage type -> per-wave LDS staging -> 16-byte row stores ----
    // acc[i][j][e] of lane l is C[m][n], m = i*16 + (l & 15), n = j*16 + 4*(l >> 4) + e
    unsigned char* Cb = (unsigned char*)p.C + (size_t)row0 * p.ldc * 2;
    const uint32_t bytesC = (uint32_t)(rowsA * p.ldc) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcC = __builtin_amdgcn_make_buffer_rsrc((void*)Cb, 0, (int)bytesC, 0x00020000);
    // split-K: fp32 partial tile -> ws[split][m][n], 16 bytes per lane straight from the
    // accumulators (N % 4 == 0 is a launch precondition); splitk_reduce_kernel adds the
    // splits in order, applies alpha / beta and rounds once
    auto store_partials = [&]() __attribute__((always_inline)) {
        // descriptor over this tile's rows of the split's M x N fp32 matrix: rows past M fall
        // outside it and are dropped by the range check (the host keeps M*N*4 below 2^31)
        float* P = p.ws + ((size_t)blockIdx.y * M + row0) * N;
        const __amdgpu_buffer_rsrc_t rsrcP =
            __builtin_amdgcn_make_buffer_rsrc((void*)P, 0, (int)((uint32_t)(rowsA * N) * 4u), 0x00020000);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int m_loc = wm * TM + i * 16 + l16;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int n = col0 + wn * TN + j * 16 + 4 * q;
                const uint32_t off = (uint32_t)(m_loc * N + n) * 4u;
                if (!EDGE || n < N)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, acc[i][j]), rsrcP, off, 0, 0);
            }
        }
    };
    auto epilogue = [&](auto scaled_c) __attribute__((always_inline)) {
        // alpha / beta epilogue (see scale_acc): a second copy of this block behind a uniform branch
        constexpr bool SCALED = decltype(scaled_c)::value;
        const float alpha = p.alpha, beta = p.beta;
        // The predicated variant masks rows past M, stores 16 bytes at any 2-byte boundary
        // (odd N) and splits only the chunk that straddles N into 2-byte stores.
        // C is written once and not read again here: in the aligned variant non-temporal stores
        // (cache policy bit 1) keep it from displacing A and B panels in the memory-side cache
        // and L2 (measured: loads arrive sooner, 2385 -> 2363 cycles per K step, +1.5 % at
        // 8192^3).  Not in the predicated variant: its stores may cover parts of cache lines
        // (rows at odd offsets), which non-temporal writes do not merge (-4 % at 4095x6143x3073).
        constexpr int C_STORE_POLICY = EDGE ? 0 : 2;
        constexpr int CPR = TN / 8;                 // 16-byte chunks per row of the wave tile
        constexpr bool POW2 = (CPR & (CPR - 1)) == 0;
        static_assert(CPR % 2 == 0 && (TM * CPR) % 64 == 0, "C staging layout");
        // rows of a power-of-two width are spread over the banks by the row number, 192-byte
        // rows (4 rows = 3 bank rounds) by row / 4
        auto cswz = [](int row) __attribute__((always_inline)) {
            return POW2 ? (row & (CPR - 1)) : ((row >> 2) & 3);
        };
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // all waves done with the last stage
        unsigned char* stg = lds + wave * (TM * TN * 2);
        // In pieces of 32 rows (where they are whole numbers of 64-lane store instructions): the
        // stores of one piece drain while the next is converted, instead of 128 KB per CU queueing
        // up at once.
        constexpr int CH_ROWS = (TM % 32 == 0 && (32 * CPR) % 64 == 0) ? 32 : TM;
#pragma unroll
        for (int c = 0; c < TM / CH_ROWS; ++c) {
#pragma unroll
        for (int i = c * (CH_ROWS / 16); i < (c + 1) * (CH_ROWS / 16); ++i) {
            const int row = i * 16 + l16;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int chunk = (j * 2 + (q >> 1)) ^ cswz(row);
                u32x2_t w;
                w[0] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][0], alpha, beta), scale_acc<SCALED>(acc[i][j][1], alpha, beta));
                w[1] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][2], alpha, beta), scale_acc<SCALED>(acc[i][j][3], alpha, beta));
                *(u32x2_t*)(stg + row * (TN * 2) + chunk * 16 + (q & 1) * 8) = w;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int r = c * (CH_ROWS * CPR / 64); r < (c + 1) * (CH_ROWS * CPR / 64); ++r) {
            // chunk r*64 + lane of the wave tile, rows first
            const int idx = r * 64 + lane;
            const int row = POW2 ? r * (64 / CPR) + lane / CPR : idx / CPR;
            const int rc = POW2 ? lane % CPR : idx % CPR;
            const u32x4_t v = *(const u32x4_t*)(stg + row * (TN * 2) + ((rc ^ cswz(row)) << 4));
            const int m_loc = wm * TM + row;
            const int n = col0 + wn * TN + rc * 8;
            const uint32_t off = (uint32_t)(m_loc * p.ldc + n) * 2u;
            if constexpr (!EDGE) {
                __builtin_amdgcn_raw_buffer_store_b128(v, rsrcC, off, 0, C_STORE_POLICY);
            } else {
                if (m_loc < rowsA) {
                    if (n + 7 < N) {
                        __builtin_amdgcn_raw_buffer_store_b128(v, rsrcC, off, 0, C_STORE_POLICY);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (n + e < N)
                                __builtin_amdgcn_raw_buffer_store_b16(
                                    (uint16_t)(v[e >> 1] >> ((e & 1) * 16)), rsrcC, off + 2 * e, 0, C_STORE_POLICY);
                    }
                }
            }
        }
        }
    };
    if constexpr (SPLITK) {
        store_partials();
    } else if constexpr (MI_ABLATED(8)) {
        // (ablation bit 3: no epilogue at all -- what hiding it completely could gain at most)
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j) asm volatile("" :: "a"(acc[i][j]));
    } else {
        if (p.alpha != 1.0f || p.beta != 0.0f) epilogue(std::true_type{});
        else epilogue(std::false_type{});
    }
    if constexpr (TRACE) {
        if (p.DB != nullptr && tid == 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            tr_store = tr_now() - tr_store;
            int* rec = p.DB + 6 * ((size_t)blockIdx.y * gridDim.x + blockIdx.x);      // (blockIdx.y: the piece of a split-K launch)
            rec[0] = (int)tr_wait;
            rec[1] = tr_cnt;
            rec[2] = (int)tr_loop;
            rec[3] = KT;
            rec[4] = (int)tr_store;
            rec[5] = 1;
        }
    }
}

// ---------------------------------------------------------------------------------------
// Ring variant: K slab = one 32-deep MFMA slice (64-byte LDS rows, chunks stored at
// chunk ^ ((row >> 2) & 3)), NS stages, loads issued NS slabs ahead and dealt out one per
// few MFMAs (spread evenly over the slots that follow the fragment reads, so that the four
// or eight waves of a CU do not queue up at the texture addresser), `vmcnt((NS-2)*L)` waits
// (never on the youngest loads), one barrier per slab.
// A slab has NS-1 steps (~3000 cycles at NS = 4) to land instead of ~1.
template <int BM_, int BN_, int WM_, int WN_, int NS_, int GROUP_, int DT_>
struct Ring16Config {
    static constexpr int BM = BM_, BN = BN_, BK = 32;
    static constexpr int WM = WM_, WN = WN_, NS = NS_, GROUP = GROUP_, DT = DT_;
    static constexpr int NT = WM * WN * 64, NW = WM * WN;
    static constexpr int TM = BM / WM, TN = BN / WN;
    static constexpr int MI = TM / 16, NI = TN / 16;
    static constexpr int RPP = NW * 16;                  // rows one pass of all waves loads (16 per wave)
    static constexpr int LA = BM / RPP, LB = BN / RPP;
    static constexpr int L = LA + LB;
    static constexpr int A_STAGE = BM * 64, B_STAGE = BN * 64, STAGE = A_STAGE + B_STAGE;
    static constexpr int LDS_BYTES = NS * STAGE;
    static constexpr int WAVES_PER_EU = NT / 256;
    static constexpr int NMMA = MI * NI, NFR = MI + NI;
    static constexpr int DSP = (NMMA - NFR) / L;         // MFMA slots between two load instructions
    static_assert(NT == 256 || NT == 512, "one or two waves per SIMD");
    static_assert(TM % 16 == 0 && TN % 16 == 0, "wave tile must be a multiple of 16x16");
    static_assert(BM % RPP == 0 && BN % RPP == 0, "tile rows divide over the waves");
    static_assert(DSP >= 1, "reads and loads each get an MFMA slot");
    static_assert(NS >= 3 && NS <= 5 && (NS - 1) * L <= 63, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
    static_assert(BM * BN * 2 <= LDS_BYTES, "the epilogue stages the C tile in the ring");
};

template <class Cfg, bool TRACE = false>
__global__ void __launch_bounds__(Cfg::NT)
__attribute__((amdgpu_waves_per_eu(Cfg::WAVES_PER_EU, Cfg::WAVES_PER_EU)))
gemm_ring16_kernel(const GemmArgs p) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, WN = Cfg::WN;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, LA = Cfg::LA, L = Cfg::L, RPP = Cfg::RPP;
    constexpr int A_STAGE = Cfg::A_STAGE, STAGE = Cfg::STAGE;
    constexpr int NMMA = Cfg::NMMA, NFR = Cfg::NFR, DT = Cfg::DT;
    constexpr int TM = Cfg::TM, TN = Cfg::TN;

    __shared__ __attribute__((aligned(128))) unsigned char lds[Cfg::LDS_BYTES];

    long long tr_wait = 0, tr_t0 = 0, tr_loop = 0;
    int tr_cnt = 0;
    auto tr_now = [&]() __attribute__((always_inline)) { return (long long)__builtin_readcyclecounter(); };
    if constexpr (TRACE) tr_loop = tr_now();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;

    int tm, tn;
    tile_of_block<Cfg::GROUP>(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
    const int row0 = tm * BM, col0 = tn * BN;
    const int K = p.K;
    const int KT = K / 32;                               // slabs; host checks K % (32*NS) == 0

    const unsigned char* Ab = (const unsigned char*)p.A + (size_t)row0 * p.lda * 2;
    const unsigned char* Bb = (const unsigned char*)p.B + (size_t)col0 * p.ldb * 2;
    const uint32_t bytesA = (uint32_t)((BM - 1) * p.lda + K) * 2u;
    const uint32_t bytesB = (uint32_t)((BN - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcNone = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, 0, 0x00020000);

    // one load instruction fills 16 rows x 64 bytes: lane l -> row l >> 2, chunk position l & 3
    const int dr = lane >> 2;
    const int dchunk = (lane & 3) ^ ((dr >> 2) & 3);
    const uint32_t dvoffA = (uint32_t)((wave * 16 + dr) * p.lda + dchunk * 8) * 2u;
    const uint32_t dvoffB = (uint32_t)((wave * 16 + dr) * p.ldb + dchunk * 8) * 2u;
    const uint32_t passA = (uint32_t)(RPP * p.lda) * 2u;
    const uint32_t passB = (uint32_t)(RPP * p.ldb) * 2u;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const uint32_t dlds = lds_base + (uint32_t)wave * 1024u;
    auto dma = [&](const __amdgpu_buffer_rsrc_t& rsrc, uint32_t voff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
    };
    auto dma_one = [&](int t, int s, int d) __attribute__((always_inline)) {
        const uint32_t kb = (uint32_t)t * 64u;
        const bool live = t < KT;
        if (d < LA)
            dma(live ? rsrcA : rsrcNone, dvoffA + kb + d * passA, dlds + s * STAGE + d * (RPP * 64));
        else
            dma(live ? rsrcB : rsrcNone, dvoffB + kb + (d - LA) * passB,
                dlds + s * STAGE + A_STAGE + (d - LA) * (RPP * 64));
    };

    // fragment reads: lane holds row (lane & 15), chunk (lane >> 4) of the 64-byte row
    const int l16 = lane & 15, q = lane >> 4;
    const int rd_off = l16 * 64 + ((q ^ ((l16 >> 2) & 3)) << 4);
    const int a_wave = wm * TM * 64;
    const int b_wave = A_STAGE + wn * TN * 64;

    u32x4_t fa[2][MI], fb[2][NI];
    f32x4_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.0f;

    auto mma_one = [&](int buf, int idx) __attribute__((always_inline)) {
        const int i = idx / NI, j = idx % NI;
        acc[i][j] = mfma_16x16x32<DT>(fb[buf][j], fa[buf][i], acc[i][j]);
    };
    auto read_one = [&](int s, int buf, int r) __attribute__((always_inline)) {
        if (r == 0 || r > NI) {
            const int i = r == 0 ? 0 : r - NI;
            fa[buf][i] = *(const u32x4_t*)(lds + s * STAGE + a_wave + i * 1024 + rd_off);
        } else {
            const int j = r - 1;
            fb[buf][j] = *(const u32x4_t*)(lds + s * STAGE + b_wave + j * 1024 + rd_off);
        }
    };

    // ---- prologue: slabs 0 .. NS-1 ----
#pragma unroll
    for (int t = 0; t < NS; ++t)
#pragma unroll
        for (int d = 0; d < L; ++d) dma_one(t, t, d);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"((NS - 1) * L) : "memory");    // slab 0 is in
#pragma unroll
    for (int r = 0; r < NFR; ++r) read_one(0, 0, r);

    // One slab.  Fragments of slab t are in register buffer `buf`; stage s held slab t and is
    // idle (its fragments were fetched during the previous step).
    //   vmcnt((NS-2)*L) + barrier : slab t+1 has landed for every wave
    //   32 MFMAs | fetch fragments of slab t+1 | loads of slab t+NS into stage s
    auto step = [&](int t, auto s_c, auto buf_c) __attribute__((always_inline)) {
        constexpr int s = decltype(s_c)::value, buf = decltype(buf_c)::value;
        constexpr int sn = (s + 1) % NS;
        if constexpr (TRACE) tr_t0 = tr_now();
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"((NS - 2) * L) : "memory");
        if constexpr (TRACE) { tr_wait += tr_now() - tr_t0; ++tr_cnt; }
#pragma unroll
        for (int idx = 0; idx < NMMA; ++idx) {
            mma_one(buf, idx);
            if (idx < NFR) read_one(sn, buf ^ 1, idx);
            const int d = idx - NFR;
            if (d >= 0 && d % Cfg::DSP == 0 && d / Cfg::DSP < L) dma_one(t + NS, s, d / Cfg::DSP);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    static_assert(NS == 4, "the step loop below is unrolled for a ring of four");
    for (int t0 = 0; t0 < KT; t0 += 4) {
        step(t0, std::integral_constant<int, 0>{}, B0{});
        step(t0 + 1, std::integral_constant<int, 1>{}, B1{});
        step(t0 + 2, std::integral_constant<int, 2>{}, B0{});
        step(t0 + 3, std::integral_constant<int, 3>{}, B1{});
    }
    // requests past K are still heading for the ring: drain before reusing it
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");

    long long tr_store = 0;
    if constexpr (TRACE) {
        tr_store = tr_now();
        tr_loop = tr_store - tr_loop;
    }
    unsigned char* Cb = (unsigned char*)p.C + (size_t)row0 * p.ldc * 2;
    const uint32_t bytesC = (uint32_t)(BM * p.ldc) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcC = __builtin_amdgcn_make_buffer_rsrc((void*)Cb, 0, (int)bytesC, 0x00020000);
    auto epilogue = [&](auto scaled_c) __attribute__((always_inline)) {
        constexpr bool SCALED = decltype(scaled_c)::value;   // alpha / beta epilogue: second copy behind a uniform branch
        const float alpha = p.alpha, beta = p.beta;
        constexpr int CPR = TN / 8;
        constexpr int RPI = 64 / CPR;
        unsigned char* stg = lds + wave * (TM * TN * 2);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int row = i * 16 + l16;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int chunk = (j * 2 + (q >> 1)) ^ (row & (CPR - 1));
                u32x2_t w;
                w[0] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][0], alpha, beta), scale_acc<SCALED>(acc[i][j][1], alpha, beta));
                w[1] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][2], alpha, beta), scale_acc<SCALED>(acc[i][j][3], alpha, beta));
                *(u32x2_t*)(stg + row * (TN * 2) + chunk * 16 + (q & 1) * 8) = w;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const int rr = lane / CPR, rc = lane % CPR;
        const uint32_t cbase = (uint32_t)((wm * TM + rr) * p.ldc + col0 + wn * TN + rc * 8) * 2u;
#pragma unroll
        for (int r = 0; r < TM / RPI; ++r) {
            const int row = r * RPI + rr;
            const u32x4_t v = *(const u32x4_t*)(stg + row * (TN * 2) + ((rc ^ (row & (CPR - 1))) << 4));
            __builtin_amdgcn_raw_buffer_store_b128(v, rsrcC, cbase + (uint32_t)(r * RPI * p.ldc) * 2u, 0, 0);
        }
    };
    if (p.alpha != 1.0f || p.beta != 0.0f) epilogue(std::true_type{});
    else epilogue(std::false_type{});
    if constexpr (TRACE) {
        if (p.DB != nullptr && tid == 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            tr_store = tr_now() - tr_store;
            int* rec = p.DB + 6 * (size_t)blockIdx.x;
            rec[0] = (int)tr_wait;
            rec[1] = tr_cnt;
            rec[2] = (int)tr_loop;
            rec[3] = KT;
            rec[4] = (int)tr_store;
            rec[5] = 1;
        }
    }
}

template <class Cfg, bool TRACE = false>
hipError_t launch_ring16_kernel(const GemmArgs& args, hipStream_t stream) {
    const int grid = args.tiles_m * args.tiles_n;
    return launch_kernel(gemm_ring16_kernel<Cfg, TRACE>, dim3(grid), dim3(Cfg::NT), stream, args);
}

template <class Cfg, bool TRACE = false>
hipError_t launch_mfma16_kernel(const GemmArgs& args, hipStream_t stream) {
    const int grid = args.tiles_m * args.tiles_n;
    if (args.splits > 1) {
        if constexpr (Cfg::KG == 1)
            return launch_kernel(gemm_mfma16_kernel<Cfg, TRACE, true>, dim3(grid, args.splits), dim3(Cfg::NT), stream, args);
        else
            return hipErrorInvalidValue;        // K is already split inside the workgroup
    }
    return launch_kernel(gemm_mfma16_kernel<Cfg, TRACE>, dim3(grid), dim3(Cfg::NT), stream, args);
}

}  // namespace mi
