// gemm_ring_kernel.hpp -- the aligned-shape gfx950 GEMM kernel: a ring of NS LDS stages,
// each one K slab of 32 elements, filled by direct-to-LDS buffer loads that run NS-1 slabs
// ahead of the MFMAs.
//
//   C[M,N] = A[M,K] . B[N,K]^T     M % BM == 0, N % BN == 0, K % (32*NS) == 0, 16-byte aligned
//
// Compared with the two-stage kernel of gemm_kernel.hpp (which remains the predicated
// kernel for ragged shapes) the K step is halved and the ring deepened, so that
//   * the global -> LDS loads of a slab are dealt out evenly, one per few MFMAs, over the
//     whole time a slab is being multiplied, instead of in a burst after the barrier (the
//     burst backs up the CU's single load path and stalls the MFMA issue of every wave);
//   * a slab has about 2.5 K steps to land instead of 0.75;
//   * no wait ever covers the youngest loads: `s_waitcnt vmcnt((NS-2)*L)` asks only for
//     the slab needed next (loads retire in order).
// It stands where the TMA + mbarrier full/empty ring of the reference's kernels stands
// (matmul_utils.cuh:394-456, 505-526; matmul_h100.cu.jinja:122-263): the ring is the same
// idea, the mechanism is buffer_load ... lds + s_waitcnt + one s_barrier per slab.
//
// LDS stage layout: [A: BM rows x 64 bytes][B: BN rows x 64 bytes]; a row is four 16-byte
// chunks stored at  chunk ^ ((row >> 2) & 3)  so that the ds_read_b128 fragment reads of 16
// consecutive rows cover all 64 banks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "gemm_kernel.hpp"

namespace mi {

template <int BM_, int BN_, int WM_, int WN_, int NS_, int GROUP_, int DT_>
struct RingConfig {
    static constexpr int BM = BM_, BN = BN_, BK = 32;
    static constexpr int WM = WM_, WN = WN_, NS = NS_, GROUP = GROUP_, DT = DT_;
    static constexpr int NT = WM * WN * 64, NW = WM * WN;
    static constexpr int TM = BM / WM, TN = BN / WN;
    static constexpr int MI = TM / 32, NI = TN / 32;
    static constexpr int RPP = NW * 16;                 // tile rows one pass of all waves loads
    static constexpr int LA = BM / RPP, LB = BN / RPP;  // load instructions per wave per slab
    static constexpr int L = LA + LB;
    static constexpr int A_STAGE = BM * 64, B_STAGE = BN * 64, STAGE = A_STAGE + B_STAGE;
    static constexpr int LDS_BYTES = NS * STAGE;
    static constexpr int WAVES_PER_EU = NT / 256 > 0 ? NT / 256 : 1;
    static constexpr int NMMA = MI * NI, NFR = MI + NI;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(BM % RPP == 0 && BN % RPP == 0, "tile rows must divide over the waves");
    static_assert(L % 2 == 0 && L / 2 <= NMMA - NFR, "load slots follow the fragment reads");
    static_assert(NS >= 3 && (NS - 2) * L <= 63, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
    static_assert(BM * BN * 2 <= LDS_BYTES, "the epilogue stages the C tile in the ring");
};

template <class Cfg, bool TRACE = false>
__global__ void __launch_bounds__(Cfg::NT)
__attribute__((amdgpu_waves_per_eu(Cfg::WAVES_PER_EU, Cfg::WAVES_PER_EU)))
gemm_ring_kernel(const GemmArgs p) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, WN = Cfg::WN;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, LA = Cfg::LA, LB = Cfg::LB, L = Cfg::L;
    constexpr int RPP = Cfg::RPP, A_STAGE = Cfg::A_STAGE, STAGE = Cfg::STAGE;
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
    const int KT = K / 32;                       // K slabs; a multiple of NS (host checks)

    // ---- global side ----
    const unsigned char* Ab = (const unsigned char*)p.A + (size_t)row0 * p.lda * 2;
    const unsigned char* Bb = (const unsigned char*)p.B + (size_t)col0 * p.ldb * 2;
    // Descriptors end with the tile's last row: slabs requested past K (the ring keeps
    // asking NS slabs ahead) fall outside for every row but would alias the next row for
    // the others, so those requests use the empty descriptor instead.
    const uint32_t bytesA = (uint32_t)((BM - 1) * p.lda + K) * 2u;
    const uint32_t bytesB = (uint32_t)((BN - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcNone = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, 0, 0x00020000);

    // A load instruction fills 16 consecutive 64-byte rows: lane l lands on chunk position
    // l & 3 of row l >> 2, so it fetches logical chunk (l & 3) ^ swz(row).  The row index of
    // pass j is j*RPP + wave*16 + (l >> 2); its swizzle depends only on the lane.
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
    // load instruction d (0 .. L-1) of K slab t into ring stage s
    auto dma_one = [&](int t, int s, int d) __attribute__((always_inline)) {
        const uint32_t kb = (uint32_t)t * 64u;
        const bool live = t < KT;
        if (d < LA)
            dma(live ? rsrcA : rsrcNone, dvoffA + kb + d * passA, dlds + s * STAGE + d * (RPP * 64));
        else
            dma(live ? rsrcB : rsrcNone, dvoffB + kb + (d - LA) * passB,
                dlds + s * STAGE + A_STAGE + (d - LA) * (RPP * 64));
    };

    // ---- LDS side: fragment reads ----
    const int l32 = lane & 31, hi = lane >> 5;
    int rd_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) rd_off[ks] = l32 * 64 + ((((ks << 1) | hi) ^ ((l32 >> 2) & 3)) << 4);
    const int a_wave = wm * TM * 64;
    const int b_wave = A_STAGE + wn * TN * 64;

    u32x4_t fa[2][MI], fb[2][NI];
    f32x16_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto mma_one = [&](int buf, int idx) __attribute__((always_inline)) {
        const int i = idx / NI, j = idx % NI;
        acc[i][j] = mfma_32x32x16<DT>(fb[buf][j], fa[buf][i], acc[i][j]);
    };
    // fragment r of a k slice in the order the MFMAs first need them: A0, B0..B(NI-1), A1..
    auto read_one = [&](int s, int ks, int buf, int r) __attribute__((always_inline)) {
        if (r == 0 || r > NI) {
            const int i = r == 0 ? 0 : r - NI;
            fa[buf][i] = *(const u32x4_t*)(lds + s * STAGE + a_wave + i * 2048 + rd_off[ks]);
        } else {
            const int j = r - 1;
            fb[buf][j] = *(const u32x4_t*)(lds + s * STAGE + b_wave + j * 2048 + rd_off[ks]);
        }
    };

    // ---- prologue: slabs 0 .. NS-2 and the first half of slab NS-1 (the steady-state
    // schedule below issues the second half in its first slice) ----
    constexpr int LH = L / 2;
#pragma unroll
    for (int t = 0; t < NS; ++t)
#pragma unroll
        for (int d = 0; d < (t == NS - 1 ? LH : L); ++d) dma_one(t, t, d);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"((NS - 2) * L + LH) : "memory");   // slab 0 is in
#pragma unroll
    for (int r = 0; r < NFR; ++r) read_one(0, 0, 0, r);

    // One K slab (two 16-deep slices).  Stage s holds slab t.
    //   slice 0 : MFMA | fetch fragments of slice 1 | second half of the loads of slab t+NS-1
    //   vmcnt((NS-2)*L) + barrier : slab t+1 has landed for every wave; stage s is drained
    //   slice 1 : MFMA | fetch fragments of slice 0 of slab t+1 | first half of the loads of
    //             slab t+NS into stage s
    auto step = [&](int t, auto s_c) __attribute__((always_inline)) {
        constexpr int s = decltype(s_c)::value;
        constexpr int sn = (s + 1) % NS, sp = (s + NS - 1) % NS;
#pragma unroll
        for (int idx = 0; idx < NMMA; ++idx) {
            mma_one(0, idx);
            if (idx < NFR) read_one(s, 1, 1, idx);
            if (idx >= NMMA - LH) dma_one(t + NS - 1, sp, LH + idx - (NMMA - LH));
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (TRACE) tr_t0 = tr_now();
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"((NS - 2) * L) : "memory");
        if constexpr (TRACE) { tr_wait += tr_now() - tr_t0; ++tr_cnt; }
#pragma unroll
        for (int idx = 0; idx < NMMA; ++idx) {
            mma_one(1, idx);
            if (idx < NFR) read_one(sn, 0, 0, idx);
            if (idx >= NMMA - LH) dma_one(t + NS, s, idx - (NMMA - LH));
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for (int t0 = 0; t0 < KT; t0 += NS) {
        if constexpr (NS == 3) {
            step(t0, std::integral_constant<int, 0>{});
            step(t0 + 1, std::integral_constant<int, 1>{});
            step(t0 + 2, std::integral_constant<int, 2>{});
        } else {
            static_assert(NS == 4, "ring depth");
            step(t0, std::integral_constant<int, 0>{});
            step(t0 + 1, std::integral_constant<int, 1>{});
            step(t0 + 2, std::integral_constant<int, 2>{});
            step(t0 + 3, std::integral_constant<int, 3>{});
        }
    }
    // requests past K are still in flight towards the ring: drain before reusing it
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");

    long long tr_store = 0;
    if constexpr (TRACE) {
        tr_store = tr_now();
        tr_loop = tr_store - tr_loop;
    }
    // ---- epilogue: C tile through LDS, 16 bytes per lane, whole row segments ----
    unsigned char* Cb = (unsigned char*)p.C + (size_t)row0 * p.ldc * 2;
    const uint32_t bytesC = (uint32_t)(BM * p.ldc) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcC = __builtin_amdgcn_make_buffer_rsrc((void*)Cb, 0, (int)bytesC, 0x00020000);
    auto epilogue = [&](auto scaled_c) __attribute__((always_inline)) {
        constexpr bool SCALED = decltype(scaled_c)::value;   // alpha / beta epilogue: see scale_acc
        const float alpha = p.alpha, beta = p.beta;
        constexpr int CPR = TN / 8;
        constexpr int RPI = 64 / CPR;
        unsigned char* stg = lds + wave * (TM * TN * 2);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int row = i * 32 + l32;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int chunk = (j * 4 + g) ^ (row & (CPR - 1));
                    u32x2_t w;
                    w[0] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][g * 4 + 0], alpha, beta),
                                          scale_acc<SCALED>(acc[i][j][g * 4 + 1], alpha, beta));
                    w[1] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][g * 4 + 2], alpha, beta),
                                          scale_acc<SCALED>(acc[i][j][g * 4 + 3], alpha, beta));
                    *(u32x2_t*)(stg + row * (TN * 2) + chunk * 16 + hi * 8) = w;
                }
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
hipError_t launch_ring_kernel(const GemmArgs& args, hipStream_t stream) {
    const int grid = args.tiles_m * args.tiles_n;
    return launch_kernel(gemm_ring_kernel<Cfg, TRACE>, dim3(grid), dim3(Cfg::NT), stream, args);
}

}  // namespace mi
