// gemm_decode_kernel.hpp -- gfx950 split-K GEMM kernel for decode shapes with 32 < M <= 128:
//
//   C[M,N] = A[M,K] . B[N,K]^T     M small, B (the weights) streamed once from HBM
//
// The read of B is the cost.  Measured on MI355X with read-only probes of this access
// pattern: a CU pulls at most ~26 GB/s from HBM however many bytes it keeps in flight (its L1
// tracks a bounded number of missing lines), so every CU has to pull, and whatever else goes
// through a CU's L1 -- the A operand -- is paid for in B bandwidth; 256 CUs together reach
// ~5.9 TB/s.  The kernel is built around that:
//   * a workgroup owns BN = 128 rows of B and one contiguous piece of K (split-K over
//     blockIdx.y, as many pieces as give every CU a workgroup); it starts its walk over the
//     piece's 64-deep slabs at a slab of its own and wraps around, so that the requests in
//     flight on the chip do not share their low address bits (the same few HBM channels);
//   * B slabs (128 rows x 128 bytes, XOR-swizzled) go global -> LDS through direct-to-LDS
//     buffer loads marked non-temporal (B is read once: left to the default policy it pushes A
//     out of the L2s; 26.2 -> 23.1 us for the B stream of 128 x 8192 x 8192) into a ring of NS
//     stages of 16 KB; NS-2 slabs are always in flight.  A deeper ring is slower, not faster
//     (NS = 3 / 4 / 8: 35.5 / 36.1 / 38.6 us at M = 128);
//   * the four waves split M: wave w owns rows w*BM/4 .. of A and all 128 columns.  Both
//     operands are K-contiguous, which is the fragment layout of v_mfma_f32_16x16x32 (lane l:
//     row l & 15, 8 consecutive k at chunk l >> 4), so a wave's A fragments are plain 16-byte
//     buffer loads from L2 (A is at most 128 x K and stays there) into a register ring as
//     deep as the LDS ring -- `vmcnt` retires loads in order, so the A fragments of a slab are
//     requested together with its B rows, NS-1 slabs ahead, and A never passes through LDS;
//   * the loads of a request are dealt out between the MFMAs of the slab before (one per four
//     MFMAs at M = 128): a steady trickle instead of a burst per slab (39.3 -> 36.1 us);
//   * one s_barrier per slab; waits are `vmcnt((NS-2)*L)`, never on the youngest loads;
//   * with split-K the fp32 partial tiles go to a workspace and splitk_reduce_kernel adds
//     them in split order (a fixed order: reproducible) and rounds once; without split-K the
//     tile is rounded and stored directly.
// Where the time goes at 128 x 8192 x 8192 (four pieces, parts of the kernel switched off one
// by one): B stream alone 22.7 us (the read-only probe: 22.5), + A loads, fragment reads and
// MFMAs 27.4, + partial-sum stores 31, + the reduction launch 35.5.
// Rows of A past M and rows of B past N are never fetched (the buffer descriptors end at the
// last valid row; out-of-range loads return zero).  The reference has no counterpart: its
// kernels assert M % 128 == 0 (matmul_utils.cuh:362,386-387).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "gemm_kernel.hpp"
#include "gemm_mfma16_kernel.hpp"   // mfma_16x16x32
#include "splitk_common.hpp"   // DecodeArgs, splitk_reduce_kernel

namespace mi {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), in order
template <class F, int... Is>
__device__ __forceinline__ void static_for_each(F&& f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_each(f, std::make_integer_sequence<int, N>{});
}

template <int BM_, int BN_, int NS_, int DT_>
struct DecodeConfig {
    static constexpr int BM = BM_, BN = BN_, NS = NS_, DT = DT_;
    static constexpr int NT = 256, NW = 4;
    static constexpr int TM = BM / NW;                       // rows of A (of C) one wave owns
    static constexpr int MI = TM / 16, NI = BN / 16;         // 16x16 accumulator tiles per wave
    static constexpr int STAGE = BN * 128;                   // one B slab: BN rows x 64 k
    static constexpr int LB = BN / 8 / NW;                   // direct-to-LDS loads per wave per slab
    static constexpr int LA = MI * 2;                        // A fragment loads per wave per slab
    static constexpr int L = LA + LB;
    static constexpr int LDS_BYTES = NS * STAGE;
    static_assert(TM % 16 == 0 && BN % 32 == 0, "wave tile is whole 16x16 MFMA tiles");
    static_assert(NS >= 3 && (NS - 1) * L <= 63, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

// TRACE: the per-workgroup timing record (TraceRec) for launches that pass a trace buffer.
template <class Cfg, bool TRACE = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
gemm_decode_kernel(const DecodeArgs p) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, DT = Cfg::DT;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, TM = Cfg::TM, LA = Cfg::LA, LB = Cfg::LB, L = Cfg::L;
    constexpr int STAGE = Cfg::STAGE;
    (void)BM;

    __shared__ __attribute__((aligned(128))) unsigned char lds[Cfg::LDS_BYTES];
    TraceRec<TRACE> tr;
    tr.begin();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col0 = blockIdx.x * BN;
    const int split = blockIdx.y;
    const int M = p.M, N = p.N, K = p.K;
    const int S = p.splits;
    // this split's slabs: the contiguous range [split * KTB, split * KTB + KT), KT >= 1
    const int KTB = p.k_per_split / 64;
    const int KT = (K / 64 - split * KTB) < KTB ? (K / 64 - split * KTB) : KTB;

    const int row0 = wave * TM;                              // this wave's rows of A
    const int rowsA = (M - row0) < TM ? (M - row0) : TM;     // may be <= 0: the wave then multiplies zeros
    const int rowsB = (N - col0) < BN ? (N - col0) : BN;
    const unsigned char* Ab = (const unsigned char*)p.A + (size_t)row0 * p.lda * 2;
    const unsigned char* Bb = (const unsigned char*)p.B + (size_t)col0 * p.ldb * 2;
    // descriptors end at the last element of the last valid row
    const uint32_t bytesA = rowsA > 0 ? (uint32_t)((rowsA - 1) * p.lda + K) * 2u : 0u;
    const uint32_t bytesB = (uint32_t)((rowsB - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcNone = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, 0, 0x00020000);

    // B: one load instruction fills 8 consecutive 128-byte rows of a stage; lane l lands on
    // chunk position l & 7 of row l >> 3 and fetches logical chunk (l & 7) ^ swz(row).
    // Instruction q = wave + 4*i of a slab covers stage rows 8q .. 8q+7.
    const int lr = lane >> 3, lc = lane & 7;
    auto swz = [](int row) __attribute__((always_inline)) { return (row >> 1) & 7; };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    auto dma = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
    };
    uint32_t voffB[LB];
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = (wave + i * 4) * 8 + lr;
        voffB[i] = (uint32_t)(row * p.ldb + (lc ^ swz(row)) * 8) * 2u;
    }
    // A: fragment (i, ks) of a slab is row i*16 + (lane & 15), k chunk 4*ks + (lane >> 4)
    const int l16 = lane & 15, q4 = lane >> 4;
    uint32_t voffA[MI];
#pragma unroll
    for (int i = 0; i < MI; ++i) voffA[i] = (uint32_t)((i * 16 + l16) * p.lda + q4 * 8) * 2u;

    // Slab t of the loop is this split's slab (t + rot) mod KT, i.e. slab split + S * that of
    // the matrix.  `gs` follows the slab being requested, `issued` counts requested slabs;
    // requests past the split's last slab go through an empty descriptor (no memory access).
    int gs = (int)((blockIdx.x * 5u) % (unsigned)KT);
    int issued = 0;
    // A fragments arrive through inline asm like the B rows, so that every wait on `vmcnt` in
    // this kernel is an explicit one (the compiler, which cannot see the direct-to-LDS loads,
    // would otherwise wait for too many).
    // INVARIANT: between the asm statement that loads into a register of `areg` and the
    // wait_slab() that retires that load, no instruction reads or writes that register.  Two
    // things hold it up.  In the source, a register set is an in/out operand of every asm
    // statement that concerns it -- the loads (so a set is live from its first load to the
    // kernel's last wait, whether or not a later slab still reads it: it is never a dead value
    // whose registers the allocator may hand out) and the waits (so nothing that uses a set can
    // be moved above the wait that retires its loads) -- and only MFMAs behind such a wait read
    // it.  In the build, since the source cannot forbid the allocator to copy or move a live
    // value, isa_check.check_inflight follows the generated code of this kernel and refuses to
    // link when any instruction touches a register with one of these loads still in flight.
    u32x4_t areg[NS][LA];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int i = 0; i < LA; ++i) areg[s][i] = u32x4_t{0u, 0u, 0u, 0u};
    auto load_a = [](u32x4_t& dst, __amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, auto imm_c) __attribute__((always_inline)) {
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4"
                     : "+v"(dst) : "v"(voff), "s"(rsrc), "s"(soff), "n"(decltype(imm_c)::value) : "memory");
    };
    // A request = the L loads of one slab (LA fragment loads of A, LB direct-to-LDS loads of B),
    // issued piece by piece so that they can be dealt out between the MFMAs of a slab.
    uint32_t kb_req = 0;
    __amdgpu_buffer_rsrc_t ra_req = rsrcNone, rb_req = rsrcNone;
    auto request_begin = [&]() __attribute__((always_inline)) {
        const bool live = issued < KT;
        kb_req = (uint32_t)(split * KTB + gs) * 128u;
        gs = gs + 1 == KT ? 0 : gs + 1;
        ++issued;
        ra_req = live ? rsrcA : rsrcNone;
        rb_req = live ? rsrcB : rsrcNone;
    };
    auto request_piece = [&](auto stage_c, auto piece_c) __attribute__((always_inline)) {
        constexpr int s = decltype(stage_c)::value;
        constexpr int pc = decltype(piece_c)::value;
        if constexpr (pc < LA) {
            load_a(areg[s][pc], ra_req, voffA[pc / 2], kb_req, std::integral_constant<int, (pc & 1) * 64>{});
        } else {
            constexpr int i = pc - LA;
            dma(rb_req, voffB[i], kb_req, lds_base + (uint32_t)(s * STAGE + (wave + i * 4) * 1024));
        }
    };
    auto request = [&](auto stage_c) __attribute__((always_inline)) {
        request_begin();
        static_for<L>([&](auto pc) __attribute__((always_inline)) { request_piece(stage_c, pc); });
    };
    // all but the loads of the `Y` youngest slabs have landed for this wave; then the barrier
    auto wait_slab = [](u32x4_t (&a)[LA], auto young_c) __attribute__((always_inline)) {
        constexpr int Y = decltype(young_c)::value;
        static_assert(LA == 2 || LA == 4, "A register set of one or two 16-row groups");
        if constexpr (LA == 2)
            asm volatile("s_waitcnt vmcnt(%2) lgkmcnt(0)\n\ts_barrier"
                         : "+v"(a[0]), "+v"(a[1]) : "n"(Y * L) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(%4) lgkmcnt(0)\n\ts_barrier"
                         : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]) : "n"(Y * L) : "memory");
    };

    // B fragment reads: lane holds row (lane & 15) of a 16-row group, k chunk 4*ks + (lane >> 4)
    int rd_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) rd_off[ks] = l16 * 128 + ((((ks << 2) | q4) ^ swz(l16)) << 4);

    f32x4_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.0f;

    // One slab: its loads (and all older ones) have landed for this wave; after the barrier
    // they have for every wave, and every wave is done with the stage before it, which the
    // request for slab t + NS - 1 then refills.  TAIL >= 0 marks the last slabs of the walk,
    // TAIL-th after the requests have stopped: nothing is requested any more (it would lie
    // past the split's last slab) and the wait counts down.
    auto slab = [&](auto stage_c, auto tail_c) __attribute__((always_inline)) {
        constexpr int s = decltype(stage_c)::value;
        constexpr int TAIL = decltype(tail_c)::value;
        constexpr int sf = s == 0 ? NS - 1 : s - 1;
        tr.wait_begin();
        if constexpr (TAIL < 0) {
            wait_slab(areg[s], std::integral_constant<int, NS - 2>{});
            tr.wait_end();
            request_begin();
        } else {
            wait_slab(areg[s], std::integral_constant<int, NS - 2 - TAIL>{});
            tr.wait_end();
        }
        const unsigned char* st = lds + s * STAGE;
        // Slice 0's B fragments, then slice 1's dealt out under the MFMAs of slice 0, and the
        // loads of the request one per SPACING MFMAs (a steady trickle of requests instead of
        // a burst per slab).  The order is pinned: left alone, the scheduler interleaves the
        // two slices and the accumulators stop being updated in place (dozens of register
        // copies per slab).
        constexpr int NM = MI * NI * 2, SPACING = NM / L;
        static_assert(SPACING >= 1, "a load per MFMA slot at most");
        u32x4_t fb[2][NI];
#pragma unroll
        for (int j = 0; j < NI; ++j) fb[0][j] = *(const u32x4_t*)(st + j * 2048 + rd_off[0]);
        static_for<NM>([&](auto idx_c) __attribute__((always_inline)) {
            constexpr int idx = decltype(idx_c)::value;
            constexpr int ks = idx / (MI * NI), i = (idx / NI) % MI, j = idx % NI;
            acc[i][j] = mfma_16x16x32<DT>(fb[ks][j], areg[s][i * 2 + ks], acc[i][j]);
            if constexpr (ks == 0 && i == 0) fb[1][j] = *(const u32x4_t*)(st + j * 2048 + rd_off[1]);
            if constexpr (TAIL < 0 && idx % SPACING == 0 && idx / SPACING < L)
                request_piece(std::integral_constant<int, sf>{}, std::integral_constant<int, idx / SPACING>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // ---- prologue: slabs 0 .. NS-2 requested ----
    static_for<NS - 1>([&](auto s_c) __attribute__((always_inline)) { request(s_c); });

    // ---- main loop: NS slabs per trip, the stage (and A register set) a compile-time index ----
    int t = 0;
    for (; t + NS <= KT; t += NS)
        static_for<NS>([&](auto s_c) __attribute__((always_inline)) { slab(s_c, std::integral_constant<int, -1>{}); });
    // the remaining KT - t < NS slabs: all requested already
    static_for<NS - 1>([&](auto s_c) __attribute__((always_inline)) {
        if (t + decltype(s_c)::value < KT) slab(s_c, s_c);
    });
    // Requests past this split's last slab (empty descriptor: they fetch nothing, but zeros
    // still arrive in their registers and LDS stages) may be outstanding.  Every A register
    // set is an operand of the statement behind this wait, whichever slabs the tail ran: the
    // end of the live range that the invariant above speaks of.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    auto keep = [](u32x4_t (&a)[LA]) __attribute__((always_inline)) {
        if constexpr (LA == 2) asm volatile("" : "+v"(a[0]), "+v"(a[1]));
        else asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));
    };
    static_for<NS>([&](auto s_c) __attribute__((always_inline)) { keep(areg[decltype(s_c)::value]); });
    tr.loop_end();

    // ---- epilogue: acc[i][j][e] of lane l is C[m][n], m = row0 + i*16 + (l & 15),
    //      n = col0 + j*16 + 4*(l >> 4) + e  (N % 4 == 0 is a launch precondition) ----
    if (S == 1) {
        const bool scaled = p.alpha != 1.0f || p.beta != 0.0f;
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int m = row0 + i * 16 + l16;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int n = col0 + j * 16 + 4 * q4;
                if (m < M && n < N) {
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[i][j][e];
                        if (scaled) v[e] = scale_acc<true>(v[e], p.alpha, p.beta);
                    }
                    u32x2_t w;
                    w[0] = cvt_store2<DT>(v[0], v[1]);
                    w[1] = cvt_store2<DT>(v[2], v[3]);
                    *(u32x2_t*)((unsigned char*)p.C + ((size_t)m * p.ldc + n) * 2) = w;
                }
            }
        }
        tr.finish(p.DB, KT);
        return;
    }
    float* P = p.ws + (size_t)split * M * N;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = row0 + i * 16 + l16;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int n = col0 + j * 16 + 4 * q4;
            if (m < M && n < N) *(f32x4_t*)(P + (size_t)m * N + n) = acc[i][j];
        }
    }
    tr.finish(p.DB, KT);
}

template <class Cfg>
hipError_t launch_decode_kernel(const DecodeArgs& a, hipStream_t stream) {
    dim3 grid((a.N + Cfg::BN - 1) / Cfg::BN, a.splits);
    hipError_t e = a.DB ? launch_kernel(gemm_decode_kernel<Cfg, true>, grid, dim3(256), stream, a)
                        : launch_kernel(gemm_decode_kernel<Cfg, false>, grid, dim3(256), stream, a);
    if (e != hipSuccess || a.splits == 1) return e;
    const size_t quads = ((size_t)a.M * a.N + 3) / 4;
    return launch_kernel(splitk_reduce_kernel<Cfg::DT>, dim3((unsigned)((quads + 255) / 256)), dim3(256), stream,
                         a.ws, a.C, a.M, a.N, a.ldc, a.splits, a.alpha, a.beta);
}

}  // namespace mi
