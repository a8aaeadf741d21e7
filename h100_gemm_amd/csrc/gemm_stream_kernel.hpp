// gemm_stream_kernel.hpp -- gfx950 GEMM kernel for the thinnest decode shapes (M <= 64):
//
//   C[M,N] = A[M,K] . B[N,K]^T     one pass over B, one kernel, no workspace
//
// B (the weights) is read exactly once from HBM and that read is the whole cost, so the
// kernel is a set of independent streams, one per wave:
//   * a workgroup owns 32 rows of B (32 columns of C) over all of K; N = 8192 gives one
//     workgroup per CU;
//   * its four waves split K between them, 64-deep slab by slab (wave w takes slabs
//     w, w+4, ...), so the workgroup as a whole walks 512 contiguous bytes of every row;
//   * each wave has a private ring of NS stages in LDS, filled by direct-to-LDS buffer
//     loads (B rows and the matching k range of A, 128-byte rows, XOR-swizzled) and
//     drained by its own MFMAs; a wave waits only on its own `vmcnt`, there is no barrier
//     in the loop, and NS-1 slabs per wave are always in flight;
//   * workgroup b starts its walk over K at slab 37*b mod K/64 and wraps around: with every
//     workgroup at the same k at the same time, all requests in flight would share their
//     low address bits (rows are K*2 bytes apart) and crowd a few HBM channels; staggered
//     starts measured 6.7 TB/s against 4.7 TB/s for the same bytes;
//   * the four partial 32x32 fp32 tiles are added in wave order through LDS (a fixed order:
//     results are reproducible), rounded once and stored.
// A is re-read by every workgroup; it is at most 64 x K and stays in L2.
// Rows of A past M and rows of B past N are never fetched (the buffer descriptors end at
// the last valid row; out-of-range lanes load nothing that reaches a stored element).
// The reference has no counterpart: its kernels assert M % 128 == 0 (matmul_utils.cuh:362).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_kernel.hpp"
#include "splitk_common.hpp"

namespace mi {

template <int BM_, int NS_, int DT_>
struct StreamConfig {
    static constexpr int BM = BM_, BN = 32, NS = NS_, DT = DT_;
    static constexpr int NT = 256, NW = 4;
    static constexpr int ROWS = BM + BN;                     // rows of one stage: A then B
    static constexpr int STAGE = ROWS * 128;
    static constexpr int L = ROWS / 8;                       // load instructions per slab
    static constexpr int RING = NS * STAGE;                  // one wave's ring
    static constexpr int LDS_BYTES = NW * RING;
    static constexpr int MI = (BM + 31) / 32;                // 32-row MFMA blocks of A
    static_assert(BM == 16 || BM % 32 == 0, "A block is half of or whole 32-row MFMA operands");
    static_assert(NS >= 2 && (NS - 1) * L <= 63, "vmcnt is a 6-bit counter");
    static_assert(RING >= MI * 32 * 32 * 4, "a ring holds the wave's fp32 partial tile");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

// TRACE: the per-workgroup timing record (TraceRec; thread 0 is in wave 0, so the waits and the
// K units are that wave's) for launches that pass a trace buffer.
template <class Cfg, bool TRACE = false>
__global__ void __launch_bounds__(256) gemm_stream_kernel(const DecodeArgs p) {
    constexpr int BM = Cfg::BM, NS = Cfg::NS, DT = Cfg::DT;
    constexpr int L = Cfg::L, STAGE = Cfg::STAGE, RING = Cfg::RING, MI = Cfg::MI;

    __shared__ __attribute__((aligned(128))) unsigned char lds[Cfg::LDS_BYTES];
    TraceRec<TRACE> tr;
    tr.begin();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col0 = blockIdx.x * 32;
    const int M = p.M, N = p.N, K = p.K;
    const int KT = K / 64;                                   // slabs (K % 64 == 0 is a launch precondition)
    const int cnt = (KT - wave + 3) / 4;                     // slabs of this wave: wave, wave+4, ...

    const int rowsA = M < BM ? M : BM;
    const int rowsB = (N - col0) < 32 ? (N - col0) : 32;
    const unsigned char* Ab = (const unsigned char*)p.A;
    const unsigned char* Bb = (const unsigned char*)p.B + (size_t)col0 * p.ldb * 2;
    const uint32_t bytesA = (uint32_t)((rowsA - 1) * p.lda + K) * 2u;
    const uint32_t bytesB = (uint32_t)((rowsB - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcNone = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, 0, 0x00020000);

    // One load instruction fills 8 consecutive 128-byte rows of a stage: lane l lands on
    // chunk position l & 7 of row l >> 3 and fetches logical chunk (l & 7) ^ swz(row).
    const int lr = lane >> 3, lc = lane & 7;
    auto swz = [](int row) __attribute__((always_inline)) { return (row >> 1) & 7; };
    const uint32_t ring_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds + (uint32_t)wave * RING;
    auto dma = [&](const __amdgpu_buffer_rsrc_t& rsrc, uint32_t voff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
    };
    // B is read once: non-temporal, so that it does not push A (re-read by every workgroup) out of the L2s
    auto dma_nt = [&](const __amdgpu_buffer_rsrc_t& rsrc, uint32_t voff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
    };
    // this lane's byte offsets inside A and B for instruction q of a slab (k offset added later)
    uint32_t voff[L];
#pragma unroll
    for (int q = 0; q < L; ++q) {
        const int row = q * 8 + lr;                          // stage row: A rows first, then B rows
        const int chunk = lc ^ swz(row);
        voff[q] = q * 8 < BM ? (uint32_t)(row * p.lda + chunk * 8) * 2u
                             : (uint32_t)((row - BM) * p.ldb + chunk * 8) * 2u;
    }
    // slab i of this wave is slab (wave + 4*i + rot) mod KT of the matrix; `gs` follows the
    // slab about to be requested
    int gs = (int)(((unsigned)wave + blockIdx.x * 37u) % (unsigned)KT);
    auto dma_slab = [&](int i, int s) __attribute__((always_inline)) {
        const bool live = i < cnt;
        const uint32_t kb = (uint32_t)gs * 128u;
        gs += 4;
        while (gs >= KT) gs -= KT;
#pragma unroll
        for (int q = 0; q < L; ++q) {
            if (q * 8 < BM) dma(live ? rsrcA : rsrcNone, voff[q] + kb, ring_base + (uint32_t)(s * STAGE + q * 1024));
            else dma_nt(live ? rsrcB : rsrcNone, voff[q] + kb, ring_base + (uint32_t)(s * STAGE + q * 1024));
        }
    };

    // fragment reads: lane holds row (lane & 31), k chunk 2*ks + (lane >> 5).  With BM = 16
    // the upper half of the A operand reads B rows: finite values that only reach rows of
    // the accumulator that are never stored.
    const int l32 = lane & 31, hi = lane >> 5;
    int rd_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) rd_off[ks] = l32 * 128 + ((((ks << 1) | hi) ^ swz(l32)) << 4);

    f32x16_t acc[MI];
#pragma unroll
    for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[a][e] = 0.0f;

#pragma unroll
    for (int i = 0; i < NS - 1; ++i) dma_slab(i, i);

    const unsigned char* ring = lds + wave * RING;
    int s = 0;
    for (int i = 0; i < cnt; ++i) {
        // slab i of this wave has landed; its predecessor's fragments are in registers
        tr.wait_begin();
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" :: "n"((NS - 2) * L) : "memory");
        tr.wait_end();
        dma_slab(i + NS - 1, s == 0 ? NS - 1 : s - 1);
        const unsigned char* st = ring + s * STAGE;
        u32x4_t fa[MI][4], fb[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int a = 0; a < MI; ++a) fa[a][ks] = *(const u32x4_t*)(st + a * 4096 + rd_off[ks]);
            fb[ks] = *(const u32x4_t*)(st + BM * 128 + rd_off[ks]);
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int a = 0; a < MI; ++a) acc[a] = mfma_32x32x16<DT>(fb[ks], fa[a][ks], acc[a]);
        s = s + 1 == NS ? 0 : s + 1;
    }
    // requests past K are still heading for the ring: drain before it is reused
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    tr.loop_end();

    // ---- add the four partial tiles in wave order, round, store ----
    // lane holds P[m][n .. n+3], m = 32a + (lane & 31), n = 8g + 4*(lane >> 5)
    float* part = (float*)(lds + wave * RING);
#pragma unroll
    for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float4 v = {acc[a][g * 4 + 0], acc[a][g * 4 + 1], acc[a][g * 4 + 2], acc[a][g * 4 + 3]};
            *(float4*)(part + (a * 32 + l32) * 32 + g * 8 + hi * 4) = v;
        }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < MI; ++a) {
        const int m = a * 32 + (tid >> 3), n = (tid & 7) * 4;
        float4 sum = *(const float4*)((const float*)lds + m * 32 + n);
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const float4 v = *(const float4*)((const float*)(lds + w * RING) + m * 32 + n);
            sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
        }
        if (p.alpha != 1.0f || p.beta != 0.0f) {
            sum.x = mul_add_unfused(sum.x, p.alpha, p.beta);
            sum.y = mul_add_unfused(sum.y, p.alpha, p.beta);
            sum.z = mul_add_unfused(sum.z, p.alpha, p.beta);
            sum.w = mul_add_unfused(sum.w, p.alpha, p.beta);
        }
        if (m < M && col0 + n < N) {                         // N % 4 == 0 is a launch precondition
            u32x2_t w2;
            w2[0] = cvt_store2<DT>(sum.x, sum.y);
            w2[1] = cvt_store2<DT>(sum.z, sum.w);
            *(u32x2_t*)((unsigned char*)p.C + ((size_t)m * p.ldc + col0 + n) * 2) = w2;
        }
    }
    tr.finish(p.DB, cnt);
}

template <class Cfg>
hipError_t launch_stream_kernel(const DecodeArgs& a, hipStream_t stream) {
    return a.DB ? launch_kernel(gemm_stream_kernel<Cfg, true>, dim3((a.N + 31) / 32), dim3(256), stream, a)
                : launch_kernel(gemm_stream_kernel<Cfg, false>, dim3((a.N + 31) / 32), dim3(256), stream, a);
}

}  // namespace mi
