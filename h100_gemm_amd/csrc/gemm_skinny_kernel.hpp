// gemm_skinny_kernel.hpp -- gfx950 split-K GEMM kernel for decode-shaped problems (M <= 128):
//
//   C[M,N] = A[M,K] . B[N,K]^T     M small, B (the weights) streamed once from HBM
//
// These shapes are bound by the HBM read of B, not by MFMA, so the kernel is organised
// around keeping bytes of B in flight on every CU:
//   * a workgroup owns BN = 128 rows of B and every splits-th 64-deep K slab (split-K over
//     blockIdx.y, slabs dealt out round-robin), which gives >= 256 workgroups for N = 8192
//     while each still amortises its A reads over 128 columns;
//   * B and A slabs (128-byte rows, XOR-swizzled) go global -> LDS through direct-to-LDS
//     buffer loads into a ring of NS stages; at the top of a slab the next one has already
//     landed and NS-3 more are in flight, a further one is requested during the slab;
//   * a workgroup starts its walk over its slabs at one that depends on its position in the
//     grid and wraps around; together with the round-robin deal this spreads the requests
//     in flight over every 128-byte position of a row, instead of all workgroups asking for
//     the same k (the same low address bits, hence the same few HBM channels) at once;
//   * one s_barrier per slab; waits are `vmcnt((NS-3)*L)`, never on the youngest loads;
//   * 4 waves in a WM x WN grid, v_mfma_f32_32x32x16 with the operands swapped so that a
//     lane holds 4 consecutive n; the fragments of k slice ks+1 (or of slice 0 of the next
//     slab) are fetched while slice ks multiplies, dealt out over the MFMA slots;
//   * with split-K the fp32 partial tiles go to a workspace and splitk_reduce_kernel adds
//     them in split order -- a fixed order, so results are reproducible -- and rounds once
//     to the storage type; without split-K the tile is rounded and stored directly.  (Adding
//     the partials in the last workgroup to arrive instead was measured 3x slower: the
//     device-scope fences it needs write back and invalidate the whole L2 of the XCD once
//     per workgroup.)
// The reference has no counterpart: its kernels assert M % 128 == 0 (matmul_utils.cuh:362,
// 386-387).  Rows of A past M are never fetched (the buffer descriptor ends at row M-1 and
// out-of-range loads return zero).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_kernel.hpp"

namespace mi {

struct SkinnyArgs {
    const void* A;
    const void* B;
    void* C;              // storage-type output
    float* ws;            // [splits][M][N] fp32 partials (used when splits > 1)
    int M, N, K;
    int lda, ldb, ldc;
    int k_per_split;      // unused by the kernels (host bookkeeping)
    int splits;           // <= K / 64
    float alpha = 1.0f;   // C = (CType)(acc * alpha + beta), applied where the sum over K is
    float beta = 0.0f;    // complete
};

template <int BM_, int BN_, int NS_, int DT_>
struct SkinnyConfig {
    static constexpr int BM = BM_, BN = BN_, NS = NS_, DT = DT_;
    static constexpr int NT = 256, NW = 4;
    static constexpr int WM = BM >= 64 ? 2 : 1, WN = NW / WM;   // wave grid
    static constexpr int TM = BM / WM, TN = BN / WN;         // wave tile
    static constexpr int MI = TM / 32, NI = TN / 32;
    static constexpr int NMMA = MI * NI, NFR = MI + NI;
    static constexpr int ROWS = BM + BN;                     // rows of one stage: A then B
    static constexpr int STAGE = ROWS * 128;
    static constexpr int L = ROWS / 8 / NW;                  // load instructions per wave per slab
    static constexpr int LDS_BYTES = NS * STAGE;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "MFMA blocks are 32x32");
    static_assert((ROWS / 8) % NW == 0, "load instructions divide over the waves");
    static_assert(NS >= 3 && (NS - 1) * L <= 63, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

template <class Cfg>
__global__ void __launch_bounds__(256) gemm_skinny_kernel(const SkinnyArgs p) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, DT = Cfg::DT;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, TM = Cfg::TM, TN = Cfg::TN, L = Cfg::L, STAGE = Cfg::STAGE;
    constexpr int NMMA = Cfg::NMMA, NFR = Cfg::NFR;

    __shared__ __attribute__((aligned(128))) unsigned char lds[Cfg::LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    const int col0 = blockIdx.x * BN;
    const int split = blockIdx.y;
    const int M = p.M, N = p.N, K = p.K;
    const int S = p.splits;
    const int KT = (K / 64 - split + S - 1) / S;             // slabs of this split: split, split+S, .. (>= 1)

    const int rowsA = M < BM ? M : BM;
    const int rowsB = (N - col0) < BN ? (N - col0) : BN;
    const unsigned char* Ab = (const unsigned char*)p.A;
    const unsigned char* Bb = (const unsigned char*)p.B + (size_t)col0 * p.ldb * 2;
    // descriptors end at the last element of the last valid row
    const uint32_t bytesA = (uint32_t)((rowsA - 1) * p.lda + K) * 2u;
    const uint32_t bytesB = (uint32_t)((rowsB - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcNone = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, 0, 0x00020000);

    // One load instruction fills 8 consecutive 128-byte rows of a stage: lane l lands on
    // chunk position l & 7 of row l >> 3 and therefore fetches logical chunk
    // (l & 7) ^ swz(row), swz(row) = (row >> 1) & 7.  Instruction q (0 .. ROWS/8-1) of a slab
    // covers stage rows 8q .. 8q+7; rows below BM belong to A, the rest to B; wave w issues
    // q = w, w + 4, ...
    const int lr = lane >> 3, lc = lane & 7;
    auto swz = [](int row) __attribute__((always_inline)) { return (row >> 1) & 7; };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    auto dma = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
    };
    uint32_t voff[L];
#pragma unroll
    for (int i = 0; i < L; ++i) {
        const int q = wave + i * 4;                          // wave-uniform
        const int row = q * 8 + lr;                          // stage row of this lane
        const int chunk = lc ^ swz(row);
        voff[i] = q * 8 < BM ? (uint32_t)(row * p.lda + chunk * 8) * 2u
                             : (uint32_t)((row - BM) * p.ldb + chunk * 8) * 2u;
    }
    // Slab t of the loop is this split's slab (t + rot) mod KT, i.e. slab split + S * that of
    // the matrix.  `gs` follows the slab being requested, `issued` counts requested slabs.
    int gs = (int)((blockIdx.x * 5u) % (unsigned)KT);
    int issued = 0;
    uint32_t kb_cur = 0;
    bool live_cur = false;
    auto begin_slab = [&]() __attribute__((always_inline)) {
        live_cur = issued < KT;
        kb_cur = (uint32_t)(split + S * gs) * 128u;
        gs = gs + 1 == KT ? 0 : gs + 1;
        ++issued;
    };
    auto dma_one = [&](int s, int i) __attribute__((always_inline)) {
        const int q = wave + i * 4;
        const uint32_t dst = lds_base + (uint32_t)(s * STAGE + q * 1024);
        if (q * 8 < BM) {
            dma(live_cur ? rsrcA : rsrcNone, voff[i] + kb_cur, dst);
        } else {
            dma(live_cur ? rsrcB : rsrcNone, voff[i] + kb_cur, dst);
        }
    };

    // fragment reads: lane holds row (lane & 31), k chunk 2*ks + (lane >> 5)
    const int l32 = lane & 31, hi = lane >> 5;
    int rd_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) rd_off[ks] = l32 * 128 + ((((ks << 1) | hi) ^ swz(l32)) << 4);
    const int a_wave = wm * TM * 128;
    const int b_wave = (BM + wn * TN) * 128;

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
    auto read_one = [&](const unsigned char* st, int ks, int buf, int r) __attribute__((always_inline)) {
        if (r == 0 || r > NI) {
            const int i = r == 0 ? 0 : r - NI;
            fa[buf][i] = *(const u32x4_t*)(st + a_wave + i * 4096 + rd_off[ks]);
        } else {
            const int j = r - 1;
            fb[buf][j] = *(const u32x4_t*)(st + b_wave + j * 4096 + rd_off[ks]);
        }
    };
    constexpr int RPS = (NFR + NMMA - 1) / NMMA;             // LDS reads per MFMA slot
    constexpr int DPS = (L + 4 * NMMA - 1) / (4 * NMMA);     // load instructions per MFMA slot

    // ---- prologue: slabs 0 .. NS-2 requested, slab 0 landed, its first fragments fetched ----
#pragma unroll
    for (int t = 0; t < NS - 1; ++t) {
        begin_slab();
#pragma unroll
        for (int i = 0; i < L; ++i) dma_one(t, i);
    }
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"((NS - 2) * L) : "memory");
#pragma unroll
    for (int r = 0; r < NFR; ++r) read_one(lds, 0, 0, r);

    int s = 0;
    for (int t = 0; t < KT; ++t) {
        const int sn = s + 1 == NS ? 0 : s + 1;              // stage of slab t+1
        const int sf = s == 0 ? NS - 1 : s - 1;              // stage of slab t-1: refilled now
        // slab t+1 has landed for every wave, every wave is done with slab t-1
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"((NS - 3) * L) : "memory");
        begin_slab();
        const unsigned char* st = lds + s * STAGE;
        const unsigned char* stn = lds + sn * STAGE;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int idx = 0; idx < NMMA; ++idx) {
                mma_one(ks & 1, idx);
#pragma unroll
                for (int r = idx * RPS; r < (idx + 1) * RPS && r < NFR; ++r) {
                    if (ks < 3) read_one(st, ks + 1, (ks + 1) & 1, r);
                    else read_one(stn, 0, 0, r);             // after the last slab: stale bytes, never used
                }
#pragma unroll
                for (int d = (ks * NMMA + idx) * DPS; d < (ks * NMMA + idx + 1) * DPS && d < L; ++d)
                    dma_one(sf, d);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        s = sn;
    }
    // loads requested past this split's last slab are still heading for the ring
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

    // ---- epilogue: lane holds C[m][n..n+3], m = i*32 + (lane & 31), n = 8g + 4*(lane>>5) ----
    if (S == 1) {
        const bool scaled = p.alpha != 1.0f || p.beta != 0.0f;
        unsigned char* Cb = (unsigned char*)p.C;
        const __amdgpu_buffer_rsrc_t rsrcC =
            __builtin_amdgcn_make_buffer_rsrc((void*)Cb, 0, (int)((uint32_t)(M * p.ldc) * 2u), 0x00020000);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int m = wm * TM + i * 32 + l32;
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = col0 + wn * TN + j * 32 + g * 8 + hi * 4;
                    if (m < M && n < N) {           // N % 4 == 0 is a launch precondition
                        u32x2_t w;
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            v[e] = acc[i][j][g * 4 + e];
                            if (scaled) v[e] = scale_acc<true>(v[e], p.alpha, p.beta);
                        }
                        w[0] = cvt_store2<DT>(v[0], v[1]);
                        w[1] = cvt_store2<DT>(v[2], v[3]);
                        __builtin_amdgcn_raw_buffer_store_b64(w, rsrcC, (uint32_t)(m * p.ldc + n) * 2u, 0, 0);
                    }
                }
        }
        return;
    }
    float* P = p.ws + (size_t)split * M * N;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = wm * TM + i * 32 + l32;
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = col0 + wn * TN + j * 32 + g * 8 + hi * 4;
                if (m < M && n < N) {
                    float4 v = {acc[i][j][g * 4 + 0], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2],
                                acc[i][j][g * 4 + 3]};
                    *(float4*)(P + (size_t)m * N + n) = v;
                }
            }
    }
}

// C[m][n] = round(alpha * (sum over splits, in split order, of ws[s][m][n]) + beta); 4 elements per thread.
template <int DT>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ ws, void* C, int M,
                                                            int N, int ldc, int splits, float alpha,
                                                            float beta) {
    const size_t idx = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const size_t total = (size_t)M * N;
    if (idx >= total) return;
    float4 a = *(const float4*)(ws + idx);
    for (int s = 1; s < splits; ++s) {
        const float4 b = *(const float4*)(ws + (size_t)s * total + idx);
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    if (alpha != 1.0f || beta != 0.0f) {
        a.x = mul_add_unfused(a.x, alpha, beta);
        a.y = mul_add_unfused(a.y, alpha, beta);
        a.z = mul_add_unfused(a.z, alpha, beta);
        a.w = mul_add_unfused(a.w, alpha, beta);
    }
    const size_t m = idx / N, n = idx % N;
    u32x2_t w;
    w[0] = cvt_store2<DT>(a.x, a.y);
    w[1] = cvt_store2<DT>(a.z, a.w);
    *(u32x2_t*)((unsigned char*)C + (m * ldc + n) * 2) = w;
}

template <class Cfg>
hipError_t launch_skinny_kernel(const SkinnyArgs& a, hipStream_t stream) {
    dim3 grid((a.N + Cfg::BN - 1) / Cfg::BN, a.splits);
    hipLaunchKernelGGL((gemm_skinny_kernel<Cfg>), grid, dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || a.splits == 1) return e;
    const size_t quads = ((size_t)a.M * a.N + 3) / 4;
    hipLaunchKernelGGL((splitk_reduce_kernel<Cfg::DT>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0,
                       stream, a.ws, a.C, a.M, a.N, a.ldc, a.splits, a.alpha, a.beta);
    return hipGetLastError();
}

}  // namespace mi
