// splitk_common.hpp -- what the split-K launches share: the argument block of the decode
// kernels and the kernel that adds the fp32 partial tiles.
//
// A split-K launch leaves `splits` partial results [split][M][N] in an fp32 workspace;
// splitk_reduce_kernel adds them in split order -- a fixed order, so results are reproducible
// run to run -- applies the golden's epilogue C = (CType)(acc * alpha + beta) (reference.h:40)
// and rounds once to the storage type.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_kernel.hpp"

namespace mi {

struct DecodeArgs {
    const void* A;
    const void* B;
    void* C;              // storage-type output
    float* ws;            // [splits][M][N] fp32 partials (used when splits > 1)
    int M, N, K;
    int lda, ldb, ldc;
    int k_per_split;      // K range of one split (a contiguous piece), a multiple of 64
    int splits;           // <= K / 64
    float alpha = 1.0f;   // C = (CType)(acc * alpha + beta), applied where the sum over K is
    float beta = 0.0f;    // complete
    int* DB = nullptr;    // optional trace buffer: one record of six ints per workgroup
};

// The per-workgroup timing record of the trace buffer `DB` of runKernel's signature, in the
// format its harness parses (matmul_h100_optimal.cu:182-198): {sumLoad, cntLoad, sumCompute,
// cntCompute, sumStore, cntStore} = {cycles thread 0 spent waiting for loads (and at the
// barriers behind those waits), number of such waits, cycles from the kernel's start to the end
// of its K loop, K units it multiplied, cycles from there to its last store, 1}.  Workgroup
// (x, y) of a grid writes record y * gridDim.x + x.  With ON = false every member is empty.
template <bool ON>
struct TraceRec {
    long long wait = 0, t0 = 0, loop = 0, store = 0;
    int cnt = 0;
    static __device__ __forceinline__ long long now() { return (long long)__builtin_readcyclecounter(); }
    __device__ __forceinline__ void begin() { if constexpr (ON) loop = now(); }
    __device__ __forceinline__ void wait_begin() { if constexpr (ON) t0 = now(); }
    __device__ __forceinline__ void wait_end() { if constexpr (ON) { wait += now() - t0; ++cnt; } }
    __device__ __forceinline__ void loop_end() { if constexpr (ON) { store = now(); loop = store - loop; } }
    __device__ __forceinline__ void finish(int* DB, int units) {
        if constexpr (ON) {
            if (DB != nullptr && threadIdx.x == 0) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                store = now() - store;
                int* rec = DB + 6 * ((size_t)blockIdx.y * gridDim.x + blockIdx.x);
                rec[0] = (int)wait;
                rec[1] = cnt;
                rec[2] = (int)loop;
                rec[3] = units;
                rec[4] = (int)store;
                rec[5] = 1;
            }
        }
    }
};

// C[m][n] = round(alpha * (sum over splits, in split order, of ws[s][m][n]) + beta); 4 elements per thread.
template <int DT>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ ws, void* C, int M,
                                                            int N, int ldc, int splits, float alpha,
                                                            float beta) {
    const size_t idx = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const size_t total = (size_t)M * N;
    if (idx >= total) return;
    // four pieces' loads in flight at a time, added in piece order (one load per trip made a
    // reduction over 16 pieces a chain of 16 memory latencies); the sum starts from +0, which
    // changes no bit of it (a piece's sums come out of accumulators that started from +0 and
    // are never -0)
    float4 a = {0.0f, 0.0f, 0.0f, 0.0f};
    int s = 0;
    for (; s + 4 <= splits; s += 4) {
        const float4 b0 = *(const float4*)(ws + (size_t)s * total + idx);
        const float4 b1 = *(const float4*)(ws + (size_t)(s + 1) * total + idx);
        const float4 b2 = *(const float4*)(ws + (size_t)(s + 2) * total + idx);
        const float4 b3 = *(const float4*)(ws + (size_t)(s + 3) * total + idx);
        a.x += b0.x; a.y += b0.y; a.z += b0.z; a.w += b0.w;
        a.x += b1.x; a.y += b1.y; a.z += b1.z; a.w += b1.w;
        a.x += b2.x; a.y += b2.y; a.z += b2.z; a.w += b2.w;
        a.x += b3.x; a.y += b3.y; a.z += b3.z; a.w += b3.w;
    }
    if (s + 2 <= splits) {
        const float4 b0 = *(const float4*)(ws + (size_t)s * total + idx);
        const float4 b1 = *(const float4*)(ws + (size_t)(s + 1) * total + idx);
        a.x += b0.x; a.y += b0.y; a.z += b0.z; a.w += b0.w;
        a.x += b1.x; a.y += b1.y; a.z += b1.z; a.w += b1.w;
        s += 2;
    }
    if (s < splits) {
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

}  // namespace mi
