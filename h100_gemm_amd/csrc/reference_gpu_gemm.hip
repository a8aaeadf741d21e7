// reference_gpu_gemm.hip -- the plain, order-preserving GPU GEMM the harness checks the
// MFMA kernels against.  It takes the place of reference_gpu_gemm / reference_gpu_gemm_kernel
// (reference.h:49-90), which the reference's own harness uses as golden
// (matmul_h100.cu.jinja:1043-1047), and keeps that kernel's contract: one fp32
// accumulator per C element fed in ascending k, terms with k >= K are zero, stores are
// predicated on m < M and n < N, and C = (CType)(acc * alpha + beta) with beta a plain
// scalar.  acc * alpha and + beta are two separately rounded operations, as in the host
// version of the same formula (reference.h:40).
//
// 64x64 output tile per workgroup, 16x16 threads, 4x4 outputs per thread, K walked in
// chunks of 16 through LDS.  Not a fast kernel and not meant to be one.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mi_gemm.h"

namespace {

template <int DT>
__device__ __forceinline__ float load_f32(const uint16_t* p) {
    if constexpr (DT == MI_DTYPE_BF16) {
        return __builtin_bit_cast(float, (uint32_t)(*p) << 16);
    } else {
        return (float)__builtin_bit_cast(_Float16, *p);
    }
}
// x * a + b as two separately rounded fp32 operations (HIP's __fmul_rn / __fadd_rn are the
// plain operators and would be contracted into one fma under the default -ffp-contract=fast)
__device__ __forceinline__ float mul_add_unfused(float x, float a, float b) {
#pragma clang fp contract(off)
    const float t = x * a;
    return t + b;
}
template <int DT>
__device__ __forceinline__ uint16_t store_f32(float f) {
    if constexpr (DT == MI_DTYPE_BF16) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    } else {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
}

template <int DT>
__global__ void __launch_bounds__(256)
naive_gemm_kernel(int M, int N, int K, const uint16_t* __restrict__ A,
                  const uint16_t* __restrict__ B, uint16_t* __restrict__ C, float alpha,
                  float beta) {
    __shared__ float sa[16][64 + 1];
    __shared__ float sb[16][64 + 1];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += 16) {
        // 64 rows x 16 k per operand = 1024 values, 4 per thread
        for (int i = threadIdx.x; i < 1024; i += 256) {
            const int r = i >> 4, kk = i & 15;
            const int k = k0 + kk;
            float a = 0.0f, b = 0.0f;
            if (k < K) {
                if (m0 + r < M) a = load_f32<DT>(A + (size_t)(m0 + r) * K + k);
                if (n0 + r < N) b = load_f32<DT>(B + (size_t)(n0 + r) * K + k);
            }
            sa[kk][r] = a;
            sb[kk][r] = b;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __fadd_rn(acc[i][j], __fmul_rn(sa[kk][ty * 4 + i], sb[kk][tx * 4 + j]));
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < M && n < N)
                C[(size_t)m * N + n] = store_f32<DT>(mul_add_unfused(acc[i][j], alpha, beta));
        }
}

}  // namespace

namespace mi {
hipError_t launch_reference_gpu_gemm(int dtype, int M, int N, int K, const void* A, const void* B,
                                     void* C, float alpha, float beta, hipStream_t stream) {
    dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
    // the status of this launch (not an error some earlier call of the process left behind)
    const uint16_t* a = (const uint16_t*)A;
    const uint16_t* b = (const uint16_t*)B;
    uint16_t* c = (uint16_t*)C;
    void* args[] = {&M, &N, &K, &a, &b, &c, &alpha, &beta};
    const void* kernel = dtype == MI_DTYPE_BF16 ? (const void*)naive_gemm_kernel<MI_DTYPE_BF16>
                                                : (const void*)naive_gemm_kernel<MI_DTYPE_FP16>;
    return hipLaunchKernel(kernel, grid, block, args, 0, stream);
}
}  // namespace mi
