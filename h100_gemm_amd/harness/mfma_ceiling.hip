// mfma_ceiling.hip -- what the MFMA pipes alone sustain on this chip, for reading the GEMM's
// roofline fraction: a loop of nothing but v_mfma_f32_16x16x32_bf16 (64 accumulator tiles in
// AGPRs per wave, one wave per SIMD, one workgroup per CU, 8 + 8 operand fragments visited in
// the order the GEMM kernel uses), timed long enough for the clock to settle.  The chip is
// power limited: the issue rate is the same for every data set (~16.3 cycles per MFMA), the
// clock is not -- zeros run near the peak clock, random bf16 operands far below it.
//
//     ./mfma_ceiling [milliseconds per data set] [zeros|uniform|normal]     default 300, all three
//
// One line per data set: cycles per MFMA (the shader-cycle counter of one wave), shader clock
// (cycles / wall time), and the rate of the whole chip in TFLOP/s.  No memory traffic, no
// LDS; not part of the library.
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s:%d %s\n", __FILE__, __LINE__, hipGetErrorString(e_));          \
            exit(1);                                                                          \
        }                                                                                     \
    } while (0)

constexpr int NACC = 64;   // 16x16 accumulator tiles per wave: the 128x128 wave tile of the GEMM kernel

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
mfma_only(float* out, long long* cycles, int iters, const uint4* operands) {
    f32x4 acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = f32x4{0, 0, 0, 0};
    bf16x8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = __builtin_bit_cast(bf16x8, operands[(threadIdx.x + 256 * i) & 4095]);
        b[i] = __builtin_bit_cast(bf16x8, operands[(threadIdx.x + 256 * i + 2048) & 4095]);
    }
#pragma unroll
    for (int i = 0; i < NACC; ++i) asm volatile("" : "+a"(acc[i]));
    const long long t0 = (long long)__builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < NACC; ++k) {
            const int i = k / 8, j = (i & 1) ? 7 - k % 8 : k % 8;   // rows in turn, columns back and forth
            acc[k] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j], a[i], acc[k], 0, 0, 0);
        }
    }
    const long long t1 = (long long)__builtin_readcyclecounter();
    float s = 0;
#pragma unroll
    for (int i = 0; i < NACC; ++i) s += acc[i][0] + acc[i][3];
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (threadIdx.x == 0) cycles[blockIdx.x] = t1 - t0;
}

static uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

int main(int argc, char** argv) {
    const double ms_per_set = argc > 1 ? atof(argv[1]) : 300.0;
    const char* only = argc > 2 ? argv[2] : nullptr;       // one data set: "zeros", "uniform" or "normal"
    int dev = 0, cus = 0;
    HIP_OK(hipGetDevice(&dev));
    HIP_OK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    float* out;
    long long* cycles;
    uint4* operands;
    HIP_OK(hipMalloc(&out, (size_t)cus * 256 * sizeof(float)));
    HIP_OK(hipMalloc(&cycles, (size_t)cus * sizeof(long long)));
    HIP_OK(hipMalloc(&operands, 4096 * sizeof(uint4)));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    printf("%d CUs, one workgroup of 4 waves each, %d MFMA 16x16x32 bf16 per loop iteration\n", cus, NACC);

    struct Set { const char* name; int kind; };
    const Set sets[] = {{"zeros", 0}, {"uniform [-1,1) bf16", 1}, {"normal(0,1) bf16", 2}};
    for (const Set& set : sets) {
        if (only && strncmp(set.name, only, strlen(only)) != 0) continue;
        std::vector<uint16_t> h(4096 * 8);
        uint64_t x = 0x9E3779B97F4A7C15ull;
        auto next = [&]() {
            x ^= x << 13; x ^= x >> 7; x ^= x << 17;
            return (double)(x >> 11) * (1.0 / 9007199254740992.0);
        };
        for (size_t i = 0; i < h.size(); ++i) {
            float v = 0.0f;
            if (set.kind == 1) v = (float)(2.0 * next() - 1.0);
            if (set.kind == 2) v = (float)(std::sqrt(-2.0 * std::log(1.0 - next())) * std::cos(6.283185307179586 * next()));
            h[i] = to_bf16(v);
        }
        HIP_OK(hipMemcpy(operands, h.data(), h.size() * 2, hipMemcpyHostToDevice));
        // one launch of ~20 ms at a time until ms_per_set has passed (the clock settles within
        // ~100 ms under load); the last launch is the one reported
        const int iters = 40000;
        double total_ms = 0;
        float ms = 0;
        do {
            HIP_OK(hipEventRecord(e0));
            hipLaunchKernelGGL(mfma_only, dim3(cus), dim3(256), 0, 0, out, cycles, iters, operands);
            HIP_OK(hipGetLastError());
            HIP_OK(hipEventRecord(e1));
            HIP_OK(hipEventSynchronize(e1));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            total_ms += ms;
        } while (total_ms < ms_per_set);
        long long c0 = 0;
        HIP_OK(hipMemcpy(&c0, cycles, sizeof(c0), hipMemcpyDeviceToHost));
        const double n = (double)iters * NACC;
        const double tflops = (double)cus * 4.0 * n * (16.0 * 16 * 32 * 2) / (ms * 1e-3) / 1e12;
        printf("%-22s %.2f cycles per MFMA, clock %.2f GHz, %.0f TFLOP/s\n", set.name, (double)c0 / n,
               (double)c0 / (ms * 1e-3) / 1e9, tflops);
    }
    HIP_OK(hipFree(out));
    HIP_OK(hipFree(cycles));
    HIP_OK(hipFree(operands));
    return 0;
}
