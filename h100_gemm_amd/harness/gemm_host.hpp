// gemm_host.hpp -- host-side C++ surface of the GEMM library, shaped like the reference
// project's harness headers so that a program written against them keeps compiling:
//
//   GemmParams<A,B,C,Acc>                    common.h:206-221
//   CPUTimer / GPUTimer                      common.h:223-273
//   alloc_*/free_*/copy_* tensor helpers     common.h:275-365
//   random_fill / arange_fill / constant_fill   common.h:283-307
//   assert_allclose                          common.h:367-397
//   get_sm_count                             common.h:43-60
//   reference_gpu_gemm(GemmParams)           reference.h:78-90
//   gpu_gemm<..>(GemmParams)                 matmul_h100.cu.jinja:927-985
//   runKernel / run_kernel                   matmul_h100_optimal.cu:32-59, 75-84
//   randomize_matrix / verify_matrix         matmul_h100_optimal.cu:86-108
//
// Everything device-side goes through the C ABI in include/mi_gemm.h; this header is plain
// host C++17 and needs no HIP headers.  Errors keep the reference's convention: print the
// message with file:line and exit(EXIT_FAILURE) (common.h:29-37, matmul_h100_optimal.cu:21-28).
#pragma once

#include <algorithm>
#include <cassert>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <iostream>
#include <numeric>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "../../include/mi_gemm.h"

#define MI_CHECK(call)                                                                   \
    do {                                                                                 \
        int rc_ = (call);                                                                \
        if (rc_ != MI_OK) {                                                              \
            std::cerr << "Got bad status " << rc_ << ": " << mi_last_error() << " at "   \
                      << __FILE__ << ":" << __LINE__ << std::endl;                       \
            exit(EXIT_FAILURE);                                                          \
        }                                                                                \
    } while (0)

// ---- 16-bit storage types ------------------------------------------------------------
// Stand-ins for __nv_bfloat16 / half on the host: construct from float (round to nearest
// even), convert back to float.

struct bf16 {
    uint16_t bits;
    bf16() = default;
    bf16(float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) {
            bits = (uint16_t)((u >> 16) | 0x0040u);
        } else {
            u += 0x7fffu + ((u >> 16) & 1u);
            bits = (uint16_t)(u >> 16);
        }
    }
    bf16(double d) : bf16((float)d) {}
    bf16(int i) : bf16((float)i) {}
    operator float() const {
        uint32_t u = (uint32_t)bits << 16;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

struct half_t {
    uint16_t bits;
    half_t() = default;
    half_t(float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
        uint32_t a = u & 0x7fffffffu;
        if (a > 0x7f800000u) {
            bits = sign | 0x7e00u;
        } else if (a >= 0x477ff000u) {
            bits = sign | 0x7c00u;
        } else if (a < 0x38800000u) {
            if (a < 0x33000000u) {
                bits = sign;
            } else {
                float v;
                std::memcpy(&v, &a, 4);
                bits = sign | (uint16_t)std::nearbyint(v * 16777216.0f);
            }
        } else {
            a += 0xfffu + ((a >> 13) & 1u);
            bits = sign | (uint16_t)((a - 0x38000000u) >> 13);
        }
    }
    half_t(double d) : half_t((float)d) {}
    half_t(int i) : half_t((float)i) {}
    operator float() const {
        const uint32_t sign = (uint32_t)(bits & 0x8000u) << 16;
        const uint32_t exp = (bits >> 10) & 0x1fu, man = bits & 0x3ffu;
        uint32_t u;
        if (exp == 0) {
            if (man == 0) {
                u = sign;
            } else {
                float v = (float)man * 5.9604644775390625e-08f;
                std::memcpy(&u, &v, 4);
                u |= sign;
            }
        } else if (exp == 31) {
            u = sign | 0x7f800000u | (man << 13);
        } else {
            u = sign | ((exp + 112u) << 23) | (man << 13);
        }
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

template <class T> struct mi_dtype_of;
template <> struct mi_dtype_of<bf16> { static constexpr int value = MI_DTYPE_BF16; };
template <> struct mi_dtype_of<half_t> { static constexpr int value = MI_DTYPE_FP16; };

// ---- GemmParams (common.h:206-221) ----------------------------------------------------

template <class AType, class BType, class CType, class AccumType>
struct GemmParams {
    const int M;
    const int N;
    const int K;
    const AType* A;
    const BType* B;
    CType* C;
    const AccumType alpha;
    const AccumType beta;

    GemmParams(const int M, const int N, const int K, const AType* A, const BType* B, CType* C,
               const AccumType alpha, const AccumType beta)
        : M(M), N(N), K(K), A(A), B(B), C(C), alpha(alpha), beta(beta) {}
};

// ---- timers (common.h:223-273) ---------------------------------------------------------

struct Timer {
    virtual void tick() = 0;
    virtual double report_last_ms() = 0;
    virtual ~Timer() = default;
};

struct CPUTimer : public Timer {
    void tick() final {
        trace_[cur_] = std::chrono::high_resolution_clock::now();
        cur_ = 1 - cur_;
    }
    double report_last_ms() final {
        auto d = std::chrono::duration_cast<std::chrono::microseconds>(trace_[1 - cur_] - trace_[cur_]);
        return d.count() / 1e3;
    }

  private:
    decltype(std::chrono::high_resolution_clock::now()) trace_[2];
    int cur_ = 0;
};

struct GPUTimer : public Timer {
    GPUTimer() {
        MI_CHECK(mi_event_create(&events_[0]));
        MI_CHECK(mi_event_create(&events_[1]));
    }
    ~GPUTimer() {
        mi_event_destroy(events_[0]);
        mi_event_destroy(events_[1]);
    }
    void tick() final {
        MI_CHECK(mi_event_record(events_[cur_], nullptr));
        cur_ = 1 - cur_;
    }
    double report_last_ms() final {
        float ms;
        MI_CHECK(mi_event_sync(events_[1 - cur_]));
        MI_CHECK(mi_event_elapsed_ms(&ms, events_[cur_], events_[1 - cur_]));
        return ms;
    }
    void sync_all() { MI_CHECK(mi_device_sync()); }

  private:
    void* events_[2];
    int cur_ = 0;
};

// ---- tensors (common.h:275-365) --------------------------------------------------------

inline size_t shape_numel(const std::vector<int>& shape) {
    return std::accumulate(shape.begin(), shape.end(), (size_t)1, std::multiplies<size_t>());
}

template <class DType>
DType* alloc_cpu_tensor(std::vector<int> shape) {
    return (DType*)malloc(shape_numel(shape) * sizeof(DType));
}

// values (r % 1000 * 1 / 100 % 10 - 5.0): integers in [-5, 4] from rand(), as the reference.
template <class DType>
void random_fill(DType* tensor, std::vector<int> shape) {
    const size_t length = shape_numel(shape);
    for (size_t i = 0; i < length; ++i) tensor[i] = (DType)((rand() % 1000 * 1 / 100 % 10 - 5.0));
}

template <class DType>
void arange_fill(DType* tensor, std::vector<int> shape, int bound = 1024) {
    const size_t length = shape_numel(shape);
    for (size_t i = 0; i < length; ++i) tensor[i] = (DType)((int)(i % (size_t)bound));
}

template <class DType>
void constant_fill(DType* tensor, std::vector<int> shape, DType value) {
    const size_t length = shape_numel(shape);
    for (size_t i = 0; i < length; ++i) tensor[i] = value;
}

// Seeded, counter-based fills used for the benchmark configurations: element i of stream s
// is a pure function of (seed, s, i), so the same matrices can be regenerated anywhere.
// (The reference's own generators are unseeded rand() and a library-defined
// std::normal_distribution; these are this library's additions.)
inline uint64_t mi_mix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
inline uint64_t mi_rng_u64(uint64_t seed, uint64_t stream, uint64_t index) {
    return mi_mix64(mi_mix64(seed ^ (stream * 0xd1342543de82ef95ull)) + index);
}
// fn(begin, end) over [0, length) in contiguous pieces on up to 16 host threads (the fills below
// are pure functions of the index, so the result does not depend on the split)
template <class Fn>
void for_index_ranges(size_t length, Fn fn) {
    const unsigned hw = std::thread::hardware_concurrency();
    const size_t nt = std::min<size_t>(std::min<size_t>(hw ? hw : 1, 16), std::max<size_t>(1, length >> 20));
    if (nt <= 1) return fn((size_t)0, length);
    std::vector<std::thread> pool;
    for (size_t t = 0; t < nt; ++t) pool.emplace_back(fn, length * t / nt, length * (t + 1) / nt);
    for (auto& th : pool) th.join();
}
// i.i.d. uniform on the 2^-23 grid of [-1, 1), rounded to the storage type.
template <class DType>
void uniform_fill(DType* tensor, std::vector<int> shape, uint64_t seed, uint64_t stream) {
    for_index_ranges(shape_numel(shape), [=](size_t b, size_t e) {
        for (size_t i = b; i < e; ++i) {
            const float u = (float)(mi_rng_u64(seed, stream, i) >> 40) * (1.0f / 16777216.0f);
            tensor[i] = DType(2.0f * u - 1.0f);
        }
    });
}
// i.i.d. N(0, sigma^2) by Box-Muller in double, rounded once to the storage type.
template <class DType>
void normal_fill(DType* tensor, std::vector<int> shape, uint64_t seed, uint64_t stream,
                 float sigma = 1.0f) {
    for_index_ranges(shape_numel(shape), [=](size_t b, size_t e) {
        for (size_t i = b; i < e; ++i) {
            const uint64_t r = mi_rng_u64(seed, stream, i);
            const double u1 = ((double)(r >> 40) + 1.0) * (1.0 / 16777216.0);
            const double u2 = (double)(r & 0xffffffull) * (1.0 / 16777216.0);
            const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2);
            tensor[i] = DType((float)(z * (double)sigma));
        }
    });
}

template <class DType>
DType* alloc_gpu_tensor(std::vector<int> shape) {
    void* dt;
    MI_CHECK(mi_malloc(&dt, shape_numel(shape) * sizeof(DType)));
    return (DType*)dt;
}

template <class DType>
void free_cpu_tensor(DType* ptr) {
    free(ptr);
}

template <class DType>
void free_gpu_tensor(DType* ptr) {
    MI_CHECK(mi_free((void*)ptr));
}

template <class DType>
void copy_to_gpu(DType* hptr, DType* dptr, std::vector<int> shape) {
    MI_CHECK(mi_memcpy_h2d(dptr, hptr, shape_numel(shape) * sizeof(DType)));
}

template <class DType>
void copy_to_cpu(DType* hptr, DType* dptr, std::vector<int> shape) {
    MI_CHECK(mi_memcpy_d2h(hptr, dptr, shape_numel(shape) * sizeof(DType)));
}

// assert_allclose (common.h:367-397): pure relative test |r-g| > rtol*|g|, no infinities
// allowed, error statistics printed, and the process aborts when any element fails.
template <class DType>
void assert_allclose(DType* res_ptr, DType* golden_ptr, std::vector<int> shape, float rtol = 1e-5,
                     bool dump = false) {
    long long errors = 0;
    const size_t length = shape_numel(shape);
    const int row_size = shape[shape.size() - 1];
    double total_diff = 0.0;
    for (size_t i = 0; i < length; ++i) {
        float r = (float)res_ptr[i];
        float g = (float)golden_ptr[i];
        if (std::isinf(r)) { std::cout << "Result value contains inf.\n"; abort(); }
        if (std::isinf(g)) { std::cout << "Golden value contains inf.\n"; abort(); }
        if (std::fabs(r - g) > rtol * std::fabs(g)) {
            errors += 1;
            total_diff += std::fabs(r - g);
        }
        if (dump) {
            std::cout << "(" << r << " " << g << ") ";
            if ((i + 1) % row_size == 0) std::cout << "\n";
        }
    }
    if (errors > 0) {
        std::cout << "Wrong answer! " << errors << " errors! " << (float)errors / length * 100 << "%\n";
        std::cout << "Average diff = " << total_diff / errors << "\n";
        std::cout.flush();
        abort();   // the reference's assert(errors == 0), kept alive under NDEBUG
    }
}

inline int get_sm_count() {
    mi_device_props p;
    if (mi_get_device_props(&p) != MI_OK) {
        std::cerr << "mi_get_device_props() returned error " << mi_last_error() << std::endl;
        return 1;
    }
    return p.compute_units;
}

// ---- launchers ---------------------------------------------------------------------------

// reference_gpu_gemm (reference.h:78-90): plain ascending-k GEMM on the GPU, used as golden.
template <class AType, class BType, class CType, class AccumType>
void reference_gpu_gemm(GemmParams<AType, BType, CType, AccumType> params) {
    static_assert(mi_dtype_of<AType>::value == mi_dtype_of<BType>::value &&
                  mi_dtype_of<AType>::value == mi_dtype_of<CType>::value, "one storage type");
    MI_CHECK(mi_reference_gpu_gemm(mi_dtype_of<AType>::value, params.M, params.N, params.K,
                                   params.A, params.B, params.C, (float)params.alpha,
                                   (float)params.beta, nullptr));
}

// gpu_gemm (matmul_h100.cu.jinja:927-985).  The reference's six integer template arguments
// selected a Hopper tile; here the kernel configuration is a run-time index (or name) into
// the library's table, MI_CONFIG_AUTO by default.  Like the reference kernel it ignores
// alpha and beta (matmul_h100.cu.jinja:696) and computes alpha = 1, beta = 0.
template <class AType, class BType, class CType, class AccumType>
void gpu_gemm(GemmParams<AType, BType, CType, AccumType> gemm_params, int config = MI_CONFIG_AUTO) {
    static_assert(mi_dtype_of<AType>::value == mi_dtype_of<BType>::value &&
                  mi_dtype_of<AType>::value == mi_dtype_of<CType>::value, "one storage type");
    MI_CHECK(mi_gemm_ex(config, mi_dtype_of<AType>::value, gemm_params.M, gemm_params.N,
                        gemm_params.K, gemm_params.A, gemm_params.B, gemm_params.C, nullptr,
                        nullptr));
}

// gpu_gemm with the epilogue the reference's kernels leave out: C = (CType)(acc * alpha + beta)
// from the GemmParams (beta a plain scalar, reference.h:40), C row-major or column-major
// (C[n*M + m], what the bf16 kernel behind runKernel writes, matmul_utils.cuh:529,545).
template <class AType, class BType, class CType, class AccumType>
void gpu_gemm_epilogue(GemmParams<AType, BType, CType, AccumType> gemm_params, int c_layout = MI_C_ROW_MAJOR,
                       int config = MI_CONFIG_AUTO) {
    static_assert(mi_dtype_of<AType>::value == mi_dtype_of<BType>::value &&
                  mi_dtype_of<AType>::value == mi_dtype_of<CType>::value, "one storage type");
    MI_CHECK(mi_gemm_epilogue(config, mi_dtype_of<AType>::value, gemm_params.M, gemm_params.N,
                              gemm_params.K, gemm_params.A, gemm_params.B, gemm_params.C,
                              (float)gemm_params.alpha, (float)gemm_params.beta, c_layout, nullptr));
}

// runKernel / run_kernel (matmul_h100_optimal.cu:32-59, 75-84).  kernel_num 1 is this
// library's kernel.  0 is a vendor BLAS in the reference (runCublasGemmBF16,
// matmul_h100_optimal.cu:63-73): the library links none, so a program that wants that arm
// defines MI_HOST_VENDOR_GEMM to its own `void f(int M, int N, int K, void* A, void* B,
// void* C)` before including this header (vendor_bench.cpp does, with hipBLASLt).
inline void runKernel(int M, int N, int K, bf16* A, bf16* B, bf16* C, int* DB) {
    MI_CHECK(mi_gemm_bf16(M, N, K, (const uint16_t*)A, (const uint16_t*)B, (uint16_t*)C, DB, nullptr));
}

inline void run_kernel(int kernel_num, int M, int N, int K, bf16* A, bf16* B, bf16* C,
                       int* DB = nullptr) {
    switch (kernel_num) {
#ifdef MI_HOST_VENDOR_GEMM
        case 0:
            MI_HOST_VENDOR_GEMM(M, N, K, (void*)A, (void*)B, (void*)C);
            break;
#endif
        case 1:
            runKernel(M, N, K, A, B, C, DB);
            break;
        default:
            std::cerr << "run_kernel: kernel " << kernel_num << " is not built into this library\n";
            exit(1);
    }
}

// randomize_matrix (matmul_h100_optimal.cu:86-92): N(0,1) from a default_random_engine(69)
// shared by all calls.
inline std::default_random_engine& mi_generator() {
    static std::default_random_engine generator(69);
    return generator;
}
inline void randomize_matrix(bf16* mat, size_t N) {
    std::normal_distribution<float> distribution(0, 1);
    for (size_t i = 0; i < N; i++) mat[i] = bf16(distribution(mi_generator()));
}

// verify_matrix (matmul_h100_optimal.cu:94-108): bf16(ref - out) must not exceed 0.1.
inline bool verify_matrix(bf16* matRef, bf16* matOut, size_t N) {
    for (size_t i = 0; i < N; i++) {
        double diff = std::fabs((float)bf16((float)matRef[i] - (float)matOut[i]));
        if (diff > 0.1) {
            printf("Divergence! Should %5.2f, Is %5.2f (Diff %5.2f) at %zu\n", (float)matRef[i],
                   (float)matOut[i], diff, i);
            return false;
        }
    }
    return true;
}

// The acceptance test of this library's benchmark configurations (not a reference
// function): every element must satisfy
//     |out - ref| <= 2^-7 * |ref| + 1e-3 * sqrt(K) * max|a| * max|b|.
// verify_matrix's absolute 0.1 is tighter than one bf16 unit in the last place once
// |C| >= 16, so two correct fp32-accumulating GEMMs that sum in different orders fail it
// at the benchmark sizes; the reference leaves it disabled (matmul_h100_optimal.cu:177).
// Returns the number of violating elements and prints the first one.
template <class DType>
inline size_t verify_tolerance(const DType* ref, const DType* out, size_t n, int K, double max_a,
                               double max_b) {
    const double abs_term = 1e-3 * std::sqrt((double)K) * max_a * max_b;
    size_t bad = 0;
    for (size_t i = 0; i < n; ++i) {
        const double r = (float)ref[i], o = (float)out[i];
        const double err = std::fabs(o - r);
        if (!(err <= std::fabs(r) / 128.0 + abs_term)) {
            if (bad == 0)
                printf("Divergence! Should %5.2f, Is %5.2f (Diff %5.2f) at %zu\n", r, o, err, i);
            ++bad;
        }
    }
    return bad;
}
template <class DType>
inline double max_abs_value(const DType* x, size_t n) {
    double m = 0.0;
    for (size_t i = 0; i < n; ++i) m = std::max(m, (double)std::fabs((float)x[i]));
    return m;
}
