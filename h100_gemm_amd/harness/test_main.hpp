// test_main.hpp -- body of the `./test M m N n K k` program of the reference
// (main() of matmul_h100.cu.jinja:987-1079), shared by the library-dispatch build
// (gemm_test.cpp) and by the tuner's rendered single-configuration programs
// (template/matmul_mi355x.hip.jinja).
//
// Same flow as the reference: integer random_fill inputs, golden from reference_gpu_gemm,
// the kernel's output compared with assert_allclose(rtol = 1e-3), then a timed loop, and the
// same stdout lines the tuner parses ("Shape ...", "Correct!", "Average latency (ms) is X").
// Extra key/value pairs, ignored by the reference's parser:
//     cfg <index|name>   kernel configuration (library build only; default: its own choice)
//     dtype <bf16|fp16>  storage type (default bf16; the reference program is fp16)
//     iters <n>          timed launches (default 200, as in the reference)
//     check <0|1>        skip / run the comparison (default 1)
//     rotate <n>         copies of A and B the timed launches take in turn.  Default 0: for
//                        a shape that HBM bounds (fewer flops per byte than the chip's peaks
//                        stand for) and whose A, B and C together fit the 256 MB memory-side
//                        cache, as many as make the set 512 MiB, at most eight; else one.
//                        That cache would otherwise hold a B of 128 MiB from one launch to
//                        the next, and a timing loop over one buffer would rank the decode
//                        kernels by how they read the cache, not HBM
//     fill <int|uniform|normal>  inputs: the reference's integer random_fill (default),
//                        seeded U[-1,1), or seeded A ~ N(0,1), B ~ N(0,0.02^2); with the
//                        last two the sums are inexact and the comparison is the bound
//                        2^-7*|ref| + 1e-3*sqrt(K)*max|a|*max|b| instead of rtol
//     alpha <a> beta <b> the golden's epilogue C = (CType)(acc*alpha + beta), beta a plain
//                        scalar (reference.h:40; the reference's harness passes 1 and 0,
//                        matmul_h100.cu.jinja:1014-1015)           } library build only:
//     cmajor <0|1>       1: the kernel writes C column-major,      } the launch function
//                        C[n*M + m] (matmul_utils.cuh:545)         } reads test_epilogue()
#pragma once

#include <algorithm>
#include <functional>
#include <string>
#include <vector>

#include "gemm_host.hpp"

// launch(dtype, config, M, N, K, A, B, C): enqueue one GEMM on the null stream
using TestLaunchFn = std::function<void(int, int, int, int, int, const void*, const void*, void*)>;

// epilogue options of the run (alpha, beta, C layout); a launch function that cannot honour
// them leaves `supported` false and test_main refuses non-default values
struct TestEpilogue {
    float alpha = 1.0f, beta = 0.0f;
    int c_layout = MI_C_ROW_MAJOR;
    bool supported = false;
};
inline TestEpilogue& test_epilogue() {
    static TestEpilogue e;
    return e;
}

const int testM = 4096;
const int testN = 4096;
const int testK = 4096;

template <class T>
int run_test(int M, int N, int K, int config, int iters, bool check, int rotate, const std::string& fill,
             const TestLaunchFn& launch, const std::function<std::string(int)>& label) {
    using AType = T;
    using BType = T;
    using CType = T;
    using AccumType = float;
    AccumType alpha = test_epilogue().alpha;
    AccumType beta = test_epilogue().beta;
    const bool cmajor = test_epilogue().c_layout == MI_C_COL_MAJOR;
    constexpr int dt = mi_dtype_of<T>::value;

    std::vector<int> AShape = {M, K};
    std::vector<int> BShape = {N, K};
    std::vector<int> CShape = {M, N};
    auto hA = alloc_cpu_tensor<AType>(AShape);
    auto hB = alloc_cpu_tensor<BType>(BShape);
    if (fill == "uniform") {
        uniform_fill(hA, AShape, 69, 1);
        uniform_fill(hB, BShape, 69, 2);
    } else if (fill == "normal") {
        normal_fill(hA, AShape, 69, 1, 1.0f);
        normal_fill(hB, BShape, 69, 2, 0.02f);
    } else {
        random_fill(hA, AShape);
        random_fill(hB, BShape);
    }
    // (without the comparison the initial contents of C do not matter: no rand() pass over them)
    auto hC = alloc_cpu_tensor<CType>(CShape);
    auto goldenC = alloc_cpu_tensor<CType>(CShape);
    if (check) {
        random_fill(hC, CShape);
        random_fill(goldenC, CShape);
    } else {
        memset(hC, 0, shape_numel(CShape) * sizeof(CType));
        memset(goldenC, 0, shape_numel(CShape) * sizeof(CType));
    }
    auto dA = alloc_gpu_tensor<AType>(AShape);
    auto dB = alloc_gpu_tensor<BType>(BShape);
    auto dgC = alloc_gpu_tensor<CType>(CShape);
    auto dC = alloc_gpu_tensor<CType>(CShape);

    GPUTimer gpu_timer;

    copy_to_gpu(hA, dA, AShape);
    copy_to_gpu(hB, dB, BShape);
    copy_to_gpu(hC, dC, CShape);
    copy_to_gpu(goldenC, dgC, CShape);

    GemmParams<AType, BType, CType, AccumType> gpu_params(M, N, K, dA, dB, dgC, alpha, beta);

    if (check) {
        reference_gpu_gemm(gpu_params);
        copy_to_cpu(goldenC, dgC, CShape);
    }
    launch(dt, config, M, N, K, dA, dB, dC);
    copy_to_cpu(hC, dC, CShape);
    if (cmajor) {   // bring the column-major result into the golden's row-major order
        auto t = alloc_cpu_tensor<CType>(CShape);
        for (int m = 0; m < M; ++m)
            for (int n = 0; n < N; ++n) t[(size_t)m * N + n] = hC[(size_t)n * M + m];
        free_cpu_tensor(hC);
        hC = t;
    }
    if (check) {
        if (fill == "int") {
            assert_allclose(hC, goldenC, CShape, /*rtol=*/1e-3, /*dump=*/false);
        } else {
            // inexact sums: a pure relative test fails on results near zero; use the bound
            // 2^-7*|ref| + 1e-3*sqrt(K)*max|a|*max|b| instead
            const size_t bad = verify_tolerance(goldenC, hC, shape_numel(CShape), K,
                                                max_abs_value(hA, shape_numel(AShape)) * std::fabs((double)alpha),
                                                max_abs_value(hB, shape_numel(BShape)));
            if (bad != 0) {
                std::cout << "Wrong answer! " << bad << " errors!\n";
                std::cout.flush();
                abort();
            }
        }
        std::cout << "Correct!\n";
    }

    // the operand copies the timed launches rotate through
    if (rotate <= 0) {
        const size_t ab = (shape_numel(AShape) + shape_numel(BShape)) * sizeof(T);
        const size_t abc = ab + shape_numel(CShape) * sizeof(T);
        const bool hbm_bound = 2.0 * M * N * K / (double)abc < 2.5e15 / 8.0e12;       // flops per byte below the chip's ridge
        rotate = !hbm_bound || abc >= ((size_t)256 << 20) ? 1 : (int)std::min<size_t>(8, (((size_t)512 << 20) + ab - 1) / ab);
    }
    if (rotate > 1) std::cout << "Timing over " << rotate << " copies of A and B in turn\n";
    std::vector<AType*> rA = {dA};
    std::vector<BType*> rB = {dB};
    for (int c = 1; c < rotate; ++c) {
        rA.push_back(alloc_gpu_tensor<AType>(AShape));
        rB.push_back(alloc_gpu_tensor<BType>(BShape));
        copy_to_gpu(hA, rA.back(), AShape);
        copy_to_gpu(hB, rB.back(), BShape);
    }
    for (int i = 0; i < rotate; ++i) launch(dt, config, M, N, K, rA[i], rB[i], dC);   // untimed: first touch of every copy

    gpu_timer.sync_all();
    gpu_timer.tick();
    for (int i = 0; i < iters; ++i) launch(dt, config, M, N, K, rA[i % rotate], rB[i % rotate], dC);
    gpu_timer.tick();
    gpu_timer.sync_all();
    for (int c = 1; c < rotate; ++c) {
        free_gpu_tensor(rA[c]);
        free_gpu_tensor(rB[c]);
    }
    float latency = gpu_timer.report_last_ms() / float(iters);
    std::cout << "Average latency (ms) is " << latency << "\n";
    const double tflops = 2.0 * M * N * K / (latency * 1e-3) / 1e12;
    std::cout << "Config " << label(config) << ", " << tflops << " TFLOP/s\n";

    free_cpu_tensor(hA);
    free_cpu_tensor(hB);
    free_cpu_tensor(hC);
    free_cpu_tensor(goldenC);
    free_gpu_tensor(dA);
    free_gpu_tensor(dB);
    free_gpu_tensor(dC);
    free_gpu_tensor(dgC);
    return 0;
}

inline int test_main(int argc, char** argv, const TestLaunchFn& launch,
                     const std::function<std::string(int)>& label,
                     const std::function<int(const char*)>& parse_config) {
    int M = testM, N = testN, K = testK;
    int iters = 200, config = MI_CONFIG_AUTO, rotate = 0;
    bool check = true;
    std::string dtype = "bf16", fill = "int";
    if (argc > 1) {
        assert((argc - 1) % 2 == 0);
        for (int i = 1; i + 1 < argc; i += 2) {
            std::string keys(argv[i]);
            char* value = argv[i + 1];
            if (keys == "M") M = std::atoi(value);
            else if (keys == "N") N = std::atoi(value);
            else if (keys == "K") K = std::atoi(value);
            else if (keys == "iters") iters = std::atoi(value);
            else if (keys == "check") check = std::atoi(value) != 0;
            else if (keys == "rotate") rotate = std::atoi(value);
            else if (keys == "dtype") dtype = value;
            else if (keys == "fill") fill = value;
            else if (keys == "alpha") test_epilogue().alpha = (float)std::atof(value);
            else if (keys == "beta") test_epilogue().beta = (float)std::atof(value);
            else if (keys == "cmajor") test_epilogue().c_layout = std::atoi(value) ? MI_C_COL_MAJOR : MI_C_ROW_MAJOR;
            else if (keys == "cfg") {
                config = parse_config(value);
                if (config < 0) {
                    std::cerr << "unknown kernel config " << value << "\n";
                    return 2;
                }
            }
        }
    }
    const TestEpilogue& ep = test_epilogue();
    if (!ep.supported && (ep.alpha != 1.0f || ep.beta != 0.0f || ep.c_layout != MI_C_ROW_MAJOR)) {
        std::cerr << "alpha / beta / cmajor need the library build of this program (gemm_test.cpp)\n";
        return 2;
    }
    std::cout << "Shape M=" << M << ", N=" << N << ", K=" << K << "\n";
    if (dtype == "fp16") return run_test<half_t>(M, N, K, config, iters, check, rotate, fill, launch, label);
    return run_test<bf16>(M, N, K, config, iters, check, rotate, fill, launch, label);
}
