// vendor_bench.cpp -- this library's kernel side by side with the vendor BLAS on the same
// device buffers: the `for (int kernel_num : {0, 1})` loop of the reference's benchmark
// program (matmul_h100_optimal.cu:157-217), where kernel 0 is a vendor GEMM
// (runCublasGemmBF16 / cublasGemmEx, matmul_h100_optimal.cu:63-73; hipBLASLt here) and
// kernel 1 is the hand-written one.  The vendor library is linked into THIS program only:
// it is a comparison, never a dispatch path of libmi_gemm.so.
//
//     ./vendor_bench [M N K] [repeats] [settle_ms]      default 8192 8192 8192 200 150
//
// Per kernel: `KERNEL n`, one verification launch (kernel 1 is compared element by element
// with kernel 0's result -- the check matmul_h100_optimal.cu:177-180 leaves disabled -- with
// the bound 2^-7*|ref| + 1e-3*sqrt(K)*max|a|*max|b|), `settle_ms` of untimed launches (the
// chip needs ~100 ms under load before its clock settles; the reference sleeps 5 s and
// times 8 launches cold), then `repeats` launches between two events and the reference's
// line `Average elapsed time: (s) s, performance: (T) TFLOPS. size: (M).`
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

static void runVendorGemmBF16(int M, int N, int K, void* A, void* B, void* C);
#define MI_HOST_VENDOR_GEMM runVendorGemmBF16
#include "gemm_host.hpp"

#define HIP_OK(call)                                                                        \
    do {                                                                                    \
        hipError_t e_ = (call);                                                             \
        if (e_ != hipSuccess) {                                                             \
            std::cerr << __FILE__ << ":" << __LINE__ << " " << hipGetErrorString(e_) << "\n"; \
            exit(1);                                                                        \
        }                                                                                   \
    } while (0)
#define LT_OK(call)                                                                         \
    do {                                                                                    \
        hipblasStatus_t s_ = (call);                                                        \
        if (s_ != HIPBLAS_STATUS_SUCCESS) {                                                 \
            std::cerr << __FILE__ << ":" << __LINE__ << " hipBLASLt status " << (int)s_ << "\n"; \
            exit(1);                                                                        \
        }                                                                                   \
    } while (0)

// C[M,N] (row-major) = A[M,K] . B[N,K]^T, bf16 storage, fp32 compute.  In the column-major
// terms of the BLAS: C' (N x M, ld N) = op(B') . A' with B' = K x N (ld K) transposed and
// A' = K x M (ld K) as is -- the "TN" GEMM.  Handle, descriptors, the heuristic's first
// algorithm and a 64 MiB workspace are set up once per shape.
static void runVendorGemmBF16(int M, int N, int K, void* A, void* B, void* C) {
    static hipblasLtHandle_t handle = nullptr;
    static hipblasLtMatmulDesc_t desc = nullptr;
    static hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    static hipblasLtMatmulHeuristicResult_t algo;
    static void* workspace = nullptr;
    static const size_t workspace_bytes = 64u << 20;
    static int cm = -1, cn = -1, ck = -1;
    if (!handle) {
        LT_OK(hipblasLtCreate(&handle));
        HIP_OK(hipMalloc(&workspace, workspace_bytes));
    }
    if (cm != M || cn != N || ck != K) {
        if (desc) {
            hipblasLtMatmulDescDestroy(desc);
            hipblasLtMatrixLayoutDestroy(la);
            hipblasLtMatrixLayoutDestroy(lb);
            hipblasLtMatrixLayoutDestroy(lc);
        }
        LT_OK(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
        const hipblasOperation_t opT = HIPBLAS_OP_T, opN = HIPBLAS_OP_N;
        LT_OK(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opT, sizeof(opT)));
        LT_OK(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opN, sizeof(opN)));
        LT_OK(hipblasLtMatrixLayoutCreate(&la, HIP_R_16BF, K, N, K));   // B' (stored K x N)
        LT_OK(hipblasLtMatrixLayoutCreate(&lb, HIP_R_16BF, K, M, K));   // A'
        LT_OK(hipblasLtMatrixLayoutCreate(&lc, HIP_R_16BF, N, M, N));   // C'
        hipblasLtMatmulPreference_t pref;
        LT_OK(hipblasLtMatmulPreferenceCreate(&pref));
        LT_OK(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES,
                                                    &workspace_bytes, sizeof(workspace_bytes)));
        int found = 0;
        LT_OK(hipblasLtMatmulAlgoGetHeuristic(handle, desc, la, lb, lc, lc, pref, 1, &algo, &found));
        hipblasLtMatmulPreferenceDestroy(pref);
        if (found < 1) {
            std::cerr << "hipBLASLt has no algorithm for " << M << "x" << N << "x" << K << "\n";
            exit(1);
        }
        cm = M, cn = N, ck = K;
    }
    const float alpha = 1.0f, beta = 0.0f;
    LT_OK(hipblasLtMatmul(handle, desc, &alpha, B, la, A, lb, &beta, C, lc, C, lc, &algo.algo,
                          workspace, workspace_bytes, nullptr));
}

int main(int argc, char** argv) {
    long m = 8192, n = 8192, k = 8192;
    int arg = 1;
    if (argc >= 4) {
        m = std::atol(argv[1]), n = std::atol(argv[2]), k = std::atol(argv[3]);
        arg = 4;
    }
    const int repeat_times = argc > arg ? std::atoi(argv[arg]) : 200;
    const double settle_ms = argc > arg + 1 ? std::atof(argv[arg + 1]) : 150.0;
    if (m < 1 || n < 1 || k < 1 || repeat_times < 1) {
        std::cerr << "usage: vendor_bench [M N K] [repeats] [settle_ms]\n";
        return 2;
    }
    printf("Shape M=%ld, N=%ld, K=%ld\n", m, n, k);

    float elapsed_time;
    void *start, *stop;
    MI_CHECK(mi_event_create(&start));
    MI_CHECK(mi_event_create(&stop));

    const size_t ea = (size_t)m * k, eb = (size_t)n * k, ec = (size_t)m * n;
    bf16* A = (bf16*)malloc(sizeof(bf16) * ea);
    bf16* B = (bf16*)malloc(sizeof(bf16) * eb);
    bf16* C = (bf16*)malloc(sizeof(bf16) * ec);
    bf16* C_ref = (bf16*)malloc(sizeof(bf16) * ec);
    randomize_matrix(A, ea);
    randomize_matrix(B, eb);
    const double max_a = max_abs_value(A, ea), max_b = max_abs_value(B, eb);

    void *dA, *dB, *dC, *dC_ref;
    MI_CHECK(mi_malloc(&dA, sizeof(bf16) * ea));
    MI_CHECK(mi_malloc(&dB, sizeof(bf16) * eb));
    MI_CHECK(mi_malloc(&dC, sizeof(bf16) * ec));
    MI_CHECK(mi_malloc(&dC_ref, sizeof(bf16) * ec));
    MI_CHECK(mi_memcpy_h2d(dA, A, sizeof(bf16) * ea));
    MI_CHECK(mi_memcpy_h2d(dB, B, sizeof(bf16) * eb));

    double tflops[2] = {0, 0};
    for (int kernel_num : {0, 1}) {
        std::cout << "KERNEL " << kernel_num << std::endl;
        void* out = kernel_num == 0 ? dC_ref : dC;
        MI_CHECK(mi_memset(out, 0, sizeof(bf16) * ec));
        run_kernel(kernel_num, (int)m, (int)n, (int)k, (bf16*)dA, (bf16*)dB, (bf16*)out);
        MI_CHECK(mi_device_sync());
        if (kernel_num > 0) {
            MI_CHECK(mi_memcpy_d2h(C, dC, sizeof(bf16) * ec));
            MI_CHECK(mi_memcpy_d2h(C_ref, dC_ref, sizeof(bf16) * ec));
            const size_t bad = verify_tolerance(C_ref, C, ec, (int)k, max_a, max_b);
            if (bad != 0) {
                std::cout << "~~~~~~~~~~~~~~~~ Failed to pass the correctness verification against the "
                             "vendor BLAS. ~~~~~~~~~~~~~~~~ (" << bad << " elements)" << std::endl;
                return 1;
            }
            std::cout << "Matches the vendor BLAS within tolerance." << std::endl;
        }
        // untimed launches until the clock has settled under load
        if (settle_ms > 0) {
            float ms = 0;
            do {
                MI_CHECK(mi_event_record(start, nullptr));
                for (int j = 0; j < 10; j++) run_kernel(kernel_num, (int)m, (int)n, (int)k, (bf16*)dA, (bf16*)dB, (bf16*)out);
                MI_CHECK(mi_event_record(stop, nullptr));
                MI_CHECK(mi_event_sync(stop));
                MI_CHECK(mi_event_elapsed_ms(&elapsed_time, start, stop));
                ms += elapsed_time;
            } while (ms < settle_ms);
        }
        MI_CHECK(mi_event_record(start, nullptr));
        for (int j = 0; j < repeat_times; j++) run_kernel(kernel_num, (int)m, (int)n, (int)k, (bf16*)dA, (bf16*)dB, (bf16*)out);
        MI_CHECK(mi_event_record(stop, nullptr));
        MI_CHECK(mi_event_sync(start));
        MI_CHECK(mi_event_sync(stop));
        MI_CHECK(mi_event_elapsed_ms(&elapsed_time, start, stop));

        const double flops = 2.0 * (double)m * (double)n * (double)k;
        tflops[kernel_num] = (repeat_times * flops * 1e-9) / elapsed_time;
        printf("Average elapsed time: (%7.6f) s, performance: (%7.1f) TFLOPS. size: (%ld).\n\n",
               elapsed_time / 1000.0 / repeat_times, tflops[kernel_num], m);
    }
    printf("kernel 1 / kernel 0: %.3f\n", tflops[1] / tflops[0]);

    free(A); free(B); free(C); free(C_ref);
    mi_free(dA); mi_free(dB); mi_free(dC); mi_free(dC_ref);
    return 0;
}
