// mi_gemm.hip -- C ABI of libmi_gemm.so (declared in include/mi_gemm.h): the kernel
// configuration table, shape -> kernel dispatch, and the thin HIP layer the harness uses.
//
// The launch path stands where the reference's host launchers stand: runKernel
// (matmul_h100_optimal.cu:32-59) and gpu_gemm (matmul_h100.cu.jinja:927-985).  Those build
// TMA descriptors, set a shared-memory attribute and launch a persistent grid of 128 CTAs;
// here a launch is a plain grid of one workgroup per output tile, the descriptors are
// built inside the kernel from the raw pointers, and nothing is cached between calls (the
// reference keeps descriptors in globals keyed on M alone, matmul_utils.cuh:49-51).
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/mi_gemm.h"
#include "gemm_kernel.hpp"
#include "kernel_table.hpp"

namespace mi {
hipError_t launch_reference_gpu_gemm(int dtype, int M, int N, int K, const void* A, const void* B,
                                     void* C, float alpha, float beta, hipStream_t stream);
}

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

#define MI_HIP(call)                                                                  \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess)                                                         \
            return fail(MI_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                        __FILE__, __LINE__);                                          \
    } while (0)

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// The aligned kernels assume full tiles, K a multiple of two K steps, 16-byte aligned
// rows of A and B and 8-byte aligned rows of C; everything else takes the predicated twin.
bool shape_is_aligned(const mi::KernelEntry& e, int M, int N, int K, const void* A,
                      const void* B, const void* C) {
    return M % e.BM == 0 && N % e.BN == 0 && K % 128 == 0 && aligned16(A) && aligned16(B) &&
           aligned16(C);
}

int check_args(int config, int dtype, int M, int N, int K, const void* A, const void* B,
               const void* C) {
    if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
        return fail(MI_ERR_INVALID, "unknown dtype %d", dtype);
    if (M <= 0 || N <= 0 || K <= 0)
        return fail(MI_ERR_INVALID, "M, N, K must be positive (got %d, %d, %d)", M, N, K);
    if (!A || !B || !C) return fail(MI_ERR_INVALID, "null matrix pointer");
    if (config != MI_CONFIG_AUTO && (config < 0 || config >= mi::kNumKernels))
        return fail(MI_ERR_INVALID, "unknown kernel config %d", config);
    // 32-bit byte offsets inside one tile's row panel, and `int` element indices as in the
    // reference (reference.h:30,40 index with int).
    if ((long long)M * K > 0x7fffffffLL || (long long)N * K > 0x7fffffffLL ||
        (long long)M * N > 0x7fffffffLL)
        return fail(MI_ERR_INVALID, "matrix with more than 2^31-1 elements");
    if ((long long)K * 2 * 256 > 0x7fffffffLL) return fail(MI_ERR_INVALID, "K too large");
    return MI_OK;
}

}  // namespace

extern "C" {

const char* mi_last_error(void) { return g_err; }

int mi_gemm_num_configs(void) { return mi::kNumKernels; }

const char* mi_gemm_config_name(int config) {
    if (config < 0 || config >= mi::kNumKernels) return nullptr;
    return mi::kKernels[config].name;
}

int mi_gemm_find_config(const char* name) {
    if (!name) return -1;
    for (int i = 0; i < mi::kNumKernels; ++i)
        if (strcmp(name, mi::kKernels[i].name) == 0) return i;
    return -1;
}

int mi_gemm_config_lds_bytes(int config) {
    if (config < 0 || config >= mi::kNumKernels) return 0;
    return mi::kKernels[config].lds_bytes;
}

int mi_gemm_config_supports(int config, int dtype, int M, int N, int K) {
    if (config < 0 || config >= mi::kNumKernels) return 0;
    if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16) return 0;
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return mi::kKernels[config].launch[dtype][1] != nullptr;
}

int mi_gemm_config_grid(int config, int M, int N, int K) {
    if (config < 0 || config >= mi::kNumKernels || M <= 0 || N <= 0 || K <= 0) return 0;
    const mi::KernelEntry& e = mi::kKernels[config];
    return ((M + e.BM - 1) / e.BM) * ((N + e.BN - 1) / e.BN);
}

int mi_gemm_select_config(int dtype, int M, int N, int K) {
    (void)dtype;
    (void)K;
    return mi::select_kernel(M, N, K);
}

size_t mi_gemm_trace_words(int M, int N, int K) {
    // enough for whichever kernel configuration ends up running the shape
    size_t grid = 0;
    for (int c = 0; c < mi::kNumKernels; ++c) {
        const size_t g = (size_t)mi_gemm_config_grid(c, M, N, K);
        if (g > grid) grid = g;
    }
    return grid * 6 + 1;
}

int mi_gemm_ex(int config, int dtype, int M, int N, int K, const void* A, const void* B,
               void* C, int* DB, void* stream) {
    int rc = check_args(config, dtype, M, N, K, A, B, C);
    if (rc != MI_OK) return rc;
    if (config == MI_CONFIG_AUTO) config = mi::select_kernel(M, N, K);
    const mi::KernelEntry& e = mi::kKernels[config];

    mi::GemmArgs args;
    args.A = A;
    args.B = B;
    args.C = C;
    args.M = M;
    args.N = N;
    args.K = K;
    args.lda = K;
    args.ldb = K;
    args.ldc = N;
    args.tiles_m = (M + e.BM - 1) / e.BM;
    args.tiles_n = (N + e.BN - 1) / e.BN;
    args.c_vec_ok = (N % 4 == 0) && (((uintptr_t)C & 7u) == 0);
    args.DB = DB;

    const bool edge = !shape_is_aligned(e, M, N, K, A, B, C);
    mi::LaunchFn fn = e.launch[dtype][edge ? 1 : 0];
    if (!fn) return fail(MI_ERR_UNSUPPORTED, "config %s has no %s kernel for dtype %d", e.name,
                         edge ? "predicated" : "aligned", dtype);
    hipError_t err = fn(args, (hipStream_t)stream);
    if (err != hipSuccess)
        return fail(MI_ERR_HIP, "launch of %s failed: %s", e.name, hipGetErrorString(err));
    return MI_OK;
}

int mi_gemm_bf16(int M, int N, int K, const uint16_t* A, const uint16_t* B, uint16_t* C, int* DB,
                 void* stream) {
    return mi_gemm_ex(MI_CONFIG_AUTO, MI_DTYPE_BF16, M, N, K, A, B, C, DB, stream);
}

int mi_reference_gpu_gemm(int dtype, int M, int N, int K, const void* A, const void* B, void* C,
                          float alpha, float beta, void* stream) {
    int rc = check_args(MI_CONFIG_AUTO, dtype, M, N, K, A, B, C);
    if (rc != MI_OK) return rc;
    hipError_t err =
        mi::launch_reference_gpu_gemm(dtype, M, N, K, A, B, C, alpha, beta, (hipStream_t)stream);
    if (err != hipSuccess)
        return fail(MI_ERR_HIP, "launch of the reference GEMM failed: %s", hipGetErrorString(err));
    return MI_OK;
}

// ---- thin HIP layer -------------------------------------------------------------------

int mi_malloc(void** dptr, size_t bytes) {
    if (!dptr) return fail(MI_ERR_INVALID, "mi_malloc: null out pointer");
    MI_HIP(hipMalloc(dptr, bytes));
    return MI_OK;
}
int mi_free(void* dptr) {
    MI_HIP(hipFree(dptr));
    return MI_OK;
}
int mi_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    MI_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return MI_OK;
}
int mi_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    MI_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return MI_OK;
}
int mi_memset(void* dst, int value, size_t bytes) {
    MI_HIP(hipMemset(dst, value, bytes));
    return MI_OK;
}
int mi_device_sync(void) {
    MI_HIP(hipDeviceSynchronize());
    return MI_OK;
}
int mi_stream_sync(void* stream) {
    MI_HIP(hipStreamSynchronize((hipStream_t)stream));
    return MI_OK;
}
int mi_event_create(void** ev) {
    if (!ev) return fail(MI_ERR_INVALID, "mi_event_create: null out pointer");
    hipEvent_t e;
    MI_HIP(hipEventCreate(&e));
    *ev = (void*)e;
    return MI_OK;
}
int mi_event_destroy(void* ev) {
    MI_HIP(hipEventDestroy((hipEvent_t)ev));
    return MI_OK;
}
int mi_event_record(void* ev, void* stream) {
    MI_HIP(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
    return MI_OK;
}
int mi_event_sync(void* ev) {
    MI_HIP(hipEventSynchronize((hipEvent_t)ev));
    return MI_OK;
}
int mi_event_elapsed_ms(float* ms, void* start, void* stop) {
    if (!ms) return fail(MI_ERR_INVALID, "mi_event_elapsed_ms: null out pointer");
    MI_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return MI_OK;
}

int mi_get_device_props(mi_device_props* out) {
    if (!out) return fail(MI_ERR_INVALID, "mi_get_device_props: null out pointer");
    int dev = 0;
    MI_HIP(hipGetDevice(&dev));
    hipDeviceProp_t p;
    MI_HIP(hipGetDeviceProperties(&p, dev));
    memset(out, 0, sizeof *out);
    snprintf(out->name, sizeof out->name, "%s", p.name);
    snprintf(out->arch, sizeof out->arch, "%s", p.gcnArchName);
    out->compute_units = p.multiProcessorCount;
    out->clock_khz = p.clockRate;
    out->mem_clock_khz = p.memoryClockRate;
    out->mem_bus_bits = p.memoryBusWidth;
    out->lds_bytes_per_block = (int)p.sharedMemPerBlock;
    out->l2_bytes = p.l2CacheSize;
    out->wavefront = p.warpSize;
    out->hbm_bytes = p.totalGlobalMem;
    return MI_OK;
}

}  // extern "C"
