/*
 * mi_gemm.h -- C ABI of the MI355X (gfx950) dense GEMM library, libmi_gemm.so.
 *
 *     C[M,N] = A[M,K] . B[N,K]^T      16-bit float storage, fp32 accumulate (MFMA)
 *
 * A is M x K row-major, B is N x K row-major ("K-major"), C is M x N row-major; leading
 * dimensions are K, K and N.  All matrix pointers are DEVICE pointers owned by the
 * caller.  Launches are asynchronous on the given HIP stream (NULL = the null stream) and
 * C is fully overwritten (no read of C, beta = 0, alpha = 1), which is what the launchers
 * this library replaces do.
 *
 * Each entry point cites the host function of the reference project (Faraz9877/H100_GEMM)
 * whose place it takes.  The reference has no FFI: its boundary is a handful of host C++
 * functions linked into one executable; `h100_gemm_amd/harness/gemm_host.hpp` rebuilds
 * those functions (same names, same arguments, same exit-on-error behaviour) as inline
 * shims over this ABI.
 *
 * Every function returning int returns 0 on success and a negative MI_ERR_* code on
 * failure; mi_last_error() then holds a message for the calling thread.
 */
#ifndef MI_GEMM_H
#define MI_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_OK 0
#define MI_ERR_INVALID (-1) /* bad shape, null pointer, unknown config or dtype */
#define MI_ERR_HIP (-2)     /* a HIP runtime call failed; see mi_last_error()   */
#define MI_ERR_UNSUPPORTED (-3) /* the chosen kernel config cannot run this shape */

#define MI_DTYPE_BF16 0
#define MI_DTYPE_FP16 1

#define MI_CONFIG_AUTO (-1)

#define MI_C_ROW_MAJOR 0 /* element (m, n) of C at C[m*N + n] */
#define MI_C_COL_MAJOR 1 /* element (m, n) of C at C[n*M + m] */

/* ---- the GEMM ---------------------------------------------------------------------- */

/* bf16 GEMM with the library's own choice of kernel for the shape.
 * Replaces  void runKernel(int M, int N, int K, bf16* A, bf16* B, bf16* C, int* DB)
 * (matmul_h100_optimal.cu:32-59) and the `case 1` arm of run_kernel
 * (matmul_h100_optimal.cu:75-84).  DB may be NULL; when it is not, it is the device
 * trace buffer of that signature (see mi_gemm_trace_words()). */
int mi_gemm_bf16(int M, int N, int K, const uint16_t* A, const uint16_t* B, uint16_t* C,
                 int* DB, void* stream);

/* The same GEMM with an explicit kernel configuration and storage type.
 * Replaces  template<...> void gpu_gemm<AType,BType,CType,AccumType,CLUSTER_M,CLUSTER_N,
 * BLOCKM,BLOCKN,BLOCKK,STAGES>(GemmParams)  (matmul_h100.cu.jinja:927-985): the template
 * arguments of that launcher become `config` (an index into the table below, or
 * MI_CONFIG_AUTO) and `dtype` (MI_DTYPE_*). */
int mi_gemm_ex(int config, int dtype, int M, int N, int K, const void* A, const void* B,
               void* C, int* DB, void* stream);

/* The same GEMM with the epilogue and the C layouts of the reference's other code paths:
 *     C = (CType)(acc * alpha + beta)
 * as two separately rounded fp32 operations with beta a plain scalar added to every
 * element -- the epilogue of the reference's golden (reference.h:40, :69-76), which its
 * hand-written kernels skip (matmul_h100.cu.jinja:696) -- and C either row-major
 * (reference.h:40, matmul_h100.cu.jinja:696) or column-major, C[n*M + m], which is how the
 * bf16 kernel behind runKernel stores it (matmul_utils.cuh:529,545).  alpha = 1, beta = 0,
 * MI_C_ROW_MAJOR is exactly mi_gemm_ex without a trace buffer.  Column-major runs the
 * kernels on the exchanged operands (C^T = B . A^T), so the kernel is chosen for N x M x K. */
int mi_gemm_epilogue(int config, int dtype, int M, int N, int K, const void* A, const void* B,
                     void* C, float alpha, float beta, int c_layout, void* stream);

/* ---- split-K workspace -----------------------------------------------------------------
 * Shapes with few output tiles and a long K (decode shapes with 32 < M <= 128, 128 x 384 x
 * 13376, 800 x 800 x 6000, ...) run as split-K: fp32 partial sums [pieces][M][N] go to a workspace and a second
 * kernel adds them in a fixed order.  The three entry points above take that workspace from
 * the library: one buffer per (device, stream), a power of two of at least 4 MiB, allocated on
 * the first call that needs it and replaced by a larger one on demand; a replaced buffer is
 * kept (an enqueued launch or a captured graph may still hold its address) until
 * mi_gemm_release_workspace gives the stream's buffers back.  At most 16 streams per device
 * hold a buffer: a further stream waits for the device to go idle (hipDeviceSynchronize) and
 * takes over the smallest entry, so a process that keeps creating streams does not keep
 * growing (a graph captured from split-K launches on the stream that loses its entry must not
 * be replayed afterwards, as after a release: captured work that shares a process with more
 * than 16 GEMM streams should bring its own workspace).  A stream under capture that has no large enough buffer yet runs the launch unsplit;
 * a first or a growing use calls hipMalloc, which must not happen while ANY thread captures
 * in hipStreamCaptureModeGlobal: reserve beforehand (mi_gemm_reserve_workspace) or use
 * mi_gemm_epilogue_ws / mi_gemm_bf16_noalloc there.  The reference's launchers allocate
 * nothing per call (matmul_h100_optimal.cu:32-59); mi_gemm_epilogue_ws gives a caller the
 * same property: it owns the workspace, per stream or per graph, and the library allocates
 * nothing. */

/* Makes sure the library holds at least `bytes` of workspace for `stream` on the current
 * device (allocating or growing now, at a time the caller chooses, instead of inside a later
 * GEMM call).  MI_ERR_UNSUPPORTED when the stream is being captured.  The reference's launcher
 * holds no per-call device memory (matmul_h100_optimal.cu:32-59); no counterpart there. */
int mi_gemm_reserve_workspace(void* stream, size_t bytes);

/* Gives the library's workspace buffers of `stream` on the current device back (the live one
 * and the ones it outgrew), after hipStreamSynchronize(stream); NULL: the buffers of every
 * stream of the current device, after hipDeviceSynchronize.  Graphs captured from split-K
 * launches through the library on that stream must not be replayed afterwards.  Call it
 * before destroying a stream that ran GEMMs: the table is keyed on the stream handle, and a
 * later stream that gets the same handle value would otherwise inherit the buffer.  The
 * reference's launcher holds no per-call device memory (matmul_h100_optimal.cu:32-59). */
int mi_gemm_release_workspace(void* stream);

/* Bytes of workspace the library currently holds for the streams of the current device (live
 * buffers; 0 after mi_gemm_release_workspace(NULL)). */
size_t mi_gemm_library_workspace_bytes(void);

/* Bytes of workspace the library's choice of kernel wants for this call (0 when the shape
 * does not run split-K).  An upper bound: the largest need over the pointer alignments a
 * launch can meet and over the two parts of a shape whose rows the automatic choice cuts
 * (2248 x 8192 x 28672: 140.5 MiB for the uncut split of an unaligned call, 25 MiB for the
 * aligned call, which is cut at 2048 rows). */
size_t mi_gemm_workspace_bytes(int config, int dtype, int M, int N, int K, int c_layout);

/* mi_gemm_epilogue with a caller-owned workspace: `ws` is a device pointer, 16-byte aligned,
 * of `ws_bytes` bytes, used only by this launch (and its successors on the same stream).
 * Never allocates or frees.  When `ws` is NULL or smaller than the split-K choice needs, the
 * launch runs unsplit (same tolerance, a different summation order, slower for the shapes
 * named above).  Takes the place of the same reference launchers as mi_gemm_epilogue. */
int mi_gemm_epilogue_ws(int config, int dtype, int M, int N, int K, const void* A, const void* B,
                        void* C, float alpha, float beta, int c_layout, void* ws, size_t ws_bytes,
                        void* stream);

/* mi_gemm_bf16 for callers that cannot allocate device memory at all and have no workspace
 * to pass (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Split-K partial sums go to a file-scope
 * device array inside the library, MI_GEMM_NOALLOC_SCRATCH_BYTES per GPU, held from the
 * moment the library is loaded until the process ends; the call makes no hipMalloc, hipFree
 * or other allocating call.  A shape whose partial sums do not fit (pieces x M x N floats,
 * see mi_gemm_workspace_bytes) is refused with MI_ERR_UNSUPPORTED.  Every call on a GPU
 * shares that GPU's array: calls that run split-K and overlap on one GPU (two streams, or a
 * graph replay next to eager calls) race on it -- keep them on one stream.  Nothing in the
 * array needs clearing between calls: the kernels write every partial sum they later read.
 * A shape whose rows the automatic choice cuts in two is refused as a whole, before anything
 * is launched, when either part's partial sums do not fit.  Results are bit-identical to
 * mi_gemm_bf16 for the same arguments wherever mi_gemm_bf16 runs the same split (it runs
 * unsplit, a different summation order, on a capturing stream without a buffer). */
#define MI_GEMM_NOALLOC_SCRATCH_BYTES ((size_t)32 << 20)
int mi_gemm_bf16_noalloc(int M, int N, int K, const uint16_t* A, const uint16_t* B, uint16_t* C,
                         void* stream);

/* Plain, order-preserving GPU GEMM used as golden by the harness: one fp32 accumulator per
 * element fed in ascending k, C = (CType)(acc * alpha + beta), beta a scalar.
 * Replaces  reference_gpu_gemm(GemmParams)  (reference.h:78-90), which the reference's
 * harness compares its kernel with (matmul_h100.cu.jinja:1043-1047). */
int mi_reference_gpu_gemm(int dtype, int M, int N, int K, const void* A, const void* B, void* C,
                          float alpha, float beta, void* stream);

/* Kernel configuration table (what the tuner sweeps; replaces the six template constants
 * of matmul_h100.cu.jinja:9-14). */
int mi_gemm_num_configs(void);
/* Human-readable name, e.g. "m256x256_w2x2_g4_b3" (16x16x32-MFMA kernel, the default),
 * "t128x128_w2x2_s1_g8_o2_d1_e1" (32x32x16-MFMA kernel), "r256x256_w2x2_n4_g8" (LDS-ring
 * kernel), "s16x32_n3" / "d128x128_n3" (single-pass / split-K decode kernels), "k64x64_n2" /
 * "k96x96_s4" (small tiles for outputs of few tiles: K split over the waves of a workgroup /
 * the waves sharing one ring of LDS stages); NULL if out of range. */
const char* mi_gemm_config_name(int config);
/* Index of the config with that name, or -1. */
int mi_gemm_find_config(const char* name);
/* The config MI_CONFIG_AUTO resolves to for this shape; -1 for a shape no launch accepts
 * (an extent <= 0, or a matrix of more than 2^31-1 elements). */
int mi_gemm_select_config(int dtype, int M, int N, int K);
/* Rows that MI_CONFIG_AUTO runs as a GEMM of their own ahead of the rest of the shape, or 0 (the
 * usual case: one GEMM).  A large shape whose last row of tiles is nearly empty (7000^3 on
 * 256x256 tiles: three rounds of workgroups and a sixteenth) is cut behind its last full row of
 * tiles when the library's time model prices the two parts 5 % below the whole; the parts run
 * back to back on the caller's stream, the same answers either way.  mi_gemm_select_config
 * names the configuration the uncut shape would run.  Assumes 16-byte aligned pointers.  The
 * reference, whose kernels take multiples of their tile only (matmul_utils.cuh:362), has no
 * counterpart. */
int mi_gemm_row_cut(int dtype, int M, int N, int K);
/* Number of `M N K config-name` lines loaded from the file named by the environment variable
 * MI_GEMM_TUNED_FILE (read once, on first use; 0 without it).  MI_CONFIG_AUTO takes a listed
 * shape's configuration instead of asking the time model -- the run-time counterpart of the
 * tuner's persisted results (gemm_tuner.py:135-164), keyed on all of M, N, K. */
int mi_gemm_tuned_entries(void);
/* 1 if `config` can run this shape (alignment / divisibility rules of that kernel). */
int mi_gemm_config_supports(int config, int dtype, int M, int N, int K);
/* Workgroups and static LDS bytes the config launches for this shape (0 if unsupported). */
int mi_gemm_config_grid(int config, int M, int N, int K);
int mi_gemm_config_lds_bytes(int config);

/* Number of `int` words a DB trace buffer must hold for this shape so that the kernel's
 * per-workgroup records plus the terminating sentinel fit (the harness of
 * matmul_h100_optimal.cu:132-139 allocates 8192*128 ints).  Every kernel family writes the
 * records -- six ints per workgroup, {cycles waiting for loads, waits, cycles to the end of the
 * K loop, K units, cycles of the stores, 1}, in the format matmul_h100_optimal.cu:182-198
 * parses -- so a trace buffer never changes which kernel MI_CONFIG_AUTO runs: a split-K launch
 * writes one record per (tile, piece), workgroup (x, y) at record y * gridDim.x + x, and a shape
 * that runs as two GEMMs (mi_gemm_row_cut) writes the first part's records, then the second's. */
size_t mi_gemm_trace_words(int M, int N, int K);

/* ---- thin HIP layer used by the C++ harness ------------------------------------------
 * These stand where the reference's harness calls the CUDA runtime directly
 * (common.h:309-365 alloc/copy/free, common.h:246-273 GPUTimer, common.h:43-60
 * get_sm_count, matmul_h100_optimal.cu:120-122,203-210 events). */
int mi_malloc(void** dptr, size_t bytes);
int mi_free(void* dptr);
int mi_memcpy_h2d(void* dst, const void* src, size_t bytes);
int mi_memcpy_d2h(void* dst, const void* src, size_t bytes);
int mi_memcpy_d2d(void* dst, const void* src, size_t bytes);
int mi_memset(void* dst, int value, size_t bytes);
int mi_device_sync(void);
int mi_stream_sync(void* stream);
int mi_event_create(void** ev);
int mi_event_destroy(void* ev);
int mi_event_record(void* ev, void* stream);
int mi_event_sync(void* ev);
int mi_event_elapsed_ms(float* ms, void* start, void* stop);

typedef struct mi_device_props {
    char name[256];
    char arch[64];
    int compute_units;       /* what get_sm_count() returns on the reference side */
    int clock_khz;           /* peak engine clock */
    int mem_clock_khz;
    int mem_bus_bits;
    int lds_bytes_per_block; /* max LDS one workgroup may use */
    int l2_bytes;
    int wavefront;
    size_t hbm_bytes;
} mi_device_props;
int mi_get_device_props(mi_device_props* out);

/* Message of the last failure on this thread ("" if none). */
const char* mi_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* MI_GEMM_H */
