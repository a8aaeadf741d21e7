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
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "../../include/mi_gemm.h"
#include "gemm_kernel.hpp"
#include "splitk_common.hpp"   // splitk_reduce_kernel
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

// Preconditions of the decode (split-K streaming) kernels: whole 16-byte chunks and whole
// 64-deep K slabs, 8-byte aligned C rows.
bool shape_is_streamable(int M, int N, int K, const void* A, const void* B, const void* C) {
    (void)M;   // each decode kernel checks M against its own BM
    return N % 4 == 0 && K % 64 == 0 && aligned16(A) && aligned16(B) &&
           (((uintptr_t)C & 7u) == 0);
}
// The small-tile kernels take any M, N and K and store a C of any alignment: A and B on 4-byte
// boundaries are all they need.
bool shape_has_word_rows(int K, const void* A, const void* B) {
    (void)K;
    return (((uintptr_t)A | (uintptr_t)B) & 3u) == 0;
}

// Split-K geometry for a decode launch.  The decode kernel is bound by what one CU can pull
// from HBM (~26 GB/s, whatever it keeps in flight), so it wants a workgroup on every CU: as
// many pieces as fit into one round of the chip (128 x 8192 x 8192: 2 / 3 / 4 pieces 53 / 39.6 /
// 35.5 us), each at least four 64-deep slabs.  Pieces are contiguous ranges of whole slabs;
// the count is re-derived from the rounded-up piece length so that no piece is empty.
// MI_GEMM_SPLITK=<n> overrides (tuning aid).
int choose_splits(int tiles_n, int K, int cus) {
    static const int env = [] { const char* s = getenv("MI_GEMM_SPLITK"); return s ? atoi(s) : 0; }();
    const int slabs = K / 64;
    int splits = env > 0 ? env : cus / tiles_n;
    if (splits > slabs / 4) splits = slabs / 4;
    if (splits < 1) splits = 1;
    if (splits > 64) splits = 64;
    const int per = (slabs + splits - 1) / splits;
    return (slabs + per - 1) / per;
}
bool is_split_k_decode(int kind) { return kind == mi::KIND_DECODE; }

// Split-K for the tiled 16x16x32 kernel: when a shape has so few tiles that most CUs would
// idle (small M x N, long K), the K range is cut into pieces of whole 128-deep steps, one
// workgroup per (tile, piece); fp32 partials go to the workspace and splitk_reduce_kernel
// adds them in order.  The piece count comes from the time model of the kernel table
// (best_splits); the reduction's vector accesses need N % 4 == 0 and an 8-byte aligned C.
// (A trace buffer changes nothing: every workgroup of a split launch writes its record.)
// MI_GEMM_TILE_SPLITK=<n> forces a piece count (1 = never split; tuning aid).
bool shape_is_splittable(int N, const void* C) {
    return N % 4 == 0 && ((uintptr_t)C & 7u) == 0;
}

int choose_tile_splits(const mi::KernelEntry& e, int M, int N, int K, bool splittable, bool ptr_aligned, int cus,
                       int* k_per_split) {
    *k_per_split = K;
    static const int env = [] { const char* s = getenv("MI_GEMM_TILE_SPLITK"); return s ? atoi(s) : 0; }();
    if (!splittable || e.kind != mi::KIND_MFMA16 || e.kg > 1 || env == 1) return 1;   // (K groups split K inside the workgroup)
    if (env > 1) {
        int s = env < K / 512 ? env : K / 512;
        if (s < 2 || (long long)((M + e.BM - 1) / e.BM) * ((N + e.BN - 1) / e.BN) * 256 * 256 * 4 >= 0x7fffffffLL) return 1;
        const int kps = ((K + s - 1) / s + 127) / 128 * 128;
        s = (K + kps - 1) / kps;
        if (s < 2) return 1;
        *k_per_split = kps;
        return s;
    }
    return mi::best_splits(e, M, N, K, true, ptr_aligned, cus, k_per_split, nullptr);
}

// Split-K for the small-tile kernels: an output of a few tiles with a very long K (128 x 384 x
// 13376: 48 tiles of 32x32) leaves most CUs idle however small the tile, so K is cut into pieces
// of whole 64-deep units, one workgroup per (tile, piece), as above.  The piece count comes from
// the kernels' time model (best_wavek_splits).  MI_GEMM_SMALL_SPLITK=<n> forces a piece count
// (1 = never split; tuning aid).
int choose_small_tile_splits(const mi::KernelEntry& e, int M, int N, int K, bool splittable, int cus, int* k_per_split) {
    *k_per_split = K;
    static const int env = [] { const char* s = getenv("MI_GEMM_SMALL_SPLITK"); return s ? atoi(s) : 0; }();
    if (!splittable || e.kind != mi::KIND_WAVEK || env == 1) return 1;
    if (env > 1) {
        int s = env < K / 128 ? env : K / 128;
        if (s < 2 || (long long)s * M * N * 4 >= 0x7fffffffLL) return 1;
        const int kps = ((K + s - 1) / s + 63) / 64 * 64;
        s = (K + kps - 1) / kps;
        if (s < 2) return 1;
        *k_per_split = kps;
        return s;
    }
    return mi::best_wavek_splits(e, M, N, K, true, cus, k_per_split, nullptr);
}

// ---- where the split-K kernels put their fp32 partial sums ----------------------------
// Three sources, chosen by the entry point:
//  * LIBRARY (mi_gemm_bf16 / _ex / _epilogue): one buffer per (device, stream), allocated on
//    first use and replaced by a larger one on demand.  Launches already enqueued and captured
//    graphs keep a buffer's address, so a replaced buffer moves to the stream's retired list
//    (sizes are powers of two, so the retired ones together stay below the live one) and
//    nothing is freed behind the caller's back: mi_gemm_release_workspace frees a stream's
//    buffers (after synchronising it), and the table holds at most kMaxStreamWs streams per
//    device -- a further stream takes over an entry once the device is idle.  Launches on one
//    stream are ordered and launches on different streams use different buffers, so
//    concurrent split-K calls do not meet.  A stream that is being captured cannot allocate:
//    if it has no buffer that is large enough yet, the launch runs unsplit instead.
//  * CALLER (mi_gemm_epilogue_ws): the caller's buffer, nothing is allocated; too small (or
//    NULL) means the launch runs unsplit.
//  * STATIC (mi_gemm_bf16_noalloc): the file-scope device array below, one copy per GPU the
//    library runs on, of a fixed size; a shape whose partials do not fit is refused.
// The kernels overwrite every partial they later read ([piece][M][N], all of it), so no
// buffer needs clearing between calls.
constexpr int kMaxDevices = 64;
constexpr size_t kScratchBytes = MI_GEMM_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

enum WsMode { WS_LIBRARY, WS_CALLER, WS_STATIC };
struct WsSource {
    WsMode mode = WS_LIBRARY;
    void* ptr = nullptr;      // WS_CALLER: the caller's buffer
    size_t bytes = 0;
};
struct StreamWs {
    hipStream_t stream;
    float* ptr;
    size_t bytes;
    std::vector<void*> retired;      // buffers this stream outgrew: an enqueued launch or a captured graph may still
                                     // hold their address, so they live until the stream's workspace is released
};
struct DeviceState {
    std::vector<StreamWs> ws;        // one entry per stream that ran a split-K launch (at most kMaxStreamWs)
    unsigned char* scratch = nullptr;   // device address of `scratch` on this device
    int cus = 0;
};
// Streams with a buffer of their own per device.  A process that keeps creating streams does not
// grow the table beyond this: the next new stream waits for the device to go idle and takes over
// an entry (see acquire_workspace), so at most this many live buffers exist per device.
constexpr size_t kMaxStreamWs = 16;
std::mutex g_ws_mutex;
DeviceState g_dev[kMaxDevices];

DeviceState& device_state() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    return g_dev[dev];
}

// Device address of the static scratch array on the current device.  In host code the
// array's name is only a handle for the runtime: the address a kernel can use comes from
// hipGetSymbolAddress, once per device (each GPU holds its own copy at its own address).
hipError_t static_scratch(unsigned char** out) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    DeviceState& st = device_state();
    if (!st.scratch) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        st.scratch = (unsigned char*)p;
    }
    *out = st.scratch;
    return hipSuccess;
}

void free_entry(StreamWs& w) {
    if (w.ptr) (void)hipFree(w.ptr);
    for (void* r : w.retired) (void)hipFree(r);
    w.ptr = nullptr;
    w.bytes = 0;
    w.retired.clear();
}

// 0: *out holds `bytes` of workspace; 1: none to be had without allocating where that is not
// possible (the caller runs the launch unsplit); < 0: MI_ERR_* with the message set.
int acquire_workspace(const WsSource& src, size_t bytes, hipStream_t stream, float** out) {
    *out = nullptr;
    if (src.mode == WS_CALLER) {
        if (!src.ptr || src.bytes < bytes) return 1;
        *out = (float*)src.ptr;
        return 0;
    }
    if (src.mode == WS_STATIC) {
        if (bytes > kScratchBytes)
            return fail(MI_ERR_UNSUPPORTED,
                        "this shape's split-K partial sums need %zu bytes, the static scratch array holds %zu",
                        bytes, kScratchBytes);
        unsigned char* p = nullptr;
        hipError_t e = static_scratch(&p);
        if (e != hipSuccess)
            return fail(MI_ERR_HIP, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
        *out = (float*)p;
        return 0;
    }
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    DeviceState& st = device_state();
    StreamWs* mine = nullptr;
    for (StreamWs& w : st.ws)
        if (w.stream == stream) mine = &w;
    if (mine && mine->bytes >= bytes) {
        *out = mine->ptr;
        return 0;
    }
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        return 1;      // e.g. the null stream while another stream captures: do not allocate
    }
    if (cap != hipStreamCaptureStatusNone) return 1;
    size_t want = (size_t)4 << 20;
    while (want < bytes) want <<= 1;
    if (!mine && st.ws.size() >= kMaxStreamWs) {
        // The table is full (a process that keeps making streams, or never releases): once the
        // device is idle no launch holds any buffer, so the smallest entry changes hands -- its
        // buffer as it is when large enough, else freed here and replaced below.
        hipError_t e = hipDeviceSynchronize();
        if (e != hipSuccess)
            return fail(MI_ERR_HIP, "hipDeviceSynchronize before reusing a split-K workspace failed: %s", hipGetErrorString(e));
        StreamWs* take = nullptr;
        for (StreamWs& w : st.ws)       // the smallest entry that is already large enough ...
            if (w.bytes >= bytes && (!take || w.bytes < take->bytes)) take = &w;
        if (!take)
            for (StreamWs& w : st.ws)   // ... else the smallest of all
                if (!take || w.bytes < take->bytes) take = &w;
        for (void* r : take->retired) (void)hipFree(r);
        take->retired.clear();
        take->stream = stream;
        if (take->bytes >= bytes) {
            *out = take->ptr;
            return 0;
        }
        if (take->ptr) (void)hipFree(take->ptr);
        take->ptr = nullptr;
        take->bytes = 0;
        mine = take;
    }
    float* p = nullptr;
    hipError_t e = hipMalloc((void**)&p, want);
    if (e != hipSuccess)
        return fail(MI_ERR_HIP, "split-K workspace allocation of %zu bytes failed: %s", want, hipGetErrorString(e));
    if (mine) {
        if (mine->ptr) mine->retired.push_back(mine->ptr);
        mine->ptr = p;
        mine->bytes = want;
    } else {
        st.ws.push_back({stream, p, want, {}});
    }
    *out = p;
    return 0;
}

int compute_units() {
    DeviceState& st = device_state();
    if (st.cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            st.cus = n;
        else
            st.cus = 256;
    }
    return st.cus;
}

// The aligned kernels assume full tiles, K a multiple of two K steps, 16-byte aligned
// rows of A and B and 8-byte aligned rows of C; everything else takes the predicated twin.
bool shape_is_aligned(const mi::KernelEntry& e, int M, int N, int K, const void* A,
                      const void* B, const void* C) {
    return M % e.BM == 0 && N % e.BN == 0 && K % 128 == 0 && aligned16(A) && aligned16(B) &&
           aligned16(C);
}

// Shapes a launch accepts: positive extents, `int` element indices as in the reference
// (reference.h:30,40 index with int) and 32-bit byte offsets inside one tile's row panel.
bool shape_in_range(int M, int N, int K) {
    return M > 0 && N > 0 && K > 0 && (long long)M * K <= 0x7fffffffLL && (long long)N * K <= 0x7fffffffLL &&
           (long long)M * N <= 0x7fffffffLL && (long long)K * 2 * 256 <= 0x7fffffffLL;
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

// Tuned shapes from a file: MI_GEMM_TUNED_FILE names a text file with one `M N K config-name`
// per line (# starts a comment), read once, on first use.  A shape listed there skips the
// time model when its configuration can run the call (the decode kernels have preconditions);
// lines that do not parse or name no compiled configuration are ignored.  Keyed on all of
// M, N and K (the reference keys its cached descriptors on M alone, matmul_utils.cuh:49-51).
struct TunedEntry {
    int M, N, K, config;
};
const std::vector<TunedEntry>& tuned_entries() {
    static const std::vector<TunedEntry> table = [] {
        std::vector<TunedEntry> t;
        const char* path = getenv("MI_GEMM_TUNED_FILE");
        FILE* f = path && *path ? fopen(path, "r") : nullptr;
        if (!f) return t;
        char line[256];
        while (fgets(line, sizeof(line), f)) {
            if (char* hash = strchr(line, '#')) *hash = 0;
            int M = 0, N = 0, K = 0;
            char name[128];
            if (sscanf(line, "%d %d %d %127s", &M, &N, &K, name) != 4 || M <= 0 || N <= 0 || K <= 0) continue;
            for (int i = 0; i < mi::kNumKernels; ++i)
                if (strcmp(name, mi::kKernels[i].name) == 0) {
                    t.push_back({M, N, K, i});
                    break;
                }
        }
        fclose(f);
        return t;
    }();
    return table;
}
// config for (M, N, K) from the tuned file, or -1
int tuned_config(int M, int N, int K, bool streamable, bool small_ok) {
    for (const TunedEntry& t : tuned_entries()) {
        if (t.M != M || t.N != N || t.K != K) continue;
        const mi::KernelEntry& e = mi::kKernels[t.config];
        if ((is_split_k_decode(e.kind) || e.kind == mi::KIND_STREAM) && (!streamable || M > e.BM)) continue;
        if (e.kind == mi::KIND_WAVEK && !small_ok) continue;
        if (e.kg > 1 && K % (128 * e.kg) != 0) continue;      // (the rule mi_gemm_config_supports applies)
        return t.config;
    }
    return -1;
}

// The automatic choice is a pure function of the shape and three flags and costs 1-3 us of
// host time (the time model runs over every candidate and piece count), which shows when
// small GEMMs are launched back to back: the last few answers are kept per thread, keyed on
// all of its inputs.  (No pointer or other per-call state is cached.)
struct Choice {
    int M, N, K, flags, requested, cus;   // key; requested = the caller's config (MI_CONFIG_AUTO or an index)
    int config, splits, k_per_split;
};
Choice compute_choice(int requested, int M, int N, int K, bool streamable, bool splittable, bool ptr_aligned,
                      bool small_ok) {
    const int flags = (streamable ? 1 : 0) | (splittable ? 2 : 0) | (ptr_aligned ? 4 : 0) | (small_ok ? 8 : 0);
    const int cus = compute_units();
    Choice c{M, N, K, flags, requested, cus, requested, 1, K};
    if (requested == MI_CONFIG_AUTO) {
        c.config = tuned_config(M, N, K, streamable, small_ok);
        if (c.config < 0) c.config = mi::select_kernel(M, N, K, streamable, splittable, ptr_aligned, small_ok, cus);
    }
    const mi::KernelEntry& e = mi::kKernels[c.config];
    if (e.kind == mi::KIND_MFMA16) {
        c.splits = choose_tile_splits(e, M, N, K, splittable, ptr_aligned, cus, &c.k_per_split);
    } else if (is_split_k_decode(e.kind) && streamable && M <= e.BM) {
        const int tiles_n = (N + e.BN - 1) / e.BN;
        c.splits = choose_splits(tiles_n, K, cus);   // no empty split
        c.k_per_split = ((K / 64 + c.splits - 1) / c.splits) * 64;
    } else if (e.kind == mi::KIND_WAVEK) {
        c.splits = choose_small_tile_splits(e, M, N, K, splittable, cus, &c.k_per_split);
    }
    return c;
}
Choice choose(int requested, int M, int N, int K, bool streamable, bool splittable, bool ptr_aligned, bool small_ok) {
    static thread_local Choice memo[4] = {};
    static thread_local int next = 0;
    const int flags = (streamable ? 1 : 0) | (splittable ? 2 : 0) | (ptr_aligned ? 4 : 0) | (small_ok ? 8 : 0);
    const int cus = compute_units();
    for (const Choice& c : memo)
        if (c.M == M && c.N == N && c.K == K && c.flags == flags && c.requested == requested && c.cus == cus &&
            c.splits > 0)
            return c;
    const Choice c = compute_choice(requested, M, N, K, streamable, splittable, ptr_aligned, small_ok);
    memo[next] = c;
    next = (next + 1) & 3;
    return c;
}

// The cut of a large ragged shape into two GEMMs is a pure function of the shape and four flags
// like the kernel choice, and costs several passes of the time model: the last answer is kept per
// thread.  MI_GEMM_ROW_CUT=0 switches the cut off (measurement aid).
int rows_to_cut(int M, int N, int K, bool streamable, bool splittable, bool ptr_aligned, bool small_ok) {
    static const int env = [] { const char* s = getenv("MI_GEMM_ROW_CUT"); return s ? atoi(s) : 1; }();
    if (env == 0 || (long long)M * N < 4096LL * 4096LL) return 0;
    struct Memo { int M, N, K, flags, cus, m1; };
    static thread_local Memo memo = {0, 0, 0, -1, 0, 0};
    const int flags = (streamable ? 1 : 0) | (splittable ? 2 : 0) | (ptr_aligned ? 4 : 0) | (small_ok ? 8 : 0);
    const int cus = compute_units();
    if (memo.M != M || memo.N != N || memo.K != K || memo.flags != flags || memo.cus != cus)
        memo = {M, N, K, flags, cus, mi::rows_to_split_off(M, N, K, streamable, splittable, ptr_aligned, small_ok, cus)};
    return memo.m1;
}

// Workgroups the main kernel of a launch has (the grid a trace buffer's records are indexed by).
size_t launch_workgroups(const mi::KernelEntry& e, int M, int N, int splits) {
    const size_t tiles_n = (size_t)(N + e.BN - 1) / e.BN;
    if (e.kind == mi::KIND_STREAM || is_split_k_decode(e.kind)) return tiles_n * (size_t)splits;
    return (size_t)((M + e.BM - 1) / e.BM) * tiles_n * (size_t)splits;
}

// One GEMM launch (two for split-K): argument checks, kernel choice, aligned / predicated twin.
// `may_cut`: the automatic choice may run the shape as two GEMMs, the first rows and the rest
// (rows_to_split_off in the kernel table); the parts themselves are not cut again.
int run_gemm(int config, int dtype, int M, int N, int K, const void* A, const void* B, void* C,
             int* DB, float alpha, float beta, void* stream, const WsSource& wsrc = WsSource{}, bool may_cut = true) {
    int rc = check_args(config, dtype, M, N, K, A, B, C);
    if (rc != MI_OK) return rc;
    const bool streamable = shape_is_streamable(M, N, K, A, B, C);
    if (may_cut && config == MI_CONFIG_AUTO &&
        tuned_config(M, N, K, streamable, shape_has_word_rows(K, A, B)) < 0) {       // (a tuned shape runs as tuned)
        const int m1 = rows_to_cut(M, N, K, streamable, shape_is_splittable(N, C),
                                   aligned16(A) && aligned16(B) && aligned16(C), shape_has_word_rows(K, A, B));
        if (m1 > 0) {
            // Both parts' workspace is settled before anything is launched: a part that could not
            // get its partial sums' room (the static array too small, an allocation that fails)
            // must not leave the other part's rows of C written and the call failed.
            const void* A2 = (const unsigned char*)A + (size_t)m1 * K * 2;
            void* C2 = (unsigned char*)C + (size_t)m1 * N * 2;
            size_t need = 0;
            size_t wgs_first = 0;            // workgroups of the first part: the second part's trace records follow theirs
            for (int part = 0; part < 2; ++part) {
                const int Mp = part ? M - m1 : m1;
                const void* Ap = part ? A2 : A;
                const void* Cp = part ? C2 : C;
                const Choice c = choose(config, Mp, N, K, shape_is_streamable(Mp, N, K, Ap, B, Cp), shape_is_splittable(N, Cp),
                                        aligned16(Ap) && aligned16(B) && aligned16(Cp), shape_has_word_rows(K, Ap, B));
                const size_t b = c.splits > 1 ? (size_t)c.splits * Mp * N * sizeof(float) : 0;
                if (b > need) need = b;
                if (part == 0) wgs_first = launch_workgroups(mi::kKernels[c.config], Mp, N, c.splits);
            }
            if (need > 0) {
                float* unused = nullptr;
                const int wrc = acquire_workspace(wsrc, need, (hipStream_t)stream, &unused);
                if (wrc < 0) return wrc;
            }
            rc = run_gemm(config, dtype, m1, N, K, A, B, C, DB, alpha, beta, stream, wsrc, false);
            if (rc != MI_OK) return rc;
            return run_gemm(config, dtype, M - m1, N, K, A2, B, C2, DB ? DB + 6 * wgs_first : nullptr, alpha, beta, stream,
                            wsrc, false);
        }
    }
    // (a trace buffer does not change the choice: every kernel family writes the records)
    const Choice choice = choose(config, M, N, K, streamable, shape_is_splittable(N, C),
                                 aligned16(A) && aligned16(B) && aligned16(C), shape_has_word_rows(K, A, B));
    config = choice.config;
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
    args.ws = nullptr;
    args.splits = 1;
    args.k_per_split = K;
    args.alpha = alpha;
    args.beta = beta;

    if (e.kind == mi::KIND_STREAM) {
        if (!streamable || M > e.BM)
            return fail(MI_ERR_UNSUPPORTED,
                        "config %s needs M <= %d, N %% 4 == 0, K %% 64 == 0 and 16-byte aligned operands",
                        e.name, e.BM);
        hipError_t err = e.launch[dtype][0](args, (hipStream_t)stream);
        if (err != hipSuccess)
            return fail(MI_ERR_HIP, "launch of %s failed: %s", e.name, hipGetErrorString(err));
        return MI_OK;
    }
    if (e.kind == mi::KIND_WAVEK) {
        if (!shape_has_word_rows(K, A, B))
            return fail(MI_ERR_UNSUPPORTED, "config %s needs 4-byte aligned A and B", e.name);
        args.splits = choice.splits;
        args.k_per_split = choice.k_per_split;
        if (args.splits > 1) {
            const int wrc = acquire_workspace(wsrc, (size_t)args.splits * M * N * sizeof(float), (hipStream_t)stream, &args.ws);
            if (wrc < 0) return wrc;
            if (wrc > 0) {           // no workspace to be had: every tile walks all of K
                args.splits = 1;
                args.k_per_split = K;
            }
        }
        hipError_t err = e.launch[dtype][0](args, (hipStream_t)stream);
        if (err != hipSuccess)
            return fail(MI_ERR_HIP, "launch of %s failed: %s", e.name, hipGetErrorString(err));
        return MI_OK;
    }
    if (is_split_k_decode(e.kind)) {
        if (!streamable || M > e.BM)
            return fail(MI_ERR_UNSUPPORTED,
                        "config %s needs M <= %d, N %% 4 == 0, K %% 64 == 0 and 16-byte aligned operands",
                        e.name, e.BM);
        args.splits = choice.splits;
        args.k_per_split = choice.k_per_split;
        if (args.splits > 1) {
            const int wrc = acquire_workspace(wsrc, (size_t)args.splits * M * N * sizeof(float), (hipStream_t)stream, &args.ws);
            if (wrc < 0) return wrc;
            if (wrc > 0) {           // no workspace to be had: one pass over all of K
                args.splits = 1;
                args.k_per_split = K;
            }
        }
        hipError_t err = e.launch[dtype][0](args, (hipStream_t)stream);
        if (err != hipSuccess)
            return fail(MI_ERR_HIP, "launch of %s failed: %s", e.name, hipGetErrorString(err));
        return MI_OK;
    }

    if (e.kg > 1 && K % (128 * e.kg) != 0)
        return fail(MI_ERR_UNSUPPORTED, "config %s splits K over %d groups of waves and needs K %% %d == 0", e.name,
                    e.kg, 128 * e.kg);
    const bool edge = !shape_is_aligned(e, M, N, K, A, B, C);
    mi::LaunchFn fn = e.launch[dtype][edge ? 1 : 0];
    if (!fn) return fail(MI_ERR_UNSUPPORTED, "config %s has no %s kernel for dtype %d", e.name,
                         edge ? "predicated" : "aligned", dtype);
    if (e.kind == mi::KIND_MFMA16) {
        args.splits = choice.splits;
        args.k_per_split = choice.k_per_split;
        if (args.splits > 1) {
            const int wrc = acquire_workspace(wsrc, (size_t)args.splits * M * N * sizeof(float), (hipStream_t)stream, &args.ws);
            if (wrc < 0) return wrc;
            if (wrc > 0) {
                args.splits = 1;
                args.k_per_split = K;
            }
        }
    }
    hipError_t err = fn(args, (hipStream_t)stream);
    if (err != hipSuccess)
        return fail(MI_ERR_HIP, "launch of %s failed: %s", e.name, hipGetErrorString(err));
    if (args.splits > 1) {
        const size_t quads = ((size_t)M * N + 3) / 4;
        const dim3 rgrid((unsigned)((quads + 255) / 256));
        err = dtype == MI_DTYPE_BF16
                  ? mi::launch_kernel(mi::splitk_reduce_kernel<mi::DT_BF16>, rgrid, dim3(256), (hipStream_t)stream,
                                      args.ws, C, M, N, N, args.splits, alpha, beta)
                  : mi::launch_kernel(mi::splitk_reduce_kernel<mi::DT_FP16>, rgrid, dim3(256), (hipStream_t)stream,
                                      args.ws, C, M, N, N, args.splits, alpha, beta);
        if (err != hipSuccess)
            return fail(MI_ERR_HIP, "launch of the split-K reduction failed: %s", hipGetErrorString(err));
    }
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
    if (!shape_in_range(M, N, K)) return 0;
    const mi::KernelEntry& e = mi::kKernels[config];
    if (is_split_k_decode(e.kind) || e.kind == mi::KIND_STREAM)
        return M <= e.BM && N % 4 == 0 && K % 64 == 0;
    if (e.kind == mi::KIND_WAVEK) return 1;
    if (e.kg > 1 && K % (128 * e.kg) != 0) return 0;
    return e.launch[dtype][1] != nullptr;
}

int mi_gemm_config_grid(int config, int M, int N, int K) {
    if (config < 0 || config >= mi::kNumKernels || !shape_in_range(M, N, K)) return 0;
    const mi::KernelEntry& e = mi::kKernels[config];
    if (e.kind == mi::KIND_STREAM) return M > e.BM || K % 64 != 0 ? 0 : (N + e.BN - 1) / e.BN;
    if (is_split_k_decode(e.kind)) {
        if (M > e.BM || K % 64 != 0) return 0;
        const int tiles_n = (N + e.BN - 1) / e.BN;
        return tiles_n * choose_splits(tiles_n, K, compute_units());
    }
    const int tiles = ((M + e.BM - 1) / e.BM) * ((N + e.BN - 1) / e.BN);
    if (e.kind == mi::KIND_WAVEK) {    // split-K pieces, assuming an aligned C and no trace buffer
        int kps = K;
        return tiles * choose_small_tile_splits(e, M, N, K, N % 4 == 0, compute_units(), &kps);
    }
    if (e.kind == mi::KIND_MFMA16) {   // split-K pieces, assuming an aligned C and no trace buffer
        int kps = K;
        return tiles * choose_tile_splits(e, M, N, K, N % 4 == 0, true, compute_units(), &kps);
    }
    return tiles;
}

int mi_gemm_select_config(int dtype, int M, int N, int K) {
    (void)dtype;
    if (!shape_in_range(M, N, K)) return -1;
    // pointer alignment is unknown here: assume the usual 256-byte aligned allocations
    const bool streamable = N % 4 == 0 && K % 64 == 0;
    const int tuned = tuned_config(M, N, K, streamable, true);
    if (tuned >= 0) return tuned;
    return mi::select_kernel(M, N, K, streamable, N % 4 == 0, true, true, compute_units());
}

int mi_gemm_row_cut(int dtype, int M, int N, int K) {
    (void)dtype;
    if (!shape_in_range(M, N, K)) return 0;
    const bool streamable = N % 4 == 0 && K % 64 == 0;
    if (tuned_config(M, N, K, streamable, true) >= 0) return 0;
    return rows_to_cut(M, N, K, streamable, N % 4 == 0, true, true);
}

int mi_gemm_tuned_entries(void) { return (int)tuned_entries().size(); }

size_t mi_gemm_trace_words(int M, int N, int K) {
    // enough for whichever kernel configuration ends up running the shape -- or its two
    // parts, one after the other, where the automatic choice cuts the shape's rows
    auto largest = [&](int rows) {
        size_t grid = 0;
        for (int c = 0; c < mi::kNumKernels; ++c) {
            const size_t g = (size_t)mi_gemm_config_grid(c, rows, N, K);
            if (g > grid) grid = g;
        }
        return grid;
    };
    size_t grid = largest(M);
    if (shape_in_range(M, N, K))
        for (int flags = 0; flags < 16; ++flags) {
            const int m1 = rows_to_cut(M, N, K, (flags & 1) != 0 && N % 4 == 0 && K % 64 == 0, (flags & 2) != 0 && N % 4 == 0,
                                       (flags & 4) != 0, (flags & 8) != 0);
            if (m1 > 0 && largest(m1) + largest(M - m1) > grid) grid = largest(m1) + largest(M - m1);
        }
    return grid * 6 + 1;
}

int mi_gemm_ex(int config, int dtype, int M, int N, int K, const void* A, const void* B,
               void* C, int* DB, void* stream) {
    return run_gemm(config, dtype, M, N, K, A, B, C, DB, 1.0f, 0.0f, stream);
}

int mi_gemm_epilogue(int config, int dtype, int M, int N, int K, const void* A, const void* B,
                     void* C, float alpha, float beta, int c_layout, void* stream) {
    if (c_layout != MI_C_ROW_MAJOR && c_layout != MI_C_COL_MAJOR)
        return fail(MI_ERR_INVALID, "unknown C layout %d", c_layout);
    if (!(alpha == alpha) || !(beta == beta)) return fail(MI_ERR_INVALID, "alpha or beta is NaN");
    // Column-major C (M x N, element (m, n) at C[n*M + m]) is the row-major N x M matrix
    // C^T = B . A^T: the same GEMM with the operands and their extents exchanged.  Every
    // element is still the k-ordered sum the kernels form for the row-major case.
    if (c_layout == MI_C_COL_MAJOR)
        return run_gemm(config, dtype, N, M, K, B, A, C, nullptr, alpha, beta, stream);
    return run_gemm(config, dtype, M, N, K, A, B, C, nullptr, alpha, beta, stream);
}

int mi_gemm_bf16(int M, int N, int K, const uint16_t* A, const uint16_t* B, uint16_t* C, int* DB,
                 void* stream) {
    return mi_gemm_ex(MI_CONFIG_AUTO, MI_DTYPE_BF16, M, N, K, A, B, C, DB, stream);
}

size_t mi_gemm_workspace_bytes(int config, int dtype, int M, int N, int K, int c_layout) {
    if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16) return 0;
    if (!shape_in_range(M, N, K)) return 0;
    if (config != MI_CONFIG_AUTO && (config < 0 || config >= mi::kNumKernels)) return 0;
    if (c_layout == MI_C_COL_MAJOR) {
        const int t = M;
        M = N;
        N = t;
    }
    // The choice also depends on the alignment of the pointers, unknown here: the largest
    // need over the cases a launch can meet -- and over the two parts, where the automatic
    // choice may cut the shape's rows in two.
    auto uncut = [&](int rows) {
        size_t need = 0;
        const bool can_stream = N % 4 == 0 && K % 64 == 0;
        for (int aligned = 0; aligned < 2; ++aligned)
            for (int streamable = 0; streamable < (can_stream && aligned ? 2 : 1); ++streamable)
                // (a launch that cannot use the small-tile kernels -- operands not 4-byte aligned --
                // may split where one that can does not: both cases)
                for (int small = 0; small < 2; ++small) {
                    const Choice c = compute_choice(config, rows, N, K, streamable != 0, N % 4 == 0, aligned != 0, small != 0);
                    const size_t b = c.splits > 1 ? (size_t)c.splits * rows * N * sizeof(float) : 0;
                    if (b > need) need = b;
                }
        return need;
    };
    size_t need = uncut(M);
    if (config == MI_CONFIG_AUTO && tuned_config(M, N, K, N % 4 == 0 && K % 64 == 0, true) < 0)
        for (int flags = 0; flags < 16; ++flags) {
            const int m1 = rows_to_cut(M, N, K, (flags & 1) != 0 && N % 4 == 0 && K % 64 == 0, (flags & 2) != 0 && N % 4 == 0,
                                       (flags & 4) != 0, (flags & 8) != 0);
            if (m1 > 0) {
                const size_t a = uncut(m1), b = uncut(M - m1);
                if (a > need) need = a;
                if (b > need) need = b;
            }
        }
    return need;
}

int mi_gemm_epilogue_ws(int config, int dtype, int M, int N, int K, const void* A, const void* B, void* C,
                        float alpha, float beta, int c_layout, void* ws, size_t ws_bytes, void* stream) {
    if (c_layout != MI_C_ROW_MAJOR && c_layout != MI_C_COL_MAJOR)
        return fail(MI_ERR_INVALID, "unknown C layout %d", c_layout);
    if (!(alpha == alpha) || !(beta == beta)) return fail(MI_ERR_INVALID, "alpha or beta is NaN");
    if (ws && !aligned16(ws)) return fail(MI_ERR_INVALID, "the workspace must be 16-byte aligned");
    WsSource src;
    src.mode = WS_CALLER;
    src.ptr = ws;
    src.bytes = ws ? ws_bytes : 0;
    if (c_layout == MI_C_COL_MAJOR)
        return run_gemm(config, dtype, N, M, K, B, A, C, nullptr, alpha, beta, stream, src);
    return run_gemm(config, dtype, M, N, K, A, B, C, nullptr, alpha, beta, stream, src);
}

int mi_gemm_bf16_noalloc(int M, int N, int K, const uint16_t* A, const uint16_t* B, uint16_t* C, void* stream) {
    WsSource src;
    src.mode = WS_STATIC;
    return run_gemm(MI_CONFIG_AUTO, MI_DTYPE_BF16, M, N, K, A, B, C, nullptr, 1.0f, 0.0f, stream, src);
}

int mi_gemm_reserve_workspace(void* stream, size_t bytes) {
    if (bytes == 0) return MI_OK;
    float* p = nullptr;
    const int rc = acquire_workspace(WsSource{}, bytes, (hipStream_t)stream, &p);
    if (rc > 0) return fail(MI_ERR_UNSUPPORTED, "the stream is being captured: no workspace can be allocated now");
    return rc < 0 ? rc : MI_OK;
}

int mi_gemm_release_workspace(void* stream) {
    // NULL: every stream's buffers on the current device, once the device is idle
    if (stream == nullptr) MI_HIP(hipDeviceSynchronize());
    else MI_HIP(hipStreamSynchronize((hipStream_t)stream));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    DeviceState& st = device_state();
    for (size_t i = 0; i < st.ws.size();) {
        if (stream == nullptr || st.ws[i].stream == (hipStream_t)stream) {
            free_entry(st.ws[i]);
            st.ws.erase(st.ws.begin() + (long)i);
        } else {
            ++i;
        }
    }
    return MI_OK;
}

size_t mi_gemm_library_workspace_bytes(void) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    size_t total = 0;
    for (const StreamWs& w : device_state().ws) total += w.bytes;
    return total;
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
int mi_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    MI_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
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
