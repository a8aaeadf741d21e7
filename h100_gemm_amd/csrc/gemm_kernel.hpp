// gemm_kernel.hpp -- the gfx950 (MI355X, CDNA4) tile GEMM kernel.
//
//   C[M,N] = A[M,K] . B[N,K]^T     A, B, C row-major 16-bit floats, fp32 accumulate.
//
// This is the device side that stands where the reference project's Hopper kernels
// stand (matmulKernel, matmul_utils.cuh:380-566; gpu_gemm_kernel,
// matmul_h100.cu.jinja:734-925).  None of their mechanisms exist on CDNA4, so each is
// replaced by what the hardware does have:
//
//   TMA bulk copy + 128B swizzle   -> every wave issues coalesced 16-byte buffer loads
//                                     (out-of-range rows read as zero through the buffer
//                                     descriptor) into registers, then ds_write_b128 into
//                                     an XOR-swizzled LDS tile whose 128-byte rows are
//                                     read back conflict-free by ds_read_b128.
//   mbarrier full/empty ring       -> software pipeline: registers hold tile k+2 in
//                                     flight, LDS holds tiles k and k+1, one s_barrier per
//                                     K step, ordering by s_waitcnt.
//   producer / consumer warpgroups -> no specialisation: one wave per SIMD (or two), each
//                                     wave loads, stores to LDS and issues MFMA.
//   setmaxnreg                     -> fixed budget: the fp32 accumulators of a
//                                     (BM/WM)x(BN/WN) wave tile sit in AGPRs, fragments,
//                                     staging registers and addresses in VGPRs.
//   WGMMA m64nNk16                 -> v_mfma_f32_32x32x16_{bf16,f16}, operands from VGPRs.
//   thread-block clusters/multicast-> workgroup ids are re-mapped so that the workgroups
//                                     resident on one XCD (they share that XCD's L2) own a
//                                     compact block of output tiles.
//
// LDS tile layout (one stage, one operand): `rows` x 64 elements, 128 bytes per row, the
// eight 16-byte chunks of a row permuted by  chunk' = chunk ^ swz(row).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include <type_traits>

#include <type_traits>

namespace mi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int DT_BF16 = 0;
constexpr int DT_FP16 = 1;

struct GemmArgs {
    const void* A;
    const void* B;
    void* C;
    int M, N, K;
    int lda, ldb, ldc;       // in elements
    int tiles_m, tiles_n;    // ceil(M/BM), ceil(N/BN)
    int c_vec_ok;            // 1: every C row start is 8-byte aligned (ldc % 4 == 0, base aligned)
    int* DB;                 // optional trace buffer (may be null)
    float* ws;               // split-K workspace (decode kernels only)
    int splits, k_per_split; // split-K geometry (decode kernels only)
    float alpha = 1.0f;      // C = (CType)(acc * alpha + beta), beta a plain scalar added to
    float beta = 0.0f;       // every element (reference.h:40)
};

// Launch `kernel` with the given arguments and return the status of THIS launch.
// (hipLaunchKernelGGL + hipGetLastError would also report -- and clear -- an error that some
// earlier, unrelated call of the process left behind, as a failure of the GEMM.)
template <class... KArgs, class... Args>
inline hipError_t launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t stream, Args... args) {
    // one slot per kernel parameter, converted to the parameter's own type
    std::tuple<std::decay_t<KArgs>...> held{static_cast<std::decay_t<KArgs>>(args)...};
    void* ptrs[sizeof...(KArgs)];
    int n = 0;
    std::apply([&](auto&... a) { ((ptrs[n++] = (void*)&a), ...); }, held);
    return hipLaunchKernel((const void*)kernel, grid, block, ptrs, 0, stream);
}

// Compile-time description of one kernel variant -- the knobs the tuner sweeps.
//   BM x BN      macro tile of one workgroup (K step is 64 elements = one 128-byte LDS row)
//   WM x WN      wave grid inside the workgroup; each wave owns (BM/WM) x (BN/WN)
//   SWZ          LDS chunk swizzle: 0 -> row & 7, 1 -> (row >> 1) & 7
//   GROUP        height, in tiles, of the column-major groups of the tile order
//   OCC          workgroups per CU the register / LDS budget is sized for
//   DTL          1: global -> LDS by direct-to-LDS buffer loads (no staging registers, no
//                ds_write); 0: global -> registers -> ds_write.  The predicated variant
//                always stages through registers (it has to mask the K tail there).
//   EPI          1: the C tile is transposed through LDS and written as whole row segments
//                (16 bytes per lane); 0: 8-byte stores straight from the accumulator layout
//                (2-byte stores in the predicated variant when C rows are not 8-byte aligned)
//   EDGE         predicated variant: any M, N, K and any alignment
//   DT           storage type (DT_BF16 / DT_FP16)
template <int BM_, int BN_, int WM_, int WN_, int SWZ_, int GROUP_, int OCC_, int DTL_, int EPI_, bool EDGE_, int DT_>
struct TileConfig {
    static constexpr int BM = BM_, BN = BN_, BK = 64;
    static constexpr int WM = WM_, WN = WN_;
    static constexpr int SWZ = SWZ_, GROUP = GROUP_, OCC = OCC_;
    static constexpr bool DTL = DTL_ != 0 && !EDGE_;
    static constexpr bool EPI = EPI_ != 0;
    static constexpr bool EDGE = EDGE_;
    static constexpr int DT = DT_;
    static constexpr int NT = WM * WN * 64;             // threads per workgroup
    static constexpr int TM = BM / WM, TN = BN / WN;    // wave tile
    static constexpr int MI = TM / 32, NI = TN / 32;    // 32x32 MFMA tiles per wave
    static constexpr int LA = BM * 8 / NT;              // 16-byte chunks per thread per K step
    static constexpr int LB = BN * 8 / NT;
    static constexpr int ROWS_PER_PASS = NT / 8;        // tile rows one pass of all threads covers
    static constexpr int A_STAGE = BM * 128, B_STAGE = BN * 128;
    static constexpr int LDS_BYTES = 2 * (A_STAGE + B_STAGE);
    static constexpr int WAVES_PER_EU = (NT / 256 > 0 ? NT / 256 : 1) * OCC;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "tile rows must divide over threads");
    static_assert(ROWS_PER_PASS % 16 == 0, "swizzle must be invariant across load passes");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

template <int DT>
__device__ __forceinline__ f32x16_t mfma_32x32x16(u32x4_t a, u32x4_t b, f32x16_t c) {
    if constexpr (DT == DT_BF16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                      __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                     __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
}

// fp32 -> storage type, round to nearest even (what `(CType)(acc)` is in reference.h:40).
template <int DT>
__device__ __forceinline__ uint16_t cvt_store(float f) {
    if constexpr (DT == DT_BF16) {
        __bf16 h = (__bf16)f;
        return __builtin_bit_cast(uint16_t, h);
    } else {
        _Float16 h = (_Float16)f;
        return __builtin_bit_cast(uint16_t, h);
    }
}
// Two values at once: one v_cvt_pk_{bf16,f16}_f32 (converting them one by one and or-ing the
// halves together costs three more VALU instructions per pair, 2000 cycles per 256x256 tile).
template <int DT>
__device__ __forceinline__ uint32_t cvt_store2(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    if constexpr (DT == DT_BF16) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
    } else {
        typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
    }
}

// Wait for this wave's LDS traffic, then meet the other waves.  Deliberately not
// __syncthreads(): that also drains vmcnt and would serialise the global prefetch.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// The epilogue of the reference's golden (reference.h:40): C = (CType)(acc * alpha + beta),
// two separately rounded fp32 operations, beta a plain scalar added to every element.
// alpha = 1, beta = 0 is what the reference's kernels compute (matmul_h100.cu.jinja:696) and
// what SCALED = false leaves out entirely: the kernels hold two copies of their epilogue
// behind one uniform branch, so the unscaled path and the K loop are unchanged by it.
// (Scaling the accumulators in place before a single epilogue costs registers in the loop.)
// x * a + b as two separately rounded fp32 operations.  (HIP's __fmul_rn / __fadd_rn are the
// plain operators and are contracted into one v_fma_f32 under the default -ffp-contract=fast;
// without the `contract` flag on these two operations they cannot be.)
__device__ __forceinline__ float mul_add_unfused(float x, float a, float b) {
#pragma clang fp contract(off)
    const float t = x * a;
    return t + b;
}
template <bool SCALED>
__device__ __forceinline__ float scale_acc(float x, float alpha, float beta) {
    if constexpr (SCALED) return mul_add_unfused(x, alpha, beta);
    else return x;
}

// blockIdx -> (tile_m, tile_n).  Hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs; undo that so each XCD walks one contiguous range of the logical order, then
// walk that order in column-major groups GROUP tiles tall so the tiles in flight on an XCD
// share A row panels and B column panels in its L2.  (Same purpose as the reference's
// cluster + 8x8 super-tile Schedule, matmul_utils.cuh:348-378.)
template <int GROUP>
__device__ __forceinline__ void tile_of_block(int pid, int nwg, int tiles_m, int tiles_n,
                                              int& tm, int& tn) {
    const int q = nwg >> 3, r = nwg & 7;
    const int x = pid & 7, loc = pid >> 3;
    const int logical = x * q + (x < r ? x : r) + loc;
    const int gw = GROUP * tiles_n;
    const int gid = logical / gw;
    const int first_m = gid * GROUP;
    const int gsz = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    const int in = logical - gid * gw;
    tm = first_m + in % gsz;
    tn = in / gsz;
}

// TRACE = true adds the per-workgroup timing record the reference's bf16 harness knows how
// to read from its `int* DB` argument (matmul_h100_optimal.cu:182-198): six ints
//   { sumLoad, cntLoad, sumCompute, cntCompute, sumStore, cntStore }
// at DB[6 * blockIdx.x], in s_memtime ticks: Load = time wave 0 spent at the per-K-step
// barrier (waiting for operands to land and for the other waves), counted once per K step;
// Compute = the whole main loop, counted per K step; Store = the epilogue, counted once.
// The caller pre-fills DB with ~0 so the first unused word terminates the list.
template <class Cfg, bool TRACE = false>
__global__ void __launch_bounds__(Cfg::NT)
__attribute__((amdgpu_waves_per_eu(Cfg::WAVES_PER_EU, Cfg::WAVES_PER_EU)))
gemm_tile_kernel(const GemmArgs p) {
    long long tr_wait = 0, tr_t0 = 0, tr_loop = 0;
    int tr_cnt = 0;
    auto tr_now = [&]() __attribute__((always_inline)) { return (long long)__builtin_readcyclecounter(); };
    if constexpr (TRACE) tr_loop = tr_now();
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
    constexpr int WN = Cfg::WN;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, LA = Cfg::LA, LB = Cfg::LB;
    constexpr int RPP = Cfg::ROWS_PER_PASS;
    constexpr int A_STAGE = Cfg::A_STAGE, B_STAGE = Cfg::B_STAGE;
    constexpr int DT = Cfg::DT;
    constexpr bool EDGE = Cfg::EDGE;

    // [A stage 0][A stage 1][B stage 0][B stage 1]
    __shared__ __attribute__((aligned(128))) unsigned char lds[Cfg::LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;

    int tm, tn;
    tile_of_block<Cfg::GROUP>(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
    const int row0 = tm * BM, col0 = tn * BN;
    const int M = p.M, N = p.N, K = p.K;
    // K steps, always an even number >= 2 so the LDS stage of every step is a compile-time
    // constant.  The aligned variant is only launched with K % 128 == 0; the predicated
    // one rounds up and the surplus step multiplies zeros.
    const int KT = EDGE ? ((K + 2 * BK - 1) / (2 * BK)) * 2 : K / BK;

    // ---- global side: one buffer descriptor per operand, covering this tile's rows ----
    const int rowsA = (M - row0) < BM ? (M - row0) : BM;
    const int rowsB = (N - col0) < BN ? (N - col0) : BN;
    const unsigned char* Ab = (const unsigned char*)p.A + (size_t)row0 * p.lda * 2;
    const unsigned char* Bb = (const unsigned char*)p.B + (size_t)col0 * p.ldb * 2;
    // The descriptors end exactly at the last element of the tile's last row: nothing past
    // the end of a matrix is ever touched.
    const uint32_t bytesA = (uint32_t)((rowsA - 1) * p.lda + K) * 2u;
    const uint32_t bytesB = (uint32_t)((rowsB - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA =
        __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB =
        __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);

    const int r_t = tid >> 3, c_t = tid & 7;       // this thread's row-in-pass and 16B chunk
    const uint32_t voffA = (uint32_t)(r_t * p.lda + c_t * 8) * 2u;
    const uint32_t voffB = (uint32_t)(r_t * p.ldb + c_t * 8) * 2u;
    const uint32_t passA = (uint32_t)(RPP * p.lda) * 2u;   // byte step between load passes
    const uint32_t passB = (uint32_t)(RPP * p.ldb) * 2u;

    // ---- LDS side ----
    auto swz = [](int row) __attribute__((always_inline)) { return Cfg::SWZ ? ((row >> 1) & 7) : (row & 7); };
    // where this thread's chunk of pass 0 lands; pass j adds j * RPP * 128 bytes
    const int wr_off = r_t * 128 + ((c_t ^ swz(r_t)) << 4);
    // fragment reads: lane holds row (lane & 31), k chunk 2*ks + (lane >> 5)
    const int l32 = lane & 31, hi = lane >> 5;
    int rd_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) rd_off[ks] = l32 * 128 + ((((ks << 1) | hi) ^ swz(l32)) << 4);
    const int a_wave = wm * Cfg::TM * 128;
    const int b_wave = wn * Cfg::TN * 128;

    u32x4_t ga[LA], gb[LB];          // global -> register staging (tile kt+2 / kt+1)
    u32x4_t fa[2][MI], fb[2][NI];    // double-buffered MFMA operand fragments
    f32x16_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto gload_a = [&](int kt) __attribute__((always_inline)) {
        const uint32_t kb = (uint32_t)kt * (BK * 2);
#pragma unroll
        for (int j = 0; j < LA; ++j)
            ga[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrcA, voffA + kb + j * passA, 0, 0);
    };
    auto gload_b = [&](int kt) __attribute__((always_inline)) {
        const uint32_t kb = (uint32_t)kt * (BK * 2);
#pragma unroll
        for (int j = 0; j < LB; ++j)
            gb[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrcB, voffB + kb + j * passB, 0, 0);
    };
    // K tail (predicated variant).  (1) The chunk at k..k+7 of a row runs into the next
    // row, or past the buffer: zero whatever lies at k >= K.  The four dword masks depend
    // only on the K step and on this thread's chunk column, so all its chunks share them.
    // (2) The range check of a buffer load works on whole dwords, so the dword holding the
    // last element (k = K-1) of the tile's last row is dropped whenever its other half lies
    // past the descriptor's end (odd K).  That one element per operand is fetched by a
    // 2-byte load up front (tailA / tailB) and put back here.
    uint32_t tailA = 0, tailB = 0;
    if constexpr (EDGE) {
        tailA = __builtin_amdgcn_raw_buffer_load_b16(rsrcA, bytesA - 2u, 0, 0);
        tailB = __builtin_amdgcn_raw_buffer_load_b16(rsrcB, bytesB - 2u, 0, 0);
    }
    auto patch_last = [&](u32x4_t& v, bool hit, int kl, uint32_t e) __attribute__((always_inline)) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t old = v[d];
            const uint32_t pv = (kl & 1) ? ((old & 0x0000ffffu) | (e << 16)) : ((old & 0xffff0000u) | e);
            v[d] = (hit && (kl >> 1) == d) ? pv : old;
        }
    };
    auto mask_tail = [&](int kt) __attribute__((always_inline)) {
        const int nvalid = K - (kt * BK + c_t * 8);
        const int kl = nvalid - 1;                     // where k = K-1 sits in this chunk
        const bool mine = kl >= 0 && kl < 8;
        uint32_t m[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int n = nvalid - 2 * d;
            m[d] = n >= 2 ? 0xffffffffu : (n == 1 ? 0x0000ffffu : 0u);
        }
#pragma unroll
        for (int j = 0; j < LA; ++j) {
            patch_last(ga[j], mine && (j * RPP + r_t == rowsA - 1), kl, tailA);
#pragma unroll
            for (int d = 0; d < 4; ++d) ga[j][d] &= m[d];
        }
#pragma unroll
        for (int j = 0; j < LB; ++j) {
            patch_last(gb[j], mine && (j * RPP + r_t == rowsB - 1), kl, tailB);
#pragma unroll
            for (int d = 0; d < 4; ++d) gb[j][d] &= m[d];
        }
    };
    auto lds_store_a = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < LA; ++j) {
            *(u32x4_t*)(lds + stage * A_STAGE + wr_off + j * (RPP * 128)) = ga[j];
        }
    };
    auto lds_store_b = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < LB; ++j) {
            *(u32x4_t*)(lds + 2 * A_STAGE + stage * B_STAGE + wr_off + j * (RPP * 128)) = gb[j];
        }
    };
    auto read_frags = [&](int stage, int ks, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
            fa[buf][i] = *(const u32x4_t*)(lds + stage * A_STAGE + a_wave + i * 4096 + rd_off[ks]);
#pragma unroll
        for (int j = 0; j < NI; ++j)
            fb[buf][j] =
                *(const u32x4_t*)(lds + 2 * A_STAGE + stage * B_STAGE + b_wave + j * 4096 + rd_off[ks]);
    };
    // Operands are passed swapped (B fragment as the MFMA "A" matrix): the 32x32 result
    // is then C^T, so a lane ends up holding 4 consecutive n for one m -> 8-byte stores
    // into row-major C.
    auto mma = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
                acc[i][j] = mfma_32x32x16<DT>(fb[buf][j], fa[buf][i], acc[i][j]);
    };

    if constexpr (Cfg::DTL) {
        // ---- direct-to-LDS pipeline (aligned shapes) ----
        // A buffer load with the `lds` modifier writes lane l's 16 bytes to LDS address
        // M0 + 16*l, so one wave instruction fills 8 consecutive 128-byte rows.  The LDS
        // swizzle is therefore applied on the global side: the lane that lands on chunk
        // position c' of row r fetches logical chunk c' ^ swz(r).  Wave w, pass j fills
        // rows (j*NW + w)*8 .. +7 of the tile.
        // The compiler knows nothing of these loads (they are inline asm), so the waits on
        // them are explicit: vmcnt(0) before the barrier that publishes a stage.
        const int lr = lane >> 3, lc = lane & 7;
        const int drow = wave * 8 + lr;                       // tile row of pass 0
        const int dchunk = lc ^ swz(drow);
        const uint32_t dvoffA = (uint32_t)(drow * p.lda + dchunk * 8) * 2u;
        const uint32_t dvoffB = (uint32_t)(drow * p.ldb + dchunk * 8) * 2u;
        const uint32_t lds_base =
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
        const uint32_t dlds = lds_base + (uint32_t)wave * 1024u;   // + stage + pass * RPP * 128
        auto dma = [&](const __amdgpu_buffer_rsrc_t& rsrc, uint32_t voff, uint32_t dst) __attribute__((always_inline)) {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                         :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
        };
        auto dma_a = [&](int kt, int stage) __attribute__((always_inline)) {
            const uint32_t kb = (uint32_t)kt * (BK * 2);
#pragma unroll
            for (int j = 0; j < LA; ++j)
                dma(rsrcA, dvoffA + kb + j * passA, dlds + stage * A_STAGE + j * (RPP * 128));
        };
        auto dma_b = [&](int kt, int stage) __attribute__((always_inline)) {
            const uint32_t kb = (uint32_t)kt * (BK * 2);
#pragma unroll
            for (int j = 0; j < LB; ++j)
                dma(rsrcB, dvoffB + kb + j * passB, dlds + 2 * A_STAGE + stage * B_STAGE + j * (RPP * 128));
        };
        auto vm_barrier = [&]() __attribute__((always_inline)) {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        };
        constexpr int NMMA = MI * NI, NFR = MI + NI;
        constexpr int DPM = (LA + LB + NMMA - 1) / NMMA;     // DMA instructions per MFMA slot
        // One MFMA, in the order (i, j) = (idx / NI, idx % NI).
        auto mma_one = [&](int buf, int idx) __attribute__((always_inline)) {
            const int i = idx / NI, j = idx % NI;
            acc[i][j] = mfma_32x32x16<DT>(fb[buf][j], fa[buf][i], acc[i][j]);
        };
        // Fragment r of a k slice, in the order the MFMAs above first need them:
        // A0, B0, B1, .., B(NI-1), A1, .., A(MI-1).
        auto read_one = [&](int stage, int ks, int buf, int r) __attribute__((always_inline)) {
            if (r == 0 || r > NI) {
                const int i = r == 0 ? 0 : r - NI;
                fa[buf][i] = *(const u32x4_t*)(lds + stage * A_STAGE + a_wave + i * 4096 + rd_off[ks]);
            } else {
                const int j = r - 1;
                fb[buf][j] = *(const u32x4_t*)(lds + 2 * A_STAGE + stage * B_STAGE + b_wave + j * 4096 + rd_off[ks]);
            }
        };
        auto dma_one = [&](int kt, int stage, int d) __attribute__((always_inline)) {
            const uint32_t kb = (uint32_t)kt * (BK * 2);
            if (d < LA)
                dma(rsrcA, dvoffA + kb + d * passA, dlds + stage * A_STAGE + d * (RPP * 128));
            else if (d < LA + LB)
                dma(rsrcB, dvoffB + kb + (d - LA) * passB,
                    dlds + 2 * A_STAGE + stage * B_STAGE + (d - LA) * (RPP * 128));
        };
        // tile 0 -> stage 0, tile 1 -> stage 1
        dma_a(0, 0);
        dma_b(0, 0);
        dma_a(1, 1);
        dma_b(1, 1);
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(LA + LB) : "memory");   // tile 0 landed
#pragma unroll
        for (int r = 0; r < NFR; ++r) read_one(0, 0, 0, r);
        // One K step.  LDS[cur] = tile kt, LDS[nxt] = tile kt+1 (landing).
        //   ks 0..2 : MFMA | fetch fragments ks+1 from LDS[cur]
        //   vmcnt(0) + barrier : tile kt+1 complete, LDS[cur] drained by every wave
        //   ks 3    : MFMA | fetch fragments ks 0 of tile kt+1 | start tile kt+2 -> LDS[cur]
        // Each slot is pinned (one MFMA, then at most one LDS read and DPM loads) so the
        // memory instructions are dealt out between the MFMAs.
        auto dstep = [&](int kt, auto cur_c, auto has1_c, auto has2_c) __attribute__((always_inline)) {
            constexpr int cur = decltype(cur_c)::value;
            constexpr int nxt = cur ^ 1;
            constexpr bool has1 = decltype(has1_c)::value;
            constexpr bool has2 = decltype(has2_c)::value;
#pragma unroll
            for (int ks = 0; ks < 3; ++ks) {
#pragma unroll
                for (int idx = 0; idx < NMMA; ++idx) {
                    mma_one(ks & 1, idx);
                    if (idx < NFR) read_one(cur, ks + 1, (ks + 1) & 1, idx);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if constexpr (has1) {
                if constexpr (TRACE) tr_t0 = tr_now();
                vm_barrier();
                if constexpr (TRACE) { tr_wait += tr_now() - tr_t0; ++tr_cnt; }
            }
#pragma unroll
            for (int idx = 0; idx < NMMA; ++idx) {
                mma_one(1, idx);
                if constexpr (has1) {
                    if (idx < NFR) read_one(nxt, 0, 0, idx);
                }
                if constexpr (has2) {
#pragma unroll
                    for (int d = 0; d < DPM; ++d) dma_one(kt + 2, cur, idx * DPM + d);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        using T = std::true_type;
        using F = std::false_type;
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        int kt = 0;
        for (; kt + 2 < KT; kt += 2) {
            dstep(kt, S0{}, T{}, T{});
            dstep(kt + 1, S1{}, T{}, T{});
        }
        dstep(kt, S0{}, T{}, F{});
        dstep(kt + 1, S1{}, F{}, F{});
    } else {
        // ---- prologue: tile 0 -> LDS stage 0, tile 1 -> registers ----
        gload_a(0);
        gload_b(0);
        if constexpr (EDGE) mask_tail(0);
        lds_store_a(0);
        lds_store_b(0);
        gload_a(1);
        gload_b(1);
        lds_barrier();
        read_frags(0, 0, 0);

        // One K step = four 16-deep k slices (ks), 16 MFMAs each for a 128x128 wave tile.
        // LDS[cur] holds tile kt, registers hold tile kt+1 (if any).
        //   ks 0 : MFMA(ks 0) | fetch fragments ks 1 | A registers (tile kt+1) -> LDS[nxt]
        //   ks 1 : MFMA(ks 1) | fetch fragments ks 2 | B registers -> LDS[nxt], global loads of
        //          A for tile kt+2
        //   ks 2 : MFMA(ks 2) | fetch fragments ks 3 | global loads of B for tile kt+2
        //   barrier: LDS[nxt] complete, LDS[cur] drained
        //   ks 3 : MFMA(ks 3) | fetch fragments ks 0 of tile kt+1 from LDS[nxt]
        // Every write to a stage follows the barrier that ended the step in which it was last
        // read, and every read follows the barrier after it was written: one barrier per step.
        // The sched_group_barrier sequences ask the scheduler to deal the memory instructions
        // of a slice out between its MFMAs instead of bunching them in front.
        auto interleave = [&](auto nmfma_c, auto nread_c, auto nwrite_c, auto nvmem_c) __attribute__((always_inline)) {
            constexpr int nmfma = decltype(nmfma_c)::value, nread = decltype(nread_c)::value;
            constexpr int nwrite = decltype(nwrite_c)::value, nvmem = decltype(nvmem_c)::value;
    #pragma unroll
            for (int i = 0; i < nmfma; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA
                if (i < nread) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
                if (i >= nmfma - nwrite) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // LDS write
                if (i >= nmfma - nvmem) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // global load
            }
        };
        constexpr int NMMA = MI * NI, NFR = MI + NI;
        static_assert(NFR <= NMMA && LA <= NMMA && LB <= NMMA, "interleave pattern assumes it");
        using I0 = std::integral_constant<int, 0>;
        using IM = std::integral_constant<int, NMMA>;
        using IR = std::integral_constant<int, NFR>;
        using IA = std::integral_constant<int, LA>;
        using IB = std::integral_constant<int, LB>;
        auto kstep = [&](int kt, auto cur_c, auto has1_c, auto has2_c, auto mask_c) __attribute__((always_inline)) {
            constexpr bool mask = decltype(mask_c)::value;   // tile kt+1 may cross K
            constexpr int cur = decltype(cur_c)::value;
            constexpr int nxt = cur ^ 1;
            constexpr bool has1 = decltype(has1_c)::value;   // tile kt+1 exists
            constexpr bool has2 = decltype(has2_c)::value;   // tile kt+2 exists
            // ks 0
            read_frags(cur, 1, 1);
            if constexpr (has1) {
                if constexpr (mask) mask_tail(kt + 1);
                lds_store_a(nxt);
            }
            mma(0);
            if constexpr (has1) interleave(IM{}, IR{}, IA{}, I0{}); else interleave(IM{}, IR{}, I0{}, I0{});
            __builtin_amdgcn_sched_barrier(0);
            // ks 1
            read_frags(cur, 2, 0);
            if constexpr (has1) lds_store_b(nxt);
            if constexpr (has2) gload_a(kt + 2);
            mma(1);
            if constexpr (has2) interleave(IM{}, IR{}, IB{}, IA{});
            else if constexpr (has1) interleave(IM{}, IR{}, IB{}, I0{});
            else interleave(IM{}, IR{}, I0{}, I0{});
            __builtin_amdgcn_sched_barrier(0);
            // ks 2
            read_frags(cur, 3, 1);
            if constexpr (has2) gload_b(kt + 2);
            mma(0);
            if constexpr (has2) interleave(IM{}, IR{}, I0{}, IB{}); else interleave(IM{}, IR{}, I0{}, I0{});
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (TRACE) tr_t0 = tr_now();
            lds_barrier();
            if constexpr (TRACE) { tr_wait += tr_now() - tr_t0; ++tr_cnt; }
            // ks 3
            if constexpr (has1) read_frags(nxt, 0, 0);
            mma(1);
            if constexpr (has1) interleave(IM{}, IR{}, I0{}, I0{});
            __builtin_amdgcn_sched_barrier(0);
        };
        using T = std::true_type;
        using F = std::false_type;
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        // Steady state, two steps per trip; then the draining steps.  Only the last two tiles
        // can cross K (KT is rounded up to even), so only the steps that move those tiles into
        // LDS carry the masking code.
        using E = std::integral_constant<bool, EDGE>;
        int kt = 0;
        for (; kt + 4 < KT; kt += 2) {
            kstep(kt, S0{}, T{}, T{}, F{});
            kstep(kt + 1, S1{}, T{}, T{}, F{});
        }
        if (KT >= 4) {
            kstep(kt, S0{}, T{}, T{}, F{});
            kstep(kt + 1, S1{}, T{}, T{}, E{});
            kt += 2;
        }
        kstep(kt, S0{}, T{}, F{}, E{});
        kstep(kt + 1, S1{}, F{}, F{}, F{});

    }

    long long tr_store = 0;
    if constexpr (TRACE) {
        tr_store = tr_now();
        tr_loop = tr_store - tr_loop;
    }
    // ---- epilogue: fp32 -> storage type -> row-major C ----
    // acc[i][j][e] of lane l is C[m][n] with m = row of A fragment = l & 31,
    // n = 8*(e/4) + 4*(l>>5) + (e%4) inside the 32x32 tile.
    unsigned char* Cb = (unsigned char*)p.C + (size_t)row0 * p.ldc * 2;
    const uint32_t bytesC = (uint32_t)(rowsA * p.ldc) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcC =
        __builtin_amdgcn_make_buffer_rsrc((void*)Cb, 0, (int)bytesC, 0x00020000);
    auto epilogue = [&](auto scaled_c) __attribute__((always_inline)) {
    constexpr bool SCALED = decltype(scaled_c)::value;   // alpha / beta epilogue: see scale_acc
    const float alpha = p.alpha, beta = p.beta;
    if constexpr (Cfg::EPI) {
        // Through LDS: each wave lays its TM x TN tile out row-major in its own slice of the
        // (now idle) stage buffers, 16-byte chunks XOR-swizzled by the row, then reads rows
        // back 16 bytes per lane so that one store instruction writes whole row segments.
        // Only the first barrier involves the other waves.  The predicated variant masks
        // rows past M and splits the chunk that straddles N into 2-byte stores; its 16-byte
        // stores may start at any 2-byte boundary (odd N).
        constexpr int TM = Cfg::TM, TN = Cfg::TN;
        constexpr int CPR = TN / 8;                 // 16-byte chunks per row of the wave tile
        constexpr bool POW2 = (CPR & (CPR - 1)) == 0;
        static_assert(CPR % 4 == 0 && (TM * CPR) % 64 == 0, "C staging layout");
        static_assert(TM * TN * 2 * Cfg::WM * Cfg::WN <= Cfg::LDS_BYTES, "staging fits the stage buffers");
        // bank-conflict-free for 8-byte writes down a column of rows: rows of a power-of-two
        // width are spread by the row number, 192-byte rows (4 rows = 3 bank rounds) by row / 4
        auto cswz = [](int row) __attribute__((always_inline)) {
            return POW2 ? (row & (CPR - 1)) : ((row >> 2) & 3);
        };
        lds_barrier();                              // every wave is done reading the last stage
        unsigned char* stg = lds + wave * (TM * TN * 2);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int row = i * 32 + l32;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int chunk = (j * 4 + g) ^ cswz(row);
                    u32x2_t w;
                    w[0] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][g * 4 + 0], alpha, beta),
                                          scale_acc<SCALED>(acc[i][j][g * 4 + 1], alpha, beta));
                    w[1] = cvt_store2<DT>(scale_acc<SCALED>(acc[i][j][g * 4 + 2], alpha, beta),
                                          scale_acc<SCALED>(acc[i][j][g * 4 + 3], alpha, beta));
                    *(u32x2_t*)(stg + row * (TN * 2) + chunk * 16 + hi * 8) = w;
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // own writes visible to own reads
#pragma unroll
        for (int r = 0; r < TM * CPR / 64; ++r) {
            // chunk r*64 + lane of the wave tile, rows first
            const int idx = r * 64 + lane;
            const int row = POW2 ? r * (64 / CPR) + lane / CPR : idx / CPR;
            const int rc = POW2 ? lane % CPR : idx % CPR;
            const u32x4_t v = *(const u32x4_t*)(stg + row * (TN * 2) + ((rc ^ cswz(row)) << 4));
            const int m_loc = wm * TM + row;
            const int n = col0 + wn * TN + rc * 8;
            const uint32_t off = (uint32_t)(m_loc * p.ldc + n) * 2u;
            if constexpr (!EDGE) {
                __builtin_amdgcn_raw_buffer_store_b128(v, rsrcC, off, 0, 0);
            } else {
                if (m_loc < rowsA) {
                    if (n + 7 < N) {
                        __builtin_amdgcn_raw_buffer_store_b128(v, rsrcC, off, 0, 0);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (n + e < N)
                                __builtin_amdgcn_raw_buffer_store_b16(
                                    (uint16_t)(v[e >> 1] >> ((e & 1) * 16)), rsrcC, off + 2 * e, 0, 0);
                    }
                }
            }
        }
    } else {
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m_loc = wm * Cfg::TM + i * 32 + l32;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = col0 + wn * Cfg::TN + j * 32 + g * 8 + hi * 4;
                const uint32_t off = (uint32_t)(m_loc * p.ldc + n) * 2u;
                const float v0 = scale_acc<SCALED>(acc[i][j][g * 4 + 0], alpha, beta);
                const float v1 = scale_acc<SCALED>(acc[i][j][g * 4 + 1], alpha, beta);
                const float v2 = scale_acc<SCALED>(acc[i][j][g * 4 + 2], alpha, beta);
                const float v3 = scale_acc<SCALED>(acc[i][j][g * 4 + 3], alpha, beta);
                if constexpr (!EDGE) {
                    u32x2_t w;
                    w[0] = cvt_store2<DT>(v0, v1);
                    w[1] = cvt_store2<DT>(v2, v3);
                    __builtin_amdgcn_raw_buffer_store_b64(w, rsrcC, off, 0, 0);
                } else {
                    if (m_loc < rowsA) {
                        if (p.c_vec_ok && n + 3 < N) {
                            u32x2_t w;
                            w[0] = cvt_store2<DT>(v0, v1);
                            w[1] = cvt_store2<DT>(v2, v3);
                            __builtin_amdgcn_raw_buffer_store_b64(w, rsrcC, off, 0, 0);
                        } else {
                            if (n + 0 < N) __builtin_amdgcn_raw_buffer_store_b16(cvt_store<DT>(v0), rsrcC, off + 0, 0, 0);
                            if (n + 1 < N) __builtin_amdgcn_raw_buffer_store_b16(cvt_store<DT>(v1), rsrcC, off + 2, 0, 0);
                            if (n + 2 < N) __builtin_amdgcn_raw_buffer_store_b16(cvt_store<DT>(v2), rsrcC, off + 4, 0, 0);
                            if (n + 3 < N) __builtin_amdgcn_raw_buffer_store_b16(cvt_store<DT>(v3), rsrcC, off + 6, 0, 0);
                        }
                    }
                }
            }
        }
    }
    }
    };
    if (p.alpha != 1.0f || p.beta != 0.0f) epilogue(std::true_type{});
    else epilogue(std::false_type{});
    if constexpr (TRACE) {
        if (p.DB != nullptr && tid == 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the stores have left the wave
            tr_store = tr_now() - tr_store;
            int* rec = p.DB + 6 * (size_t)blockIdx.x;
            rec[0] = (int)tr_wait;
            rec[1] = tr_cnt;
            rec[2] = (int)tr_loop;
            rec[3] = KT;
            rec[4] = (int)tr_store;
            rec[5] = 1;
        }
    }
}

}  // namespace mi
