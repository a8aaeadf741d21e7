// gemm_wavek_kernel.hpp -- gfx950 GEMM kernels for outputs of few tiles:
//
//   C[M,N] = A[M,K] . B[N,K]^T     small tiles; one kernel and no workspace, except for a very long K
//   gemm_wavek_kernel:        K split over the four waves of a workgroup (few tiles, long K)
//   gemm_shared_ring_kernel:  2 x 2 waves over the tile, one shared ring (further down)
//
// A 512 x 512 or 1024 x 1024 output has 16 or 64 tiles of 128 x 128: most of the chip idles,
// or K is cut into pieces whose partial sums make a round trip through memory and a second
// launch.  Here the tile is small enough (32 x 32 ... 96 x 64) for every CU to own one, and
// what a small tile loses -- each wave of a 2 x 2 wave grid would re-read most of the tile's
// LDS for very few MFMAs -- is avoided by splitting K instead of the tile:
//   * the four waves of a workgroup each multiply the WHOLE tile over a quarter of K (wave w
//     takes the 64-deep units w, w+4, ... of K, so the workgroup as a whole walks 512
//     contiguous bytes of every row) and every fragment read from LDS feeds MI (or NI) MFMAs;
//   * each wave has a private ring in LDS, filled by its own direct-to-LDS buffer loads and
//     drained by its own MFMAs: a wave waits only on its own `vmcnt`, there is no barrier in
//     the loop;
//   * a ring stage is one unit: (BM + BN) rows of 128 bytes, XOR-swizzled.  One load
//     instruction fills 8 rows: lane l lands on 16-byte position l & 7 of row l >> 3 and fetches
//     chunk (l & 7) ^ ((row >> 1) & 7) of the row, so that the fragment read (lane l: row
//     l & 15, chunk 4*slice + (l >> 4) -- the operand layout of v_mfma_f32_16x16x32) touches
//     every bank once.  Whole 128-byte lines per request matter: an L2 delivers whole lines,
//     and with 64-byte rows (a ring of half units, twice as deep) this kernel ran at half the
//     rate (1024 x 1024 x 4096 on 64 x 64 tiles: 24.3 us);
//   * all fragments of a unit are read into registers first, so its stage takes the next
//     request before the MFMAs start: a ring of NS stages keeps NS units in flight.  (A K loop
//     software-pipelined by hand -- fragment reads and requests dealt out between the MFMAs --
//     was 10-35 % slower than this plain order, which the compiler schedules itself);
//   * every workgroup walks K from its start: the workgroups of an XCD that share rows of A
//     or B then ask for them at about the same time and all but the first hit in the L2 (a
//     rotated start per workgroup, as the decode kernels use against HBM channel crowding,
//     cost 1024 x 1024 x 4096 a third: 14.8 -> 19.8 us);
//   * the four partial tiles are added in wave order through LDS (a fixed order: results are
//     reproducible), scaled, rounded once and stored with 8-byte stores.
// The kernel is bound by what a CU can pull through its L1 ((BM + BN) x 128 bytes per unit of
// K, measured 80-100 GB/s per CU), which is why the tile is as square as the shape allows.
// Rings of one or two stages leave room for two to five workgroups on a CU (32 x 32 with one
// stage: 32 KB of LDS); alone on its CU such a workgroup is level with the deep rings, with
// company it is 5-18 % ahead once the tiles run to more than one round, because co-resident
// workgroups hide each other's first loads and epilogue (1344^3 on 64 x 64: 13.2 -> 11.3 us).
// Eight waves (two per SIMD, K split eight ways, rings half as deep) ran level with or up to
// 8 % behind four on every shape tried.  Tiles of 128 x 128 and 128 x 64, which fit with a
// single stage and one workgroup per CU only, were far behind the tiled kernels (2048^3:
// 26.5 us against 19.6): alone and with one stage, loading and multiplying take turns.
// Rows of A past M and rows of B past N are never fetched (the buffer descriptors end at the
// last valid row of the tile).  Precondition, checked by the launcher's caller: 4-byte aligned A
// and B.  Any K (a partial last unit is filled up with zeros; the last k of an odd K is added in
// the epilogue).  Any N and any C: where the
// groups of four elements do not all start on 8-byte boundaries inside N, C is stored element
// by element.  Rows that start on 128-byte boundaries (K % 64 == 0, aligned bases) are what the
// kernel is fastest on: with any other pitch every 128-byte piece of a row straddles two lines.
// A very long K under an output of so few tiles that even these leave CUs idle (128 x 384 x 13376)
// is cut into pieces of whole units, one workgroup per (tile, piece) on gridDim.y: the piece's
// sums go to the workspace as fp32 and splitk_reduce_kernel adds the pieces (the host's choice,
// DecodeArgs::splits; 19.9 -> 10.8 us there).
// The reference has no counterpart: its kernels use one tile size (matmul_utils.cuh:362).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_kernel.hpp"
#include "gemm_mfma16_kernel.hpp"   // mfma_16x16x32
#include "splitk_common.hpp"        // DecodeArgs

namespace mi {

// K tail inside a 16-byte chunk (K % 8 != 0, K even).  The chunk of a row that holds k = K - 1
// also holds the first elements of the next row of the matrix; the lane that fetched it keeps
// its K % 8 leading elements and zeroes the rest, in LDS, once its loads of that unit have
// landed and before anyone reads the stage.  `ptr`: the 16 bytes this lane's load wrote.
__device__ __forceinline__ void zero_chunk_tail(unsigned char* ptr, int keep_elems) {
    u32x4_t v = *(const u32x4_t*)ptr;
    const int keep_words = keep_elems >> 1;                  // K is even: whole 32-bit words
#pragma unroll
    for (int w = 0; w < 4; ++w) v[w] = w < keep_words ? v[w] : 0u;
    *(u32x4_t*)ptr = v;
}

// One element of A or B as fp32 (the last k of an odd K, which the loops below leave out).
template <int DT>
__device__ __forceinline__ float load_elem(const void* base, size_t index) {
    const uint16_t u = ((const uint16_t*)base)[index];
    if constexpr (DT == DT_BF16) return __builtin_bit_cast(float, (uint32_t)u << 16);
    else return (float)__builtin_bit_cast(_Float16, u);
}

template <int BM_, int BN_, int NS_, int DT_>
struct WaveKConfig {
    static constexpr int BM = BM_, BN = BN_, NS = NS_, DT = DT_;
    static constexpr int NT = 256, NW = 4;
    static constexpr int MI = BM / 16, NI = BN / 16;
    static constexpr int L = (BM + BN) / 8;                  // load instructions per unit
    static constexpr int STAGE = (BM + BN) * 128;            // bytes of a ring stage
    static constexpr int RING = NS * STAGE;
    static constexpr int PITCH = BN + 4;                     // floats per row of a partial tile (bank spread)
    static constexpr int TILE = BM * PITCH * 4;              // bytes of a tile of fp32 sums
    static constexpr int PART = TILE + (BM + BN) * 4;         // ... and, behind it, the last k of an odd K: A[row0 + m][K-1], then B[col0 + n][K-1]
    static constexpr int REGION = RING > PART ? RING : PART; // one wave's share of LDS
    static constexpr int LDS_BYTES = NW * REGION;
    static constexpr int QUADS = BM * BN / 4 / NT;           // 4-element groups of C per thread
    static_assert(BM % 16 == 0 && BN % 16 == 0, "whole 16x16 MFMA tiles");
    static_assert(NS >= 1 && (NS - 1) * L <= 63, "vmcnt is a 6-bit counter");
    static_assert(BM * BN / 4 % NT == 0, "the C tile divides over the threads");
    static_assert(BM + BN <= NT, "one thread per row of the A and B panels fetches the last k of an odd K");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

// TRACE: the per-workgroup timing record (TraceRec; thread 0 is in wave 0, so the waits and the
// K units are that wave's) for launches that pass a trace buffer.
template <class Cfg, bool TRACE = false>
__global__ void __launch_bounds__(256) gemm_wavek_kernel(const DecodeArgs p) {
    TraceRec<TRACE> tr;
    tr.begin();
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, DT = Cfg::DT;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, L = Cfg::L, STAGE = Cfg::STAGE;
    constexpr int PITCH = Cfg::PITCH, REGION = Cfg::REGION;

    __shared__ __attribute__((aligned(128))) unsigned char lds[Cfg::LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // split-K (gridDim.y pieces, the host's choice for few tiles with a very long K): this
    // workgroup takes k_per_split of K from k0 on (a multiple of 64: rows keep their alignment)
    // and leaves its sums in the workspace as fp32; splitk_reduce_kernel adds the pieces
    const int k0 = p.splits > 1 ? (int)blockIdx.y * p.k_per_split : 0;
    const int M = p.M, N = p.N, K = p.splits > 1 && p.K - k0 > p.k_per_split ? p.k_per_split : p.K - k0;
    const unsigned char* A0 = (const unsigned char*)p.A + (size_t)k0 * 2;
    const unsigned char* B0 = (const unsigned char*)p.B + (size_t)k0 * 2;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tm, tn;
    tile_of_block<4>(blockIdx.x, gridDim.x, tiles_m, tiles_n, tm, tn);
    const int row0 = tm * BM, col0 = tn * BN;
    // An odd K: the loops take the even part, whole 32-bit words of every row (so that no word the
    // descriptors' range check passes or drops is half inside a row), and the last k is added to
    // the sums in the epilogue, one product per element.
    const int Ke = K & ~1;
    const int KT = (Ke + 63) / 64;                           // units of K; the last may be partial
    const int tail_chunks = ((Ke & 63) + 7) >> 3;            // 16-byte chunks of a row in a partial last unit (0: none)
    const int tail_elems = Ke & 7;                           // elements of k < Ke in the last of them (0: all eight)
    const int cnt = (KT - wave + 3) / 4;                     // units of this wave: wave, wave+4, ...

    const int rowsA = (M - row0) < BM ? (M - row0) : BM;
    const int rowsB = (N - col0) < BN ? (N - col0) : BN;
    const unsigned char* Ab = A0 + (size_t)row0 * p.lda * 2;
    const unsigned char* Bb = B0 + (size_t)col0 * p.ldb * 2;
    const uint32_t bytesA = (uint32_t)((rowsA - 1) * p.lda + K) * 2u;
    const uint32_t bytesB = (uint32_t)((rowsB - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcNone = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, 0, 0x00020000);

    const uint32_t ring_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds + (uint32_t)wave * REGION;
    auto dma = [&](const __amdgpu_buffer_rsrc_t& rsrc, uint32_t voff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
    };
    auto swz = [](int row) __attribute__((always_inline)) { return (row >> 1) & 7; };
    // this lane's byte offset inside A and B for load instruction q of a unit (stage rows: A
    // first, then B; k offset added per request)
    const int lr = lane >> 3, lc = lane & 7;
    uint32_t voff[L];
#pragma unroll
    for (int q = 0; q < L; ++q) {
        const int row = q * 8 + lr;
        const int chunk = lc ^ swz(row);
        voff[q] = q * 8 < BM ? (uint32_t)(row * p.lda + chunk * 8) * 2u
                             : (uint32_t)((row - BM) * p.ldb + chunk * 8) * 2u;
    }

    // In a partial last unit the chunks at k >= K belong to the next row of the matrix: the
    // lanes that would fetch them ask for an offset past every descriptor instead and get zeros
    // (the chunk a lane fetches depends on the parity of the instruction only: swz(8 * q + lr)).
    const bool tail_ok_even = (lc ^ (lr >> 1)) < tail_chunks, tail_ok_odd = (lc ^ (4 | (lr >> 1))) < tail_chunks;
    // unit i of this wave is unit wave + 4*i of the matrix; `rq_gs` follows the unit about to
    // be requested (requests past the last one fetch nothing), `rq_left` the live units left
    int rq_gs = wave;
    int rq_left = cnt;
    auto request = [&](int stage) __attribute__((always_inline)) {
        const bool live = rq_left > 0;
        const bool tail = tail_chunks != 0 && rq_gs == KT - 1;
        --rq_left;
        const uint32_t kb = (uint32_t)rq_gs * 128u;
        rq_gs += 4;
        const uint32_t dst = ring_base + (uint32_t)(stage * STAGE);
        if (!tail) {
#pragma unroll
            for (int q = 0; q < L; ++q)
                dma(live ? (q * 8 < BM ? rsrcA : rsrcB) : rsrcNone, voff[q] + kb, dst + (uint32_t)(q * 1024));
        } else {                                             // (a path of its own: nothing of it in the other units' way)
#pragma unroll
            for (int q = 0; q < L; ++q)
                dma(q * 8 < BM ? rsrcA : rsrcB, ((q & 1) ? tail_ok_odd : tail_ok_even) ? voff[q] + kb : 0x80000000u,
                    dst + (uint32_t)(q * 1024));
        }
    };

    // fragment read: lane holds row l & 15 of a 16-row block, chunk 4*slice + (l >> 4)
    const int l16 = lane & 15, q4 = lane >> 4;
    int rd_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) rd_off[ks] = l16 * 128 + ((((ks << 2) | q4) ^ swz(l16)) << 4);

    f32x4_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
    for (int i = 0; i < NS; ++i) request(i);

    const unsigned char* ring = lds + wave * REGION;
    int s = 0;
    for (int u = 0; u < cnt; ++u) {
        // unit u of this wave has landed
        tr.wait_begin();
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"((NS - 1) * L) : "memory");
        tr.wait_end();
        if (tail_elems != 0 && wave + 4 * u == KT - 1) {
            // the matrix's last unit ends inside a chunk: each lane looks after what it fetched
#pragma unroll
            for (int q = 0; q < L; ++q)
                if ((lc ^ (((q & 1) << 2) | (lr >> 1))) == tail_chunks - 1)
                    zero_chunk_tail(lds + wave * REGION + s * STAGE + q * 1024 + lane * 16, tail_elems);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        const unsigned char* st = ring + s * STAGE;
        u32x4_t fa[2][MI], fb[2][NI];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int i = 0; i < MI; ++i) fa[ks][i] = *(const u32x4_t*)(st + i * 2048 + rd_off[ks]);
#pragma unroll
            for (int j = 0; j < NI; ++j) fb[ks][j] = *(const u32x4_t*)(st + (BM + j * 16) * 128 + rd_off[ks]);
        }
        // its fragments are in registers: the stage takes the request NS units ahead
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        request(s);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) acc[i][j] = mfma_16x16x32<DT>(fb[ks][j], fa[ks][i], acc[i][j]);
        s = s + 1 == NS ? 0 : s + 1;
    }
    // requests past this wave's last unit (empty descriptor: zeros) are still heading for
    // the ring: drain before the partial tile takes its place
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    tr.loop_end();

    // ---- add the four partial tiles in wave order, scale, round, store ----
    // acc[i][j][e] of lane l is P[m][n], m = i*16 + (l & 15), n = j*16 + 4*(l >> 4) + e
    float* part = (float*)(lds + wave * REGION);
    // entry t of the last-k row (fetched by thread t) sits behind the tile of wave t / 64, which
    // that wave is done with; the other waves may still be in their loops
    auto last_k = [&](int t) { return (float*)(lds + (t >> 6) * REGION + Cfg::TILE) + (t & 63); };
    // the last k of an odd K: one element per row of the A and B panels into LDS (rows outside
    // M or N count as zero).  Fetched here, not ahead of the loops: a register held across them
    // and a store for every K cost the even K 1-4 % (the shared ring most), this costs the odd
    // K nothing measurable
    if ((K & 1) != 0 && tid < BM + BN) {
        const bool of_a = tid < BM;
        const int r = of_a ? row0 + tid : col0 + tid - BM;
        float last_elem = 0.0f;
        if (r < (of_a ? M : N))
            last_elem = load_elem<DT>(of_a ? A0 : B0, (size_t)r * (of_a ? p.lda : p.ldb) + K - 1);
        *last_k(tid) = last_elem;
    }
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
            *(f32x4_t*)(part + (i * 16 + l16) * PITCH + j * 16 + 4 * q4) = acc[i][j];
    __syncthreads();
    const bool scaled = p.alpha != 1.0f || p.beta != 0.0f;
    const bool c_vec_ok = (N & 3) == 0 && (p.ldc & 3) == 0 && ((uintptr_t)p.C & 7u) == 0;
    // The usual calls -- alpha 1, beta 0 and an even K in one piece with rows of C in whole
    // 8-byte groups (1) or not (3), an odd K in one piece (4), a piece of an even K (2) -- each
    // take a copy of the loop without the branches of the others: with them in the loop every
    // group of four waits for its LDS reads on its own (96x96 tiles: 0.5 us per launch).
    auto store_c = [&](auto mode_c) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_c)::value;
    constexpr bool PLAIN = MODE == 1, PIECE = MODE == 2, BY_ELEMENT = MODE == 3, ODD = MODE == 4, ANY = MODE == 0;
#pragma unroll
    for (int it = 0; it < Cfg::QUADS; ++it) {
        const int q = it * 256 + tid;
        const int m = q / (BN / 4), n = (q % (BN / 4)) * 4;
        f32x4_t sum = *(const f32x4_t*)((const float*)lds + m * PITCH + n);
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const f32x4_t v = *(const f32x4_t*)((const float*)(lds + w * REGION) + m * PITCH + n);
            sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
        }
        if (ODD || (ANY && (K & 1) != 0)) {                  // the last k of an odd K
            const float a_last = *last_k(m);
            const f32x4_t b_last = *(const f32x4_t*)last_k(BM + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] += a_last * b_last[e];
        }
        if (PIECE || (ANY && p.splits > 1)) {                // (N % 4 == 0 is a launch precondition of split-K)
            if (row0 + m < M && col0 + n < N)
                *(f32x4_t*)(p.ws + ((size_t)blockIdx.y * M + row0 + m) * N + col0 + n) = sum;
            continue;
        }
        if (ANY && scaled) {
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] = mul_add_unfused(sum[e], p.alpha, p.beta);
        }
        if (row0 + m < M && col0 + n < N) {
            u32x2_t w2;
            w2[0] = cvt_store2<DT>(sum[0], sum[1]);
            w2[1] = cvt_store2<DT>(sum[2], sum[3]);
            unsigned char* dst = (unsigned char*)p.C + ((size_t)(row0 + m) * p.ldc + col0 + n) * 2;
            if (PLAIN || (!BY_ELEMENT && c_vec_ok)) {        // every group of four starts on an 8-byte boundary inside N
                *(u32x2_t*)dst = w2;
            } else {                                         // any N, any 2-byte aligned C: element by element
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col0 + n + e < N) ((uint16_t*)dst)[e] = (uint16_t)(w2[e >> 1] >> ((e & 1) * 16));
            }
        }
    }
    };
    if ((K & 1) == 0 && p.splits > 1) store_c(std::integral_constant<int, 2>{});
    else if (p.splits > 1 || scaled) store_c(std::integral_constant<int, 0>{});
    else if ((K & 1) != 0) store_c(std::integral_constant<int, 4>{});
    else if (c_vec_ok) store_c(std::integral_constant<int, 1>{});
    else store_c(std::integral_constant<int, 3>{});
    tr.finish(p.DB, cnt);
}

// ---------------------------------------------------------------------------------------
// Shared-ring variant, for outputs whose tiles of BM x BN number at most one per CU but are too
// large to be multiplied whole by every wave (96 x 96: 1536^2 is 256 of them, where 128 x 128
// tiles leave 112 CUs idle and each busy CU takes in a third more).  The four waves form a
// 2 x 2 grid over the tile and walk all of K together; one ring of NS stages, each one
// 64-deep unit of (BM + BN) rows laid out as above, is filled by all four waves (a quarter of
// a stage's load instructions each) and read by all four.  One barrier per unit: it tells
// every wave that the unit it is about to read has landed (each wave has waited for its own
// loads) and that the stage of the unit before it has been read by everyone, so that the
// request NS - 1 units ahead can take that stage.  The workgroup is bound by the same intake
// of a CU as the kernel above; the deeper ring keeps NS - 1 units in flight while one is
// multiplied.  Same preconditions, same stage layout, same fragment reads.
template <int BM_, int BN_, int NS_, int DT_>
struct SharedRingConfig {
    static constexpr int BM = BM_, BN = BN_, NS = NS_, DT = DT_;
    static constexpr int NT = 256, NW = 4;
    static constexpr int TM = BM / 2, TN = BN / 2;           // wave tile of the 2 x 2 wave grid
    static constexpr int MI = TM / 16, NI = TN / 16;
    static constexpr int L = (BM + BN) / 8;                  // load instructions per unit
    static constexpr int LW = L / NW;                        // ... of one wave
    static constexpr int STAGE = (BM + BN) * 128;
    static constexpr int RING = NS * STAGE;
    static constexpr int PITCH = BN + 4;                     // floats per row of the staged C tile (bank spread)
    static constexpr int TILE = BM * PITCH * 4;              // bytes of a tile of fp32 sums
    static constexpr int PART = TILE + (BM + BN) * 4;         // ... and, behind it, the last k of an odd K: A[row0 + m][K-1], then B[col0 + n][K-1]
    static constexpr int LDS_BYTES = RING > PART ? RING : PART;
    static constexpr int QUADS = BM * BN / 4 / NT;           // 4-element groups of C per thread
    static_assert(BM % 32 == 0 && BN % 32 == 0, "wave tiles of whole 16x16 MFMA tiles");
    static_assert(L % NW == 0, "a stage's load instructions divide over the waves");
    static_assert(NS >= 3 && (NS - 1) * LW <= 63, "a unit being read, one being multiplied, the rest in flight; vmcnt is a 6-bit counter");
    static_assert(BM * BN / 4 % NT == 0, "the C tile divides over the threads");
    static_assert(BM + BN <= NT, "one thread per row of the A and B panels fetches the last k of an odd K");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

// TRACE: the per-workgroup timing record (TraceRec) for launches that pass a trace buffer.
template <class Cfg, bool TRACE = false>
__global__ void __launch_bounds__(256) gemm_shared_ring_kernel(const DecodeArgs p) {
    TraceRec<TRACE> tr;
    tr.begin();
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, DT = Cfg::DT;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, LW = Cfg::LW, STAGE = Cfg::STAGE;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, PITCH = Cfg::PITCH;

    __shared__ __attribute__((aligned(128))) unsigned char lds[Cfg::LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    // split-K (gridDim.y pieces, the host's choice for few tiles with a very long K): this
    // workgroup takes k_per_split of K from k0 on (a multiple of 64: rows keep their alignment)
    // and leaves its sums in the workspace as fp32; splitk_reduce_kernel adds the pieces
    const int k0 = p.splits > 1 ? (int)blockIdx.y * p.k_per_split : 0;
    const int M = p.M, N = p.N, K = p.splits > 1 && p.K - k0 > p.k_per_split ? p.k_per_split : p.K - k0;
    const unsigned char* A0 = (const unsigned char*)p.A + (size_t)k0 * 2;
    const unsigned char* B0 = (const unsigned char*)p.B + (size_t)k0 * 2;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tm, tn;
    tile_of_block<4>(blockIdx.x, gridDim.x, tiles_m, tiles_n, tm, tn);
    const int row0 = tm * BM, col0 = tn * BN;
    // An odd K: the loops take the even part, whole 32-bit words of every row (so that no word the
    // descriptors' range check passes or drops is half inside a row), and the last k is added to
    // the sums in the epilogue, one product per element.
    const int Ke = K & ~1;
    const int KT = (Ke + 63) / 64;                           // units of K; the last may be partial
    const int tail_chunks = ((Ke & 63) + 7) >> 3;            // 16-byte chunks of a row in a partial last unit (0: none)
    const int tail_elems = Ke & 7;                           // elements of k < Ke in the last of them (0: all eight)

    const int rowsA = (M - row0) < BM ? (M - row0) : BM;
    const int rowsB = (N - col0) < BN ? (N - col0) : BN;
    const unsigned char* Ab = A0 + (size_t)row0 * p.lda * 2;
    const unsigned char* Bb = B0 + (size_t)col0 * p.ldb * 2;
    const uint32_t bytesA = (uint32_t)((rowsA - 1) * p.lda + K) * 2u;
    const uint32_t bytesB = (uint32_t)((rowsB - 1) * p.ldb + K) * 2u;
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, (int)bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)Bb, 0, (int)bytesB, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcNone = __builtin_amdgcn_make_buffer_rsrc((void*)Ab, 0, 0, 0x00020000);

    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    auto dma = [&](const __amdgpu_buffer_rsrc_t& rsrc, uint32_t voff, uint32_t dst) __attribute__((always_inline)) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
    };
    auto swz = [](int row) __attribute__((always_inline)) { return (row >> 1) & 7; };
    // load instruction wave * LW + q of a unit fills stage rows 8 * that .. + 7 (A rows first,
    // then B rows): this lane's byte offset inside A or B, k offset added per request.
    // In a partial last unit the chunks at k >= K belong to the next row of the matrix: the
    // lanes that would fetch them ask for an offset past every descriptor instead and get zeros.
    const int lr = lane >> 3, lc = lane & 7;
    uint32_t voff[LW];
#pragma unroll
    for (int q = 0; q < LW; ++q) {
        const int row = (wave * LW + q) * 8 + lr;
        const int chunk = lc ^ swz(row);
        voff[q] = row < BM ? (uint32_t)(row * p.lda + chunk * 8) * 2u
                           : (uint32_t)((row - BM) * p.ldb + chunk * 8) * 2u;
    }
    // (the chunk a lane fetches depends on the parity of the instruction only: swz(8 * inst + lr);
    // `even` / `odd` below are the parities of q, the wave's first instruction being wave * LW)
    const int par0 = (wave * LW) & 1;
    const int chunk_even = lc ^ ((par0 << 2) | (lr >> 1)), chunk_odd = lc ^ (((par0 ^ 1) << 2) | (lr >> 1));
    const bool tail_ok_even = chunk_even < tail_chunks, tail_ok_odd = chunk_odd < tail_chunks;
    // `rq_unit` follows the unit about to be requested; requests past the last unit fetch nothing
    int rq_unit = 0;
    auto request = [&](int stage, auto maybe_tail_c) __attribute__((always_inline)) {
        const bool live = rq_unit < KT;
        const bool tail = decltype(maybe_tail_c)::value && tail_chunks != 0 && rq_unit == KT - 1;
        const uint32_t kb = (uint32_t)rq_unit * 128u;
        ++rq_unit;
        const uint32_t dst = lds_base + (uint32_t)(stage * STAGE + wave * LW * 1024);
        if (!tail) {
#pragma unroll
            for (int q = 0; q < LW; ++q)
                dma(live ? ((wave * LW + q) * 8 < BM ? rsrcA : rsrcB) : rsrcNone, voff[q] + kb, dst + (uint32_t)(q * 1024));
        } else {                                             // (a path of its own: nothing of it in the other units' way)
#pragma unroll
            for (int q = 0; q < LW; ++q)
                dma((wave * LW + q) * 8 < BM ? rsrcA : rsrcB,
                    ((q & 1) ? tail_ok_odd : tail_ok_even) ? voff[q] + kb : 0x80000000u, dst + (uint32_t)(q * 1024));
        }
    };

    // fragment read: lane holds row l & 15 of a 16-row block, chunk 4*slice + (l >> 4)
    const int l16 = lane & 15, q4 = lane >> 4;
    int rd_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) rd_off[ks] = l16 * 128 + ((((ks << 2) | q4) ^ swz(l16)) << 4);
    const int a_wave = wm * TM * 128, b_wave = (BM + wn * TN) * 128;

    f32x4_t acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
    for (int i = 0; i < NS - 1; ++i) request(i, std::true_type{});

    // The fragments of unit u + 1 are read while unit u is multiplied (one wave per SIMD has
    // nothing else to hide the LDS latency behind), so a unit must have landed one step before
    // it is multiplied: NS - 2 units are in flight while one is read and one multiplied.
    // Two register sets, used in turn (a copy from "next" to "current" at the end of a step
    // lets the compiler move the reads behind the MFMAs again).
    u32x4_t fa[2][2][MI], fb[2][2][NI];                      // [set][slice][block]
    auto read_unit = [&](int stage, u32x4_t (&a)[2][MI], u32x4_t (&b)[2][NI]) __attribute__((always_inline)) {
        const unsigned char* st = lds + stage * STAGE;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int i = 0; i < MI; ++i) a[ks][i] = *(const u32x4_t*)(st + a_wave + i * 2048 + rd_off[ks]);
#pragma unroll
            for (int j = 0; j < NI; ++j) b[ks][j] = *(const u32x4_t*)(st + b_wave + j * 2048 + rd_off[ks]);
        }
    };
    int s = 0;                                               // stage of the unit being multiplied
    int landed = 0;                                          // the unit whose landing the next barrier publishes
    // the matrix's last unit ends inside a chunk: each lane looks after what it fetched, after its
    // loads of that unit have landed and before the barrier that lets everyone read the stage
    auto fix_tail = [&](int stage) __attribute__((always_inline)) {
        if (tail_elems != 0 && landed == KT - 1) {
#pragma unroll
            for (int q = 0; q < LW; ++q)
                if (((q & 1) ? chunk_odd : chunk_even) == tail_chunks - 1)
                    zero_chunk_tail(lds + stage * STAGE + (wave * LW + q) * 1024 + lane * 16, tail_elems);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        ++landed;
    };
    // one step: unit u (fragments in set CUR) is multiplied while unit u + 1 is read into the other set.
    // TAIL: the step may publish or request the matrix's partial last unit.  The steps that cannot
    // are free of branches: with more than one basic block in the loop the compiler waits for
    // every LDS read before the first MFMA, the next unit's included (1440 x 1440 x 1472: 14.0 us
    // against 12.4).
    auto step = [&](auto cur_c, auto tail_c) __attribute__((always_inline)) {
        constexpr int CUR = decltype(cur_c)::value;
        constexpr bool TAIL = decltype(tail_c)::value;
        // this wave's loads of unit u + 1 have landed; after the barrier everyone's have, and
        // everyone has multiplied unit u - 1, whose stage takes the request NS - 1 units ahead
        tr.wait_begin();
        if constexpr (TAIL) {
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"((NS - 3) * LW) : "memory");
            fix_tail(s + 1 == NS ? 0 : s + 1);
            asm volatile("s_barrier" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"((NS - 3) * LW) : "memory");
            ++landed;
        }
        tr.wait_end();
        request(s == 0 ? NS - 1 : s - 1, tail_c);
        read_unit(s + 1 == NS ? 0 : s + 1, fa[CUR ^ 1], fb[CUR ^ 1]);   // (past the last unit: zeros or stale rows, never multiplied)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = mfma_16x16x32<DT>(fb[CUR][ks][j], fa[CUR][ks][i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        s = s + 1 == NS ? 0 : s + 1;
    };
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"((NS - 2) * LW) : "memory");     // unit 0 has landed
    fix_tail(0);
    asm volatile("s_barrier" ::: "memory");
    read_unit(0, fa[0], fb[0]);
    // the partial last unit (if any) is requested in step KT - NS and published in step KT - 2
    // (four steps per trip: at the loop's head the compiler waits for every LDS read, the next
    // unit's included, so the first step of a trip multiplies without that overlap; with two
    // steps per trip 512 x 1536 x 1792 on 64x64 tiles took 8.8 us, with four 7.4, with eight 7.4)
    const int plain_steps = (tail_chunks != 0 ? (KT > NS ? KT - NS : 0) : KT) & ~3;
    int u = 0;
    for (; u < plain_steps; u += 4) {
        step(std::integral_constant<int, 0>{}, std::false_type{});
        step(std::integral_constant<int, 1>{}, std::false_type{});
        step(std::integral_constant<int, 0>{}, std::false_type{});
        step(std::integral_constant<int, 1>{}, std::false_type{});
    }
    for (; u + 2 <= KT; u += 2) {
        step(std::integral_constant<int, 0>{}, std::true_type{});
        step(std::integral_constant<int, 1>{}, std::true_type{});
    }
    if (u < KT) step(std::integral_constant<int, 0>{}, std::true_type{});
    // requests past the last unit (empty descriptor: zeros) are still heading for the ring, and
    // other waves may still be reading the last stage: drain and meet before C takes its place
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    tr.loop_end();

    // ---- the C tile through LDS as fp32, then scaled, rounded once and stored 8 bytes per lane ----
    // acc[i][j][e] of lane l is C[m][n], m = wm*TM + i*16 + (l & 15), n = wn*TN + j*16 + 4*(l >> 4) + e
    float* part = (float*)lds;
    float* last_k = (float*)(lds + Cfg::TILE);
    // the last k of an odd K: one element per row of the A and B panels into LDS (rows outside
    // M or N count as zero).  Fetched here, not ahead of the loops: a register held across them
    // and a store for every K cost the even K 1-4 % (the shared ring most), this costs the odd
    // K nothing measurable
    if ((K & 1) != 0 && tid < BM + BN) {
        const bool of_a = tid < BM;
        const int r = of_a ? row0 + tid : col0 + tid - BM;
        float last_elem = 0.0f;
        if (r < (of_a ? M : N))
            last_elem = load_elem<DT>(of_a ? A0 : B0, (size_t)r * (of_a ? p.lda : p.ldb) + K - 1);
        last_k[tid] = last_elem;
    }
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
            *(f32x4_t*)(part + (wm * TM + i * 16 + l16) * PITCH + wn * TN + j * 16 + 4 * q4) = acc[i][j];
    __syncthreads();
    const bool scaled = p.alpha != 1.0f || p.beta != 0.0f;
    const bool c_vec_ok = (N & 3) == 0 && (p.ldc & 3) == 0 && ((uintptr_t)p.C & 7u) == 0;
    // The usual calls -- alpha 1, beta 0 and an even K in one piece with rows of C in whole
    // 8-byte groups (1) or not (3), an odd K in one piece (4), a piece of an even K (2) -- each
    // take a copy of the loop without the branches of the others: with them in the loop every
    // group of four waits for its LDS reads on its own (96x96 tiles: 0.5 us per launch).
    auto store_c = [&](auto mode_c) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_c)::value;
    constexpr bool PLAIN = MODE == 1, PIECE = MODE == 2, BY_ELEMENT = MODE == 3, ODD = MODE == 4, ANY = MODE == 0;
#pragma unroll
    for (int it = 0; it < Cfg::QUADS; ++it) {
        const int q = it * 256 + tid;
        const int m = q / (BN / 4), n = (q % (BN / 4)) * 4;
        f32x4_t sum = *(const f32x4_t*)(part + m * PITCH + n);
        if (ODD || (ANY && (K & 1) != 0)) {                  // the last k of an odd K
            const float a_last = last_k[m];
            const f32x4_t b_last = *(const f32x4_t*)(last_k + BM + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] += a_last * b_last[e];
        }
        if (PIECE || (ANY && p.splits > 1)) {                // (N % 4 == 0 is a launch precondition of split-K)
            if (row0 + m < M && col0 + n < N)
                *(f32x4_t*)(p.ws + ((size_t)blockIdx.y * M + row0 + m) * N + col0 + n) = sum;
            continue;
        }
        if (ANY && scaled) {
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] = mul_add_unfused(sum[e], p.alpha, p.beta);
        }
        if (row0 + m < M && col0 + n < N) {
            u32x2_t w2;
            w2[0] = cvt_store2<DT>(sum[0], sum[1]);
            w2[1] = cvt_store2<DT>(sum[2], sum[3]);
            unsigned char* dst = (unsigned char*)p.C + ((size_t)(row0 + m) * p.ldc + col0 + n) * 2;
            if (PLAIN || (!BY_ELEMENT && c_vec_ok)) {        // every group of four starts on an 8-byte boundary inside N
                *(u32x2_t*)dst = w2;
            } else {                                         // any N, any 2-byte aligned C: element by element
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col0 + n + e < N) ((uint16_t*)dst)[e] = (uint16_t)(w2[e >> 1] >> ((e & 1) * 16));
            }
        }
    }
    };
    if ((K & 1) == 0 && p.splits > 1) store_c(std::integral_constant<int, 2>{});
    else if (p.splits > 1 || scaled) store_c(std::integral_constant<int, 0>{});
    else if ((K & 1) != 0) store_c(std::integral_constant<int, 4>{});
    else if (c_vec_ok) store_c(std::integral_constant<int, 1>{});
    else store_c(std::integral_constant<int, 3>{});
    tr.finish(p.DB, KT);
}

// the second launch of a split-K run: the pieces' sums added in order, scaled, rounded once
template <int DT>
hipError_t launch_splitk_reduce(const DecodeArgs& a, hipStream_t stream) {
    const size_t quads = ((size_t)a.M * a.N + 3) / 4;
    return launch_kernel(splitk_reduce_kernel<DT>, dim3((unsigned)((quads + 255) / 256)), dim3(256), stream,
                         a.ws, a.C, a.M, a.N, a.ldc, a.splits, a.alpha, a.beta);
}

template <class Cfg>
hipError_t launch_shared_ring_kernel(const DecodeArgs& a, hipStream_t stream) {
    const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
    hipError_t e = a.DB ? launch_kernel(gemm_shared_ring_kernel<Cfg, true>, dim3(tiles, a.splits), dim3(256), stream, a)
                        : launch_kernel(gemm_shared_ring_kernel<Cfg, false>, dim3(tiles, a.splits), dim3(256), stream, a);
    return e != hipSuccess || a.splits == 1 ? e : launch_splitk_reduce<Cfg::DT>(a, stream);
}

template <class Cfg>
hipError_t launch_wavek_kernel(const DecodeArgs& a, hipStream_t stream) {
    const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
    hipError_t e = a.DB ? launch_kernel(gemm_wavek_kernel<Cfg, true>, dim3(tiles, a.splits), dim3(256), stream, a)
                        : launch_kernel(gemm_wavek_kernel<Cfg, false>, dim3(tiles, a.splits), dim3(256), stream, a);
    return e != hipSuccess || a.splits == 1 ? e : launch_splitk_reduce<Cfg::DT>(a, stream);
}

}  // namespace mi
