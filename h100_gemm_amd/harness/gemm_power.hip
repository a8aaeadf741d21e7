// gemm_power.hip -- where the cycles and the watts of the 8192^3 GEMM go: the default kernel
// (16x16x32 MFMA, 256x256 tile, drain barrier) next to copies of itself with parts of the K
// loop compiled out (the kernel's ABLATE parameter) and next to a loop of nothing but MFMAs; then
// the same kernel and its MFMA-only form on fp16 storage (the same values rounded to fp16).
//
//     ./gemm_power [seconds per variant] [M N K]         default 1.5 s, 8192 8192 8192
//
// Each variant runs back to back for the given time (after 0.3 s of warm-up: the clock takes
// ~100 ms to settle) while the host samples the socket power the driver reports
// (hwmon power1_input, microwatts) every 2 ms.  One line per variant: time per launch, TFLOP/s
// of the flops the full GEMM would do, cycles per 64-deep K step (from the kernel's own
// cycle counter, TRACE record of workgroup 0), shader clock (cycles / time), average socket
// power, joules per launch.  Not part of the library; the results of the ablated kernels are
// meaningless as GEMMs.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include <dirent.h>

#define MI_GEMM_ABLATE 1          // the kernel template with its ablation parameter (measurement build of the header)
#include "gemm_kernel.hpp"
#include "gemm_launch.hpp"
#include "gemm_mfma16_kernel.hpp"

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s:%d %s\n", __FILE__, __LINE__, hipGetErrorString(e_));          \
            exit(1);                                                                          \
        }                                                                                     \
    } while (0)

template <int DT>
using CfgT = mi::Mfma16Config<256, 256, 2, 2, 4, DT, 3, false, 1>;
using Cfg = CfgT<mi::DT_BF16>;

template <int ABLATE, int DT = mi::DT_BF16>
static void launch_variant(const mi::GemmArgs& a, bool trace) {
    const int grid = a.tiles_m * a.tiles_n;
    if (trace)
        hipLaunchKernelGGL((mi::gemm_mfma16_kernel<CfgT<DT>, true, false, ABLATE>), dim3(grid), dim3(Cfg::NT), 0, 0, a);
    else
        hipLaunchKernelGGL((mi::gemm_mfma16_kernel<CfgT<DT>, false, false, ABLATE>), dim3(grid), dim3(Cfg::NT), 0, 0, a);
}

// socket power in watts from the first hwmon node of a DRM card that has power1_input
static std::string find_power_file() {
    for (int card = 0; card < 16; ++card) {
        const std::string base = "/sys/class/drm/card" + std::to_string(card) + "/device/hwmon";
        DIR* d = opendir(base.c_str());
        if (!d) continue;
        while (dirent* e = readdir(d)) {
            if (strncmp(e->d_name, "hwmon", 5) != 0) continue;
            const std::string f = base + "/" + e->d_name + "/power1_input";
            if (FILE* t = fopen(f.c_str(), "r")) {
                fclose(t);
                closedir(d);
                return f;
            }
        }
        closedir(d);
    }
    return "";
}
static double read_watts(const std::string& file) {
    FILE* f = fopen(file.c_str(), "r");
    if (!f) return -1.0;
    double uw = -1.0;
    if (fscanf(f, "%lf", &uw) != 1) uw = -1.0;
    fclose(f);
    return uw < 0 ? -1.0 : uw * 1e-6;
}

static uint16_t to_fp16(float f) {
    const _Float16 h = (_Float16)f;
    uint16_t u;
    memcpy(&u, &h, 2);
    return u;
}
static float from_bf16(uint16_t v) {
    const uint32_t u = (uint32_t)v << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

int main(int argc, char** argv) {
    const double seconds = argc > 1 ? atof(argv[1]) : 1.5;
    const int M = argc > 4 ? atoi(argv[2]) : 8192, N = argc > 4 ? atoi(argv[3]) : 8192, K = argc > 4 ? atoi(argv[4]) : 8192;
    if (M % 256 || N % 256 || K % 128) {
        fprintf(stderr, "M, N multiples of 256 and K a multiple of 128\n");
        return 2;
    }
    const std::string power_file = find_power_file();
    // U[-1,1) operands, the benchmark's data: rounded to bf16; the same bf16 values in fp16
    // storage (exact: bf16 has the shorter mantissa); and the U[-1,1) values rounded to fp16
    // (three more mantissa bits per operand switching in the multipliers)
    const size_t na = (size_t)M * K, nb = (size_t)N * K;
    std::vector<float> f(na > nb ? na : nb);
    std::vector<uint16_t> h(f.size());
    uint64_t x = 0x9E3779B97F4A7C15ull;
    void *A, *B, *C, *A16, *B16, *A16f, *B16f;
    int* DB;
    HIP_OK(hipMalloc(&C, (size_t)M * N * 2));
    auto upload = [&](size_t n, void** bf, void** h16, void** h16f) {
        for (size_t i = 0; i < n; ++i) {
            x ^= x << 13; x ^= x >> 7; x ^= x << 17;
            f[i] = (float)(2.0 * ((double)(x >> 11) * (1.0 / 9007199254740992.0)) - 1.0);
        }
        HIP_OK(hipMalloc(bf, n * 2));
        HIP_OK(hipMalloc(h16, n * 2));
        HIP_OK(hipMalloc(h16f, n * 2));
        for (size_t i = 0; i < n; ++i) h[i] = to_bf16(f[i]);
        HIP_OK(hipMemcpy(*bf, h.data(), n * 2, hipMemcpyHostToDevice));
        for (size_t i = 0; i < n; ++i) h[i] = to_fp16(from_bf16(h[i]));
        HIP_OK(hipMemcpy(*h16, h.data(), n * 2, hipMemcpyHostToDevice));
        for (size_t i = 0; i < n; ++i) h[i] = to_fp16(f[i]);
        HIP_OK(hipMemcpy(*h16f, h.data(), n * 2, hipMemcpyHostToDevice));
    };
    upload(na, &A, &A16, &A16f);
    upload(nb, &B, &B16, &B16f);
    mi::GemmArgs a{};
    a.A = A; a.B = B; a.C = C;
    a.M = M; a.N = N; a.K = K;
    a.lda = K; a.ldb = K; a.ldc = N;
    a.tiles_m = M / 256; a.tiles_n = N / 256;
    a.c_vec_ok = 1;
    a.ws = nullptr; a.splits = 1; a.k_per_split = K;
    const size_t words = (size_t)a.tiles_m * a.tiles_n * 6 + 1;
    HIP_OK(hipMalloc(&DB, words * sizeof(int)));

    struct Variant { const char* name; void (*launch)(const mi::GemmArgs&, bool); int data; };     // data: 0 bf16, 1 fp16 holding the bf16 values, 2 fp16
    const Variant variants[] = {
        {"full kernel", launch_variant<0>, 0},
        {"no barriers", launch_variant<4>, 0},
        {"no LDS fragment reads", launch_variant<2>, 0},
        {"no global->LDS loads", launch_variant<1>, 0},
        {"no loads, no fragment reads", launch_variant<3>, 0},
        {"MFMAs only (no loads, reads, barriers)", launch_variant<7>, 0},
        {"no epilogue (C not written)", launch_variant<8>, 0},
        {"fp16 storage, the bf16 values: full kernel", launch_variant<0, mi::DT_FP16>, 1},
        {"fp16 storage, the bf16 values: MFMAs only", launch_variant<7, mi::DT_FP16>, 1},
        {"fp16 storage, U[-1,1) in fp16: full kernel", launch_variant<0, mi::DT_FP16>, 2},
        {"fp16 storage, U[-1,1) in fp16: MFMAs only", launch_variant<7, mi::DT_FP16>, 2},
    };
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    const double flops = 2.0 * M * N * K;
    printf("%dx%dx%d, U[-1,1) bf16, kernel m256x256_w2x2_g4_b3; power from %s\n", M, N, K,
           power_file.empty() ? "(no hwmon power1_input found)" : power_file.c_str());
    printf("%-46s %9s %9s %12s %7s %8s %9s\n", "variant", "ms", "TFLOP/s", "cyc/K-step", "GHz", "watts", "J/launch");
    for (const Variant& v : variants) {
        a.DB = nullptr;
        a.A = v.data == 0 ? A : v.data == 1 ? A16 : A16f;
        a.B = v.data == 0 ? B : v.data == 1 ? B16 : B16f;
        auto run_for = [&](double secs, bool sample, double* watts, double* ms_per) {
            const auto t_end = std::chrono::steady_clock::now() + std::chrono::duration<double>(secs);
            double wsum = 0;
            int wn = 0, launches = 0;
            float ms_total = 0;
            while (std::chrono::steady_clock::now() < t_end) {
                HIP_OK(hipEventRecord(e0));
                for (int i = 0; i < 40; ++i) v.launch(a, false);
                HIP_OK(hipGetLastError());
                HIP_OK(hipEventRecord(e1));
                while (hipEventQuery(e1) == hipErrorNotReady) {
                    if (sample && !power_file.empty()) {
                        const double w = read_watts(power_file);
                        if (w > 0) { wsum += w; ++wn; }
                    }
                    std::this_thread::sleep_for(std::chrono::milliseconds(2));
                }
                HIP_OK(hipEventSynchronize(e1));
                float ms;
                HIP_OK(hipEventElapsedTime(&ms, e0, e1));
                ms_total += ms;
                launches += 40;
            }
            if (watts) *watts = wn ? wsum / wn : -1.0;
            if (ms_per) *ms_per = ms_total / launches;
        };
        run_for(0.3, false, nullptr, nullptr);
        double watts = -1, ms = 0;
        run_for(seconds, true, &watts, &ms);
        // cycles per K step from the kernel's trace record, right after the timed launches
        HIP_OK(hipMemset(DB, 0xff, words * sizeof(int)));
        a.DB = DB;
        v.launch(a, true);
        HIP_OK(hipDeviceSynchronize());
        std::vector<int> db(words);
        HIP_OK(hipMemcpy(db.data(), DB, words * sizeof(int), hipMemcpyDeviceToHost));
        // record: {barrier wait, waits, cycles from kernel start to the end of the K loop, K steps,
        // cycles of the C stores, 1}
        double loop = 0, whole = 0;
        int n = 0;
        for (size_t i = 0; i + 5 < words && db[i + 5] == 1; i += 6) {
            loop += (double)db[i + 2] / db[i + 3];
            whole += (double)db[i + 2] + db[i + 4];
            ++n;
        }
        const double cyc = n ? loop / n : 0.0;
        // a CU runs tiles / CUs workgroups one after the other
        int cus = 256;
        HIP_OK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
        const double ghz = n ? (whole / n) * std::ceil((double)n / cus) / (ms * 1e-3) / 1e9 : 0.0;
        printf("%-46s %9.4f %9.0f %12.0f %7.2f %8.0f %9.3f\n", v.name, ms, flops / (ms * 1e-3) / 1e12, cyc,
               ghz, watts, watts > 0 ? watts * ms * 1e-3 : -1.0);
        fflush(stdout);
    }
    return 0;
}
