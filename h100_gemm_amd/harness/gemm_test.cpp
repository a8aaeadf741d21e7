// gemm_test.cpp -- the `./test M m N n K k` program of the reference
// (main() of matmul_h100.cu.jinja:987-1079) over libmi_gemm.so: the kernel is whatever the
// library's dispatch (or `cfg <index|name>`) selects.  See test_main.hpp for the flow and
// the extra keys.
#include "test_main.hpp"

int main(int argc, char** argv) {
    test_epilogue().supported = true;
    TestLaunchFn launch = [](int dtype, int config, int M, int N, int K, const void* A, const void* B, void* C) {
        const TestEpilogue& ep = test_epilogue();
        if (ep.alpha == 1.0f && ep.beta == 0.0f && ep.c_layout == MI_C_ROW_MAJOR)
            MI_CHECK(mi_gemm_ex(config, dtype, M, N, K, A, B, C, nullptr, nullptr));
        else
            MI_CHECK(mi_gemm_epilogue(config, dtype, M, N, K, A, B, C, ep.alpha, ep.beta, ep.c_layout, nullptr));
    };
    auto label = [](int config) { return std::string(config == MI_CONFIG_AUTO ? "auto" : mi_gemm_config_name(config)); };
    auto parse = [](const char* value) {
        char* end = nullptr;
        long idx = std::strtol(value, &end, 10);
        int config = (end && *end == 0) ? (int)idx : mi_gemm_find_config(value);
        return (config < 0 || config >= mi_gemm_num_configs()) ? -1 : config;
    };
    return test_main(argc, argv, launch, label, parse);
}
