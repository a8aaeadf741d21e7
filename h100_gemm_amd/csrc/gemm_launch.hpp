// gemm_launch.hpp -- host-side launch of one kernel configuration.
#pragma once
#include <hip/hip_runtime.h>

#include "gemm_kernel.hpp"

namespace mi {

// One workgroup per output tile, Cfg::NT threads, static LDS.  Asynchronous on `stream`,
// like the launch in runKernel (matmul_h100_optimal.cu:58) / gpu_gemm
// (matmul_h100.cu.jinja:982), which return without synchronising.
template <class Cfg, bool TRACE = false>
hipError_t launch_tile_kernel(const GemmArgs& args, hipStream_t stream) {
    const int grid = args.tiles_m * args.tiles_n;
    return launch_kernel(gemm_tile_kernel<Cfg, TRACE>, dim3(grid), dim3(Cfg::NT), stream, args);
}

}  // namespace mi
