// The kernels of gmm_generic.hpp for one element type, named by -DGG_GENERIC_DT=<n>
// (0 bf16, 1 f16, 2 f8 e4m3, 3 f8 e5m2): all layouts, vector widths and both epilogues, and the
// host function that picks among them.  One translation unit per element type keeps the build
// parallel.
#include "gmm_generic.hpp"
#include "gmm_variants.hpp"

#ifndef GG_GENERIC_DT
#error "compile with -DGG_GENERIC_DT=<element type>"
#endif

namespace gg {
namespace {

constexpr int DT = GG_GENERIC_DT;

template <int LAYOUT, int VEC, int EPI>
hipError_t launch_one(const GenericParams& gp, const HostSizes& hs, int grid, hipStream_t stream) {
  hipLaunchKernelGGL((generic::gmm_generic_kernel<DT, LAYOUT, VEC, EPI>), dim3(grid),
                     dim3(generic::THREADS), 0, stream, gp, hs);
  return hipGetLastError();
}

template <int LAYOUT, int EPI>
hipError_t launch_vec(int vec, const GenericParams& gp, const HostSizes& hs, int grid, hipStream_t stream) {
  switch (vec) {
    case 8: return launch_one<LAYOUT, 8, EPI>(gp, hs, grid, stream);
    case 4: return launch_one<LAYOUT, 4, EPI>(gp, hs, grid, stream);
    case 2: return launch_one<LAYOUT, 2, EPI>(gp, hs, grid, stream);
    default: return launch_one<LAYOUT, 1, EPI>(gp, hs, grid, stream);
  }
}

hipError_t launch(int layout, int vec, int epilogue, const GenericParams& gp, const HostSizes& hs, int grid,
                  hipStream_t stream) {
  if (layout == kTN) {
    if (epilogue == kEpiSwiGLU) return hipErrorInvalidValue;
    return epilogue == kEpiAccF32 ? launch_vec<kTN, kEpiAccF32>(vec, gp, hs, grid, stream)
                                  : launch_vec<kTN, kEpiStore>(vec, gp, hs, grid, stream);
  }
  if (epilogue == kEpiAccF32) return hipErrorInvalidValue;
  if (epilogue == kEpiSwiGLU) {
    return layout == kNN ? launch_vec<kNN, kEpiSwiGLU>(vec, gp, hs, grid, stream)
                         : launch_vec<kNT, kEpiSwiGLU>(vec, gp, hs, grid, stream);
  }
  return layout == kNN ? launch_vec<kNN, kEpiStore>(vec, gp, hs, grid, stream)
                       : launch_vec<kNT, kEpiStore>(vec, gp, hs, grid, stream);
}

const GenericOps kOps = {DT, &launch};

}  // namespace

#define GG_CAT2(a, b) a##b
#define GG_CAT(a, b) GG_CAT2(a, b)
const GenericOps* GG_CAT(generic_ops_, GG_GENERIC_DT)() { return &kOps; }

}  // namespace gg
