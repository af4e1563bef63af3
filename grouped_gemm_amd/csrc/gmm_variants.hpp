// What the host side (gmm_api.hip) and the kernel translation units (gmm_variant.hip) share:
// tile shapes, epilogue kinds and the table entry through which a variant is prepared and launched.
#pragma once

#include <hip/hip_runtime.h>

#include "gmm_kernel.hpp"

namespace gg {

constexpr int BK = 64, STAGES = 2;

// Tile shapes.  Wide: 256 x 256 outputs per workgroup, 2 x 2 waves of 128 x 128.  Short: 128 x 256,
// 1 x 4 waves of 128 x 64, for calls whose groups average few rows: with at most 128 rows per
// group all four waves then share the rows instead of two of them idling (measured 4-7 % faster
// below about 100 rows per group, slower from 128 on).  The weight-gradient layout always uses the
// wide shape: its ragged dimension is the depth, not the rows.
struct Wide {
  static constexpr int kId = 0, BM = 256, BN = 256, WAVES_M = 2, WAVES_N = 2;
  static constexpr bool RAGGED_DEPTH = false;
};
struct Short {
  static constexpr int kId = 1, BM = 128, BN = 256, WAVES_M = 1, WAVES_N = 4;
  static constexpr bool RAGGED_DEPTH = false;
};
// The wide shape for a hidden_in that is even but no multiple of 8, in the layouts whose rows run
// along the depth: the kernel then clears, in LDS, what the last 16-byte chunk of a row picks up
// from the next row (DepthMajor::clear_depth_tail), and cuts no tile along the depth.
struct WideRaggedDepth : Wide {
  static constexpr int kId = 2;
  static constexpr bool RAGGED_DEPTH = true;
};

struct VariantOps {
  int dt, layout, shape, epilogue, indexed;
  int lds_bytes;
  // raises the kernel's dynamic LDS limit on the current device
  hipError_t (*prepare)();
  hipError_t (*launch)(const GmmParams& p, const HostSizes& hs, int grid, hipStream_t stream);
};

// The kernels of gmm_generic.hpp for one element type (gmm_generic_variant.hip).
struct GenericParams;
struct GenericOps {
  int dt;
  hipError_t (*launch)(int layout, int vec, int epilogue, const GenericParams& gp, const HostSizes& hs,
                       int grid, hipStream_t stream);
};

constexpr int kGenericTileM = 128, kGenericTileN = 128;
constexpr int kNumElementTypes = 4;   // bf16, f16, f8 e4m3, f8 e5m2

}  // namespace gg
