// One kernel variant of the library: the instantiation of gmm_kernel named by
// -DGG_VARIANT_INDEX=<n> (an index of gmm_variants.def) and the two host functions that prepare
// and launch it.  One translation unit per variant keeps the build parallel.
#include "gmm_variants.hpp"

#ifndef GG_VARIANT_INDEX
#error "compile with -DGG_VARIANT_INDEX=<index of gmm_variants.def>"
#endif

namespace gg {
namespace {

template <int INDEX>
struct VariantDef;
#define GG_VARIANT(index, DT_, LAYOUT_, SHAPE_, EPI_, INDEXED_)                          \
  template <>                                                                            \
  struct VariantDef<index> {                                                             \
    static constexpr int DT = DT_, LAYOUT = LAYOUT_, EPI = EPI_;                         \
    static constexpr bool INDEXED = INDEXED_;                                            \
    using Shape = SHAPE_;                                                                \
  };
#include "gmm_variants.def"
#undef GG_VARIANT

using V = VariantDef<GG_VARIANT_INDEX>;
using S = V::Shape;
using Cfg = GmmConfig<V::LAYOUT, S::BM, S::BN, BK, STAGES, S::WAVES_M, S::WAVES_N>;

const void* kernel_address() {
  return reinterpret_cast<const void*>(
      &gmm_kernel<V::DT, V::LAYOUT, S::BM, S::BN, BK, STAGES, S::WAVES_M, S::WAVES_N, V::EPI, V::INDEXED,
                  S::RAGGED_DEPTH>);
}

hipError_t prepare() {
  return hipFuncSetAttribute(kernel_address(), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
}

hipError_t launch(const GmmParams& p, const HostSizes& hs, int grid, hipStream_t stream) {
  GmmParams params = p;
  HostSizes sizes = hs;
  void* args[2] = {&params, &sizes};
  return hipLaunchKernel(kernel_address(), dim3(grid), dim3(S::WAVES_M * S::WAVES_N * 64), args,
                         Cfg::LDS_BYTES, stream);
}

const VariantOps kOps = {V::DT, V::LAYOUT, S::kId, V::EPI, V::INDEXED ? 1 : 0, Cfg::LDS_BYTES, &prepare, &launch};

}  // namespace

#define GG_CAT2(a, b) a##b
#define GG_CAT(a, b) GG_CAT2(a, b)
const VariantOps* GG_CAT(variant_ops_, GG_VARIANT_INDEX)() { return &kOps; }

}  // namespace gg
