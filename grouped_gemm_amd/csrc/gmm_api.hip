// Host side of the C ABI declared in include/grouped_gemm_hip.h: argument checks,
// kernel selection and the launches.  No torch types, no allocation, no sync.
#include "../../include/grouped_gemm_hip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "gmm_generic.hpp"
#include "gmm_variants.hpp"

namespace gg {
const GenericOps* generic_ops_0();
const GenericOps* generic_ops_1();
const GenericOps* generic_ops_2();
const GenericOps* generic_ops_3();
#define GG_VARIANT(index, DT_, LAYOUT_, SHAPE_, EPI_, INDEXED_) const VariantOps* variant_ops_##index();
#include "gmm_variants.def"
#undef GG_VARIANT
}  // namespace gg

namespace {

using gg::Short;
using gg::Wide;

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define GG_HIP(call)                                                                     \
  do {                                                                                   \
    hipError_t err__ = (call);                                                           \
    if (err__ != hipSuccess)                                                             \
      return fail(GG_EHIP, "%s failed: %s", #call, hipGetErrorString(err__));            \
  } while (0)

const gg::VariantOps* (*const kVariantGetters[])() = {
#define GG_VARIANT(index, DT_, LAYOUT_, SHAPE_, EPI_, INDEXED_) &gg::variant_ops_##index,
#include "gmm_variants.def"
#undef GG_VARIANT
};
constexpr int kNumVariants = sizeof(kVariantGetters) / sizeof(kVariantGetters[0]);

static_assert(GG_DTYPE_BF16 == gg::kBF16 && GG_DTYPE_F16 == gg::kF16 && GG_DTYPE_F8E4M3 == gg::kF8E4M3 &&
              GG_DTYPE_F8E5M2 == gg::kF8E5M2, "the header's element types are the kernels'");

const gg::GenericOps* generic_ops(int dt) {
  switch (dt) {
    case gg::kBF16: return gg::generic_ops_0();
    case gg::kF16: return gg::generic_ops_1();
    case gg::kF8E4M3: return gg::generic_ops_2();
    default: return gg::generic_ops_3();
  }
}

const gg::VariantOps* find_variant(int dt, int layout, int shape, int epilogue, int indexed) {
  for (int i = 0; i < kNumVariants; ++i) {
    const gg::VariantOps* v = kVariantGetters[i]();
    if (v->dt == dt && v->layout == layout && v->shape == shape && v->epilogue == epilogue &&
        v->indexed == indexed)
      return v;
  }
  return nullptr;
}

// Tile rows per band of the in-group tile order.  The weight-gradient layout with shallow groups
// is mostly output writes; there an odd band height measures 5-8 % faster than 4 (the bands then
// do not line up with the 32-tile runs the XCDs take, which spreads what is written at one time
// over more of the memory channels).
constexpr int kBandHeight = 4;
constexpr int kBandHeightShallow = 3;
constexpr int kShallowBelow = 1024;   // average rows per group below which the shallow height is used
constexpr int kShortBelow = 112;      // average rows per group below which the short tile shape is used

int band_height(int64_t num_groups, int64_t tokens, int trans_a) {
  return trans_a && tokens < (int64_t)kShallowBelow * num_groups ? kBandHeightShallow : kBandHeight;
}

bool use_short_shape(int64_t num_groups, int64_t tokens, int trans_a) {
  return !trans_a && num_groups > 0 && tokens < (int64_t)kShortBelow * num_groups;
}

// NN and NT layouts: whether the groups' tiles are handed out by ascending number of tile rows
// instead of in group order (the kernel still keeps the group order if it finds a group of more
// than 8 tile rows).  Where group sizes straddle a multiple of the tile height, groups of k and of
// k + 1 tile rows alternate at random; with equal groups side by side the launch is faster.
// Measured by permuting the groups, Poisson sizes, 7168 -> 2048, b stored transposed / as stored:
// 256 groups around 256 rows -3.2 / -2.3 %, 96 around 256 -4.8 / -3.6 %, 128 around 512 -1.8 /
// -2.2 %, around 768 -3.3 / -3.4 %, 64 around 1024 -1.2 / -1.6 %; around 128, 200, 320, 384, 640,
// 1536, 2048 rows within +-0.7 %; Zipf sizes with groups of up to 57 tile rows +0.8 / +1.7 %
// (hence the kernel's guard).  It pays with deep tiles only: the same 256 groups around 256 rows
// with hidden_in 4096 -2.6 / -1.9 %, 2048 +0.6 / -1.4 %, 1024 +1.6 / +0.7 %, 512 +8.9 / +7.4 %
// (the order itself, a counting sort and a second scan of the tile counts, is 5-8 us of a launch
// of 200 us there).
constexpr int kByTileRowsGroups = 32;         // at least this many groups
constexpr int kByTileRowsRowsBelow = 2048;    // ... of fewer rows than this on average
constexpr int kByTileRowsRounds = 4;          // ... at least this many rounds of tiles
constexpr int kByTileRowsDepth = 2048;        // ... and tiles at least this deep

bool order_by_tile_rows(int64_t num_groups, int64_t tokens, int64_t tiles_n, int bm, int grid, int64_t hidden_in) {
  return num_groups >= kByTileRowsGroups && tokens < (int64_t)kByTileRowsRowsBelow * num_groups &&
         hidden_in >= kByTileRowsDepth &&
         (tokens / bm + num_groups / 2) * tiles_n >= (int64_t)kByTileRowsRounds * grid;
}

// Scratch of gg_gmm_no_alloc: the workspace of gg_gmm (arrival counters, then partial tiles) as a
// static array, one copy per device that loads this library, held until the process ends.  In
// host code `scratch` is only a handle for hipGetSymbolAddress; kernels get the address that
// call returns for the current device (DeviceInfo::scratch).
static __device__ __align__(256) unsigned char scratch[GG_WORKSPACE_BYTES];

// Most workgroups a launch may have for the static scratch to hold one partial tile each.
constexpr int kStaticScratchGrid = (GG_WORKSPACE_BYTES - gg::kWsCounterBytes) / (256 * 256 * 4);

__global__ void clear_counters_kernel(int* counters) { counters[threadIdx.x] = 0; }

struct DeviceInfo {
  int cus = 0;
  bool ok = false;
  unsigned char* scratch = nullptr;   // device address of `scratch` on this device
};

// Per device, once: the architecture check and the LDS limit of every kernel variant.
int device_info(DeviceInfo* out) {
  static DeviceInfo cache[64];
  static std::mutex mu;
  int dev = 0;
  GG_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(GG_ELIMIT, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!cache[dev].ok) {
    hipDeviceProp_t prop;
    GG_HIP(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
      return fail(GG_EHIP, "this library is built for gfx950 only, device is %s", prop.gcnArchName);
    for (int i = 0; i < kNumVariants; ++i) GG_HIP(kVariantGetters[i]()->prepare());
    void* scratch_address = nullptr;
    GG_HIP(hipGetSymbolAddress(&scratch_address, HIP_SYMBOL(scratch)));
    cache[dev].scratch = static_cast<unsigned char*>(scratch_address);
    cache[dev].cus = prop.multiProcessorCount;
    cache[dev].ok = true;
  }
  *out = cache[dev];
  return GG_OK;
}

template <typename S, int LAYOUT>
int launch_dump(const gg::GmmParams& p, const gg::HostSizes& hs, hipStream_t stream) {
  hipLaunchKernelGGL((gg::schedule_dump_kernel<LAYOUT, S::BM, S::BN>), dim3(1), dim3(64), 0, stream, p, hs);
  GG_HIP(hipGetLastError());
  return GG_OK;
}

int dispatch_dump(bool short_shape, int layout, const gg::GmmParams& p, const gg::HostSizes& hs,
                  hipStream_t stream) {
  if (layout == gg::kTN) return launch_dump<Wide, gg::kTN>(p, hs, stream);
  if (short_shape) {
    return layout == gg::kNN ? launch_dump<Short, gg::kNN>(p, hs, stream)
                             : launch_dump<Short, gg::kNT>(p, hs, stream);
  }
  return layout == gg::kNN ? launch_dump<Wide, gg::kNN>(p, hs, stream)
                           : launch_dump<Wide, gg::kNT>(p, hs, stream);
}

int check_common(const int64_t* batch_sizes, int64_t num_groups, int64_t tokens, int64_t hidden_in,
                 int64_t hidden_out, int trans_a, int trans_b) {
  if (trans_a && trans_b) return fail(GG_EINVAL, "trans_a and trans_b cannot both be set");
  if (num_groups < 0 || tokens < 0 || hidden_in < 0 || hidden_out < 0)
    return fail(GG_EINVAL, "negative dimension");
  if (num_groups > 0 && batch_sizes == nullptr) return fail(GG_EINVAL, "batch_sizes is null");
  if (hidden_in >= (1 << 22) || hidden_out >= (1 << 22))
    return fail(GG_ELIMIT, "hidden sizes must be below 2^22");
  if (tokens >= (int64_t(1) << 31)) return fail(GG_ELIMIT, "tokens must be below 2^31");
  return GG_OK;
}

// Which kernels a call runs on, from its sizes, element type and the operands' alignment.
struct Route {
  uintptr_t address_bits;
  int elem_bytes;
  bool indexed;        // any row index given
  bool indexed_fits;   // ... and a and c are within reach of the streaming kernels' 32-bit offsets
  bool relaxed;        // streaming kernel on operands that are only 4-byte aligned (see classify)
  bool ragged_width;   // ... with a width that is not a multiple of 8
  bool ragged_depth;   // ... with rows along a depth that is not a multiple of 8
  bool generic;        // the kernels of gmm_generic.hpp
  int vec;             // their vector width
  int64_t a_bytes, c_bytes;
};

Route classify(const gg_gmm_args& g) {
  Route r;
  const int64_t hidden_in = g.hidden_in, hidden_out = g.hidden_out, tokens = g.tokens;
  const bool trans_a = g.trans_a != 0, trans_b = g.trans_b != 0;
  const bool swiglu = g.epilogue == GG_EPILOGUE_SWIGLU;
  r.elem_bytes = g.dtype == GG_DTYPE_F8E4M3 || g.dtype == GG_DTYPE_F8E5M2 ? 1 : 2;
  r.address_bits =
      reinterpret_cast<uintptr_t>(g.a) | reinterpret_cast<uintptr_t>(g.b) | reinterpret_cast<uintptr_t>(g.c);
  // The streaming kernels fetch and store rows 16 bytes at a time: two-byte elements, hidden sizes
  // that are multiples of 8, operands on 16-byte boundaries, rows in place.  Everything else goes
  // to the kernels of gmm_generic.hpp, VEC elements at a time.
  r.indexed = g.a_row_index != nullptr || g.b_row_index != nullptr || g.c_row_index != nullptr;
  r.a_bytes = (g.a_num_rows > 0 ? g.a_num_rows : tokens) * hidden_in * r.elem_bytes;
  r.c_bytes = (g.c_num_rows > 0 ? g.c_num_rows : tokens) * hidden_out * 2;
  // with row indices the streaming kernels address a and c through 32-bit byte offsets
  r.indexed_fits = !trans_a && r.a_bytes < (int64_t)gg::kOutOfRangeIndexed && r.c_bytes < (int64_t)gg::kOutOfRangeIndexed;
  // (fp8 streams in 16-byte chunks like the rest: 16 elements, along whichever dimension is
  // contiguous in each operand)
  const bool f8_streams = r.elem_bytes == 1 && (!swiglu || (trans_b && !r.indexed)) &&
                          (trans_a ? hidden_in % 16 == 0 && hidden_out % 16 == 0
                                   : hidden_in % 16 == 0 && (trans_b || hidden_out % 16 == 0));
  // Two-byte elements with the plain store epilogue also stream from 4-byte boundaries: a 16-byte
  // access needs no more than that, and the end of a buffer descriptor clips it dword by dword.
  // Both hidden sizes have to be even (rows then start on 4-byte boundaries).  Along the width a
  // chunk may run past the row's end: what it picks up there lands in tile columns that are never
  // stored, and a row of c whose last chunk holds 2, 4 or 6 columns is finished with narrower
  // stores.  Along the depth (rows of a, and of b stored transposed; not in the weight-gradient
  // layout, where both operands run along their widths) such a chunk would add the next row's
  // first values to the sums: a kernel variant clears them in LDS before the slice is multiplied
  // (WideRaggedDepth; plain rows only, no row indices).
  const bool aligned = hidden_in % 8 == 0 && hidden_out % 8 == 0 && (r.address_bits & 15) == 0;
  r.relaxed = !aligned && r.elem_bytes == 2 && !swiglu && !g.accumulate_f32 && (r.address_bits & 3) == 0 &&
              hidden_out % 2 == 0 && hidden_in % 2 == 0;
  r.ragged_width = r.relaxed && hidden_out % 8 != 0;
  r.ragged_depth = !trans_a && hidden_in % 8 != 0;
  if (r.ragged_depth && r.indexed) r.relaxed = false;
  r.ragged_depth = r.ragged_depth && r.relaxed;
  r.generic = !r.relaxed &&
              ((r.elem_bytes != 2 && !f8_streams) || hidden_in % 8 != 0 || hidden_out % 8 != 0 ||
               (r.address_bits & 15));
  r.generic = r.generic || (r.indexed && !r.indexed_fits);
  r.vec = 8;
  if (r.generic) {
    while (r.vec > 1 && (hidden_in % r.vec != 0 || hidden_out % r.vec != 0 ||
                         (r.address_bits & (uintptr_t)(r.vec * 2 - 1))))
      r.vec >>= 1;
  }
  return r;
}

// Rows of a, b and c in memory, the bounds a row index is held against: an index that names no
// row is a missing row (zeros on the way in, nothing stored on the way out) on every kernel.
struct IndexedRows {
  int64_t a, b, c;
};

IndexedRows indexed_rows(const gg_gmm_args& g) {
  IndexedRows r;
  r.a = g.a_num_rows > 0 ? g.a_num_rows : g.tokens;
  r.b = g.b_num_rows > 0 ? g.b_num_rows : g.tokens;
  r.c = g.c_num_rows > 0 ? g.c_num_rows : g.tokens;
  return r;
}

// static_scratch: use the device's static scratch array as the workspace (gg_gmm_no_alloc).
int gmm_impl(const gg_gmm_args& g, bool static_scratch = false) {
  const int64_t num_groups = g.num_groups, tokens = g.tokens;
  const int64_t hidden_in = g.hidden_in, hidden_out = g.hidden_out;
  const int trans_a = g.trans_a != 0, trans_b = g.trans_b != 0;
  const bool out_f32 = g.accumulate_f32 != 0;
  int rc = check_common(g.batch_sizes, num_groups, tokens, hidden_in, hidden_out, trans_a, trans_b);
  if (rc != GG_OK) return rc;
  if (g.dtype < GG_DTYPE_BF16 || g.dtype > GG_DTYPE_F8E5M2)
    return fail(GG_EINVAL, "dtype must be one of GG_DTYPE_*");
  const int elem_bytes = g.dtype == GG_DTYPE_F8E4M3 || g.dtype == GG_DTYPE_F8E5M2 ? 1 : 2;
  if (g.epilogue != GG_EPILOGUE_NONE && g.epilogue != GG_EPILOGUE_SWIGLU)
    return fail(GG_EINVAL, "epilogue must be one of GG_EPILOGUE_*");
  const bool swiglu = g.epilogue == GG_EPILOGUE_SWIGLU;
  if (swiglu && (trans_a || out_f32))
    return fail(GG_EINVAL, "the SwiGLU epilogue is for the layouts with a row of c per token and a c of the element type");
  if (swiglu && hidden_in * hidden_out >= (int64_t(1) << 28))
    return fail(GG_ELIMIT, "hidden_in * hidden_out must be below 2^28 with the SwiGLU epilogue");
  if (g.a_num_rows < 0 || g.b_num_rows < 0 || g.c_num_rows < 0) return fail(GG_EINVAL, "negative row count");
  if (trans_a && g.c_row_index != nullptr)
    return fail(GG_EINVAL, "c_row_index scatters output rows; the trans_a output has none per token");
  if (!trans_a && g.b_row_index != nullptr)
    return fail(GG_EINVAL, "b_row_index gathers rows of b; only the trans_a layout has a row per token in b");
  if (out_f32 && !trans_a)
    return fail(GG_EINVAL, "the fp32-accumulated output exists for the trans_a layout only");
  if (out_f32 && (hidden_in >= (1 << 20) || hidden_out >= (1 << 20)))
    return fail(GG_ELIMIT, "hidden sizes must be below 2^20 for the accumulating form");
  if (num_groups == 0) return GG_OK;
  // nothing to write
  if (hidden_out == 0 || (trans_a ? hidden_in == 0 : tokens == 0)) return GG_OK;
  if (g.c == nullptr) return fail(GG_EINVAL, "c is null");
  if (tokens > 0 && (g.a == nullptr || g.b == nullptr)) return fail(GG_EINVAL, "a or b is null");
  const Route route = classify(g);
  const uintptr_t address_bits = route.address_bits;
  if (address_bits & (uintptr_t)(elem_bytes - 1) || reinterpret_cast<uintptr_t>(g.c) & (out_f32 ? 3 : 1))
    return fail(GG_ELIMIT, "a, b and c must be aligned to their element size");
  const bool indexed = route.indexed, indexed_fits = route.indexed_fits, generic = route.generic;
  const int64_t a_bytes = route.a_bytes, c_bytes = route.c_bytes;
  const int vec = route.vec;

  // Host-resident sizes are validated here; they travel in the kernel argument block.
  if (!g.batch_sizes_on_device) {
    int64_t row = 0;
    for (int64_t e = 0; e < num_groups; ++e) {
      if (g.batch_sizes[e] < 0) return fail(GG_EINVAL, "batch_sizes[%lld] is negative", (long long)e);
      if (g.batch_sizes[e] > tokens - row)
        return fail(GG_EINVAL, "batch_sizes sum past the %lld rows of a", (long long)tokens);
      row += g.batch_sizes[e];
    }
  }

  DeviceInfo info;
  rc = device_info(&info);
  if (rc != GG_OK) return rc;
  hipStream_t stream = static_cast<hipStream_t>(g.stream);
  const int layout = trans_a ? gg::kTN : (trans_b ? gg::kNT : gg::kNN);
  const int epilogue = out_f32 ? gg::kEpiAccF32 : (swiglu ? gg::kEpiSwiGLU : gg::kEpiStore);
  // deep groups: the launch is bound by the matrix pipe, and atomic additions to c cost less of
  // its time than reading, adding and writing; shallow groups: bound by the traffic of c, the reverse
  const int variant_epilogue = out_f32 && tokens >= (int64_t)kShallowBelow * num_groups ? gg::kEpiAccF32Atomic : epilogue;
  // (the short tile shape exists for two-byte elements, the plain epilogue and rows in place only)
  const bool short_shape = !generic && !swiglu && !indexed && elem_bytes == 2 && !route.ragged_depth &&
                           use_short_shape(num_groups, tokens, trans_a);
  const int bm = generic ? gg::kGenericTileM : (short_shape ? Short::BM : Wide::BM);
  // output columns per tile: half the tile's width when it holds gate and up columns
  const int bn = (generic ? gg::kGenericTileN : (short_shape ? Short::BN : Wide::BN)) / (swiglu ? 2 : 1);
  const gg::VariantOps* variant = nullptr;
  if (!generic) {
    const int shape = route.ragged_depth ? gg::WideRaggedDepth::kId : (short_shape ? Short::kId : Wide::kId);
    variant = find_variant(g.dtype, layout, shape, variant_epilogue, indexed ? 1 : 0);
    if (variant == nullptr) return fail(GG_EINVAL, "no kernel for this combination of arguments");
  }

  gg::GmmParams p{};
  p.a = static_cast<const char*>(g.a);
  p.b = static_cast<const char*>(g.b);
  p.c = static_cast<char*>(g.c);
  p.tokens = tokens;
  p.hidden_in = (int32_t)hidden_in;
  p.hidden_out = (int32_t)hidden_out;
  p.b_cols = (int32_t)(swiglu ? 2 * hidden_out : hidden_out);
  p.a_rows = g.a_row_index;
  p.c_rows = g.c_row_index;
  static_assert(GG_STATUS_NEGATIVE_SIZE == gg::kStatusNegativeSize && GG_STATUS_ROWS_PAST_END == gg::kStatusRowsPastEnd,
                "the header's status bits are the kernel's");
  p.status = g.batch_sizes_on_device ? g.size_status : nullptr;
  p.a_bytes = (uint32_t)(indexed_fits ? a_bytes : 0);
  p.c_bytes = (uint32_t)(indexed_fits ? c_bytes : 0);
  const IndexedRows index_rows = indexed_rows(g);
  p.a_index_rows = (uint32_t)(indexed_fits ? index_rows.a : 0);
  p.c_index_rows = (uint32_t)(indexed_fits ? index_rows.c : 0);
  p.group_m = band_height(num_groups, tokens, trans_a);
  static_assert(GG_FLAG_WHOLE_TILES == gg::kFlagWholeTiles && GG_FLAG_ONE_CLASS == gg::kFlagOneClass &&
                GG_FLAG_ROW_PIECES == gg::kFlagRowPieces && GG_FLAG_GROUP_ORDER == gg::kFlagGroupOrder,
                "the header's flags are the kernel's");
  p.flags = g.flags & (GG_FLAG_WHOLE_TILES | GG_FLAG_ONE_CLASS | GG_FLAG_ROW_PIECES | GG_FLAG_GROUP_ORDER);
  // (ragged widths: the fix-up of depth pieces stores 4 columns at a time; ragged depths: the
  // kernel looks for the ragged chunks in the slice hidden_in / 64 of tiles that start at depth 0.
  // Whole tiles and row pieces only, for both.)
  const bool no_depth_pieces = route.ragged_width || route.ragged_depth;
  p.sched_out = nullptr;
  if (static_scratch) {
    if (g.workspace != nullptr)
      return fail(GG_EINVAL, "gg_gmm_no_alloc brings its own scratch: workspace must be NULL");
    if (info.cus > kStaticScratchGrid)
      return fail(GG_ELIMIT, "the static scratch serves launches of up to %d workgroups, this device has %d "
                  "compute units", kStaticScratchGrid, info.cus);
    p.workspace = reinterpret_cast<char*>(info.scratch);
    p.ws_slots = (int32_t)(((uint64_t)GG_WORKSPACE_BYTES - gg::kWsCounterBytes) /
                           ((uint64_t)bm * bn * (swiglu ? 2 : 1) * 4));
    if (p.ws_slots > 1024) p.ws_slots = 1024;
    if (no_depth_pieces) p.ws_slots = 0;
    // Every call on this device shares the array and finds what the last call left: the arrival
    // counters must start at zero (a fill kernel, not a memset: callers may be capturing a graph).
    hipLaunchKernelGGL(clear_counters_kernel, dim3(1), dim3(gg::kWsCounterBytes / 4), 0, stream,
                       reinterpret_cast<int*>(info.scratch));
    GG_HIP(hipGetLastError());
  } else if (g.workspace != nullptr && !generic && !no_depth_pieces) {
    if (reinterpret_cast<uintptr_t>(g.workspace) & 255)
      return fail(GG_ELIMIT, "the workspace must be 256-byte aligned");
    const uint64_t slot_bytes = (uint64_t)bm * bn * (swiglu ? 2 : 1) * 4;
    if (g.workspace_bytes < gg::kWsCounterBytes + slot_bytes)
      return fail(GG_ELIMIT, "the workspace holds %llu bytes, the smallest useful one %llu",
                  (unsigned long long)g.workspace_bytes, (unsigned long long)(gg::kWsCounterBytes + slot_bytes));
    const uint64_t slots = (g.workspace_bytes - gg::kWsCounterBytes) / slot_bytes;
    p.workspace = static_cast<char*>(g.workspace);
    // one arrival counter per tile of the last round: at most grid / 2 of them, 1024 fit
    p.ws_slots = slots > 1024 ? 1024 : (int32_t)slots;
  }

  const int64_t tiles_n = (hidden_out + bn - 1) / bn;
  const int64_t tiles_m_fixed = (hidden_in + bm - 1) / bm;   // weight-gradient layout
  // At most GG_MAX_GROUPS_PER_LAUNCH groups per launch.  A launch sees all operands and the rows
  // its groups start at: handed over by the host for host-resident sizes, summed up by the kernel
  // itself from the sizes of the groups before it for device-resident ones.
  int64_t row = 0;
  for (int64_t first = 0; first < num_groups; first += GG_MAX_GROUPS_PER_LAUNCH) {
    const int64_t count = num_groups - first < GG_MAX_GROUPS_PER_LAUNCH
                              ? num_groups - first : GG_MAX_GROUPS_PER_LAUNCH;
    gg::HostSizes hs;
    p.first_group = (int32_t)first;
    p.num_groups = (int32_t)count;
    int64_t tiles;
    if (g.batch_sizes_on_device) {
      p.sizes_dev = g.batch_sizes;
      p.row_base = 0;
      // upper bound for any size vector (the device clips rows to `tokens`)
      tiles = trans_a ? count * tiles_m_fixed * tiles_n : (tokens / bm + count) * tiles_n;
    } else {
      p.sizes_dev = nullptr;
      p.row_base = row;
      tiles = 0;
      for (int64_t i = 0; i < count; ++i) {
        const int64_t m = g.batch_sizes[first + i];
        hs.v[i] = (int32_t)m;
        row += m;
        tiles += trans_a ? tiles_m_fixed * tiles_n : ((m + bm - 1) / bm) * tiles_n;
      }
    }
    if (tiles >= (int64_t(1) << 31)) return fail(GG_ELIMIT, "too many output tiles for one launch");
    if (tiles == 0) continue;
    p.flags &= ~gg::kFlagByTileRows;
    if (!generic && !trans_a && !(p.flags & gg::kFlagGroupOrder) && count >= kByTileRowsGroups &&
        order_by_tile_rows(num_groups, tokens, tiles_n, bm, info.cus, hidden_in))
      p.flags |= gg::kFlagByTileRows;
    // the full grid also for few tiles: the last round's tiles may be cut into pieces for
    // the workgroups that would otherwise idle
    if (generic) {
      gg::GenericParams gp;
      gp.p = p;
      gp.p.workspace = nullptr;
      gp.p.ws_slots = 0;
      gp.a_rows = g.a_row_index;
      gp.b_rows = g.b_row_index;
      gp.c_rows = g.c_row_index;
      gp.a_num_rows = index_rows.a;
      gp.b_num_rows = index_rows.b;
      gp.c_num_rows = index_rows.c;
      // light workgroups (28 KiB of LDS): two per compute unit
      const int64_t grid = tiles < 2 * info.cus ? tiles : 2 * info.cus;
      GG_HIP(generic_ops(g.dtype)->launch(layout, vec, epilogue, gp, hs, (int)grid, stream));
    } else {
      GG_HIP(variant->launch(p, hs, info.cus, stream));
    }
  }
  return GG_OK;
}

}  // namespace

extern "C" {

const char* gg_last_error(void) { return g_err; }

int gg_version(void) { return 200; }

int gg_init(void) {
  DeviceInfo info;
  return device_info(&info);
}

int gg_tile_shape(int64_t num_groups, int64_t tokens, int trans_a, int trans_b, int* bm, int* bn,
                  int* bk) {
  if (trans_a && trans_b) return fail(GG_EINVAL, "trans_a and trans_b cannot both be set");
  const bool s = use_short_shape(num_groups, tokens, trans_a);
  if (bm) *bm = s ? Short::BM : Wide::BM;
  if (bn) *bn = s ? Short::BN : Wide::BN;
  if (bk) *bk = gg::BK;
  return GG_OK;
}

int gg_gmm(const gg_gmm_args* args) {
  if (args == nullptr) return fail(GG_EINVAL, "args is null");
  if (args->struct_bytes != sizeof(gg_gmm_args))
    return fail(GG_EINVAL, "gg_gmm_args.struct_bytes is %u, this library expects %zu", args->struct_bytes,
                sizeof(gg_gmm_args));
  return gmm_impl(*args);
}

uint64_t gg_workspace_bytes_for(const gg_gmm_args* args) {
  if (args == nullptr || args->struct_bytes != sizeof(gg_gmm_args)) return 0;
  const gg_gmm_args& g = *args;
  if (g.dtype < GG_DTYPE_BF16 || g.dtype > GG_DTYPE_F8E5M2 || g.hidden_in <= 0 || g.hidden_out <= 0) return 0;
  const Route r = classify(g);
  // (the kernels never cut tiles that are combined or scattered on their way out along the depth)
  // (the fix-up of depth pieces stores 4 columns at a time: whole tiles and row pieces for ragged widths)
  if (r.generic || r.ragged_width || r.ragged_depth || r.indexed || g.epilogue == GG_EPILOGUE_SWIGLU) return 0;
  if (g.flags & (GG_FLAG_WHOLE_TILES | GG_FLAG_ROW_PIECES)) return 0;
  {
    const int64_t slice = r.elem_bytes == 1 ? 2 * gg::BK : gg::BK;   // depth elements per slice
    // (weight-gradient layout: the depth is a group's row count, and one group may hold all rows:
    // the kernel cuts the tiles of groups much deeper than the rest, plan_deep_tiles)
    const int64_t depth = g.trans_a ? g.tokens : g.hidden_in;
    if ((depth + slice - 1) / slice < 2 * gg::kMinSlicesPerPiece) return 0;
  }
  return GG_WORKSPACE_BYTES;
}

int gg_gmm_no_alloc(const gg_gmm_args* args) {
  if (args == nullptr) return fail(GG_EINVAL, "args is null");
  if (args->struct_bytes != sizeof(gg_gmm_args))
    return fail(GG_EINVAL, "gg_gmm_args.struct_bytes is %u, this library expects %zu", args->struct_bytes,
                sizeof(gg_gmm_args));
  return gmm_impl(*args, /*static_scratch=*/true);
}

int gg_gmm_bf16(const void* a, const void* b, void* c, const int64_t* batch_sizes,
                int batch_sizes_on_device, int64_t num_groups, int64_t tokens, int64_t hidden_in,
                int64_t hidden_out, int trans_a, int trans_b, void* stream) {
  gg_gmm_args g{};
  g.struct_bytes = sizeof(g);
  g.dtype = GG_DTYPE_BF16;
  g.a = a, g.b = b, g.c = c;
  g.batch_sizes = batch_sizes, g.batch_sizes_on_device = batch_sizes_on_device;
  g.num_groups = num_groups, g.tokens = tokens, g.hidden_in = hidden_in, g.hidden_out = hidden_out;
  g.trans_a = trans_a, g.trans_b = trans_b;
  g.stream = stream;
  return gmm_impl(g);
}

int gg_gmm_bf16_acc_f32(const void* a, const void* b, float* c, const int64_t* batch_sizes,
                        int batch_sizes_on_device, int64_t num_groups, int64_t tokens,
                        int64_t hidden_in, int64_t hidden_out, void* stream) {
  gg_gmm_args g{};
  g.struct_bytes = sizeof(g);
  g.dtype = GG_DTYPE_BF16;
  g.a = a, g.b = b, g.c = c;
  g.batch_sizes = batch_sizes, g.batch_sizes_on_device = batch_sizes_on_device;
  g.num_groups = num_groups, g.tokens = tokens, g.hidden_in = hidden_in, g.hidden_out = hidden_out;
  g.trans_a = 1, g.accumulate_f32 = 1;
  g.stream = stream;
  return gmm_impl(g);
}

int gg_debug_schedule(const int64_t* batch_sizes, int batch_sizes_on_device, int64_t num_groups,
                      int64_t tokens, int64_t hidden_in, int64_t hidden_out, int trans_a,
                      int trans_b, int64_t* table_out, void* stream_) {
  int rc = check_common(batch_sizes, num_groups, tokens, hidden_in, hidden_out, trans_a, trans_b);
  if (rc != GG_OK) return rc;
  if (num_groups > GG_MAX_GROUPS_PER_LAUNCH)
    return fail(GG_ELIMIT, "at most %d groups per schedule", GG_MAX_GROUPS_PER_LAUNCH);
  if (num_groups == 0) return GG_OK;
  if (table_out == nullptr) return fail(GG_EINVAL, "table_out is null");
  DeviceInfo info;
  rc = device_info(&info);
  if (rc != GG_OK) return rc;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  gg::GmmParams p{};
  p.tokens = tokens;
  p.hidden_in = (int32_t)hidden_in;
  p.hidden_out = (int32_t)hidden_out;
  p.group_m = band_height(num_groups, tokens, trans_a);
  p.num_groups = (int32_t)num_groups;
  p.b_cols = (int32_t)hidden_out;
  p.sched_out = table_out;
  const int layout = trans_a ? gg::kTN : (trans_b ? gg::kNT : gg::kNN);
  const bool short_shape = use_short_shape(num_groups, tokens, trans_a);
  {
    const int bm = short_shape ? Short::BM : Wide::BM, bn = short_shape ? Short::BN : Wide::BN;
    if (!trans_a && num_groups >= kByTileRowsGroups &&
        order_by_tile_rows(num_groups, tokens, (hidden_out + bn - 1) / bn, bm, info.cus, hidden_in))
      p.flags |= gg::kFlagByTileRows;
  }
  gg::HostSizes hs;
  if (batch_sizes_on_device) {
    p.sizes_dev = batch_sizes;
  } else {
    // the table shows what the kernel would do with these sizes: clamped like device-resident ones
    for (int64_t i = 0; i < num_groups; ++i) {
      const int64_t v = batch_sizes[i];
      hs.v[i] = (int32_t)(v < 0 ? 0 : (v > tokens ? tokens : v));
    }
  }
  return dispatch_dump(short_shape, layout, p, hs, stream);
}

}  // extern "C"
