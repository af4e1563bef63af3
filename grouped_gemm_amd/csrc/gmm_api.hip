// Host side of the C ABI declared in include/grouped_gemm_hip.h: argument checks,
// kernel selection and the single launch.  No torch types, no allocation, no sync.
#include "../../include/grouped_gemm_hip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "gmm_kernel.hpp"

namespace {

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

// Tile shapes.  Wide: 256 x 256 outputs per workgroup, 2 x 2 waves of 128 x 128.  Short: 128 x 256,
// 1 x 4 waves of 128 x 64, for calls whose groups average few rows: with at most 128 rows per
// group all four waves then share the rows instead of two of them idling (measured 4-7 % faster
// below about 100 rows per group, slower from 128 on).  The weight-gradient layout always uses the
// wide shape: its ragged dimension is the depth, not the rows.
#ifndef GG_GROUP_M
#define GG_GROUP_M 4
#endif
// The weight-gradient layout with shallow groups is mostly output writes; there an odd band
// height measures 5-8 % faster than 4 (the bands then do not line up with the 32-tile runs the
// XCDs take, which spreads what is written at one time over more of the memory channels).
#ifndef GG_GROUP_M_SHALLOW
#define GG_GROUP_M_SHALLOW 3
#endif
#ifndef GG_SHALLOW_BELOW
#define GG_SHALLOW_BELOW 1024   // average rows per group below which GG_GROUP_M_SHALLOW is used
#endif
#ifndef GG_SHORT_BELOW
#define GG_SHORT_BELOW 112   // average rows per group below which the short shape is used
#endif
constexpr int BK = 64, STAGES = 2;
struct Wide {
  static constexpr int BM = 256, BN = 256, WAVES_M = 2, WAVES_N = 2;
};
struct Short {
  static constexpr int BM = 128, BN = 256, WAVES_M = 1, WAVES_N = 4;
};

// GG_TAIL_SPLIT=0 in the environment keeps the tiles of the last round whole (read at every call).
int tail_split() {
  const char* e = getenv("GG_TAIL_SPLIT");
  return e != nullptr && e[0] == '0' ? 0 : 1;
}

int band_height(int64_t num_groups, int64_t tokens, int trans_a) {
  return trans_a && tokens < (int64_t)GG_SHALLOW_BELOW * num_groups ? GG_GROUP_M_SHALLOW : GG_GROUP_M;
}

bool use_short_shape(int64_t num_groups, int64_t tokens, int trans_a) {
  return !trans_a && num_groups > 0 && tokens < (int64_t)GG_SHORT_BELOW * num_groups;
}

struct DeviceInfo {
  int cus = 0;
  bool ok = false;
};

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
    cache[dev].cus = prop.multiProcessorCount;
    cache[dev].ok = true;
  }
  *out = cache[dev];
  return GG_OK;
}

template <typename S, int LAYOUT, bool HOST_SIZES, bool ACC_F32 = false>
int launch(const gg::GmmParams& p, const gg::HostSizes* hs, int grid, hipStream_t stream) {
  using Cfg = gg::GmmConfig<LAYOUT, S::BM, S::BN, BK, STAGES, S::WAVES_M, S::WAVES_N>;
  constexpr int kThreads = S::WAVES_M * S::WAVES_N * 64;
  const void* kernel = reinterpret_cast<const void*>(
      &gg::gmm_kernel<LAYOUT, S::BM, S::BN, BK, STAGES, S::WAVES_M, S::WAVES_N, HOST_SIZES, ACC_F32>);
  // raising the dynamic LDS limit is per device and per kernel; do it once each
  static std::mutex mu;
  static bool done[64] = {};
  int dev = 0;
  GG_HIP(hipGetDevice(&dev));
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!done[dev]) {
      GG_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                 Cfg::LDS_BYTES));
      done[dev] = true;
    }
  }
  gg::GmmParams params = p;
  gg::HostSizes sizes_arg;
  gg::NoSizes no_sizes;
  void* args[2];
  args[0] = &params;
  if constexpr (HOST_SIZES) {
    sizes_arg = *hs;
    args[1] = &sizes_arg;
  } else {
    args[1] = &no_sizes;
  }
  GG_HIP(hipLaunchKernel(kernel, dim3(grid), dim3(kThreads), args, Cfg::LDS_BYTES, stream));
  return GG_OK;
}

template <typename S, int LAYOUT, bool HOST_SIZES>
int launch_dump(const gg::GmmParams& p, const gg::HostSizes* hs, hipStream_t stream) {
  auto kernel = gg::schedule_dump_kernel<LAYOUT, S::BM, S::BN, HOST_SIZES>;
  if constexpr (HOST_SIZES) {
    hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, stream, p, *hs);
  } else {
    hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, stream, p, gg::NoSizes{});
  }
  GG_HIP(hipGetLastError());
  return GG_OK;
}

// out_f32: the accumulating form (weight-gradient layout only).
template <bool HOST_SIZES>
int dispatch(bool short_shape, int layout, bool out_f32, const gg::GmmParams& p, const gg::HostSizes* hs,
             int grid, hipStream_t stream) {
  if (out_f32) return launch<Wide, gg::kTN, HOST_SIZES, true>(p, hs, grid, stream);
  if (layout == gg::kTN) return launch<Wide, gg::kTN, HOST_SIZES>(p, hs, grid, stream);
  if (short_shape) {
    return layout == gg::kNN ? launch<Short, gg::kNN, HOST_SIZES>(p, hs, grid, stream)
                             : launch<Short, gg::kNT, HOST_SIZES>(p, hs, grid, stream);
  }
  return layout == gg::kNN ? launch<Wide, gg::kNN, HOST_SIZES>(p, hs, grid, stream)
                           : launch<Wide, gg::kNT, HOST_SIZES>(p, hs, grid, stream);
}

template <bool HOST_SIZES>
int dispatch_dump(bool short_shape, int layout, const gg::GmmParams& p, const gg::HostSizes* hs,
                  hipStream_t stream) {
  if (layout == gg::kTN) return launch_dump<Wide, gg::kTN, HOST_SIZES>(p, hs, stream);
  if (short_shape) {
    return layout == gg::kNN ? launch_dump<Short, gg::kNN, HOST_SIZES>(p, hs, stream)
                             : launch_dump<Short, gg::kNT, HOST_SIZES>(p, hs, stream);
  }
  return layout == gg::kNN ? launch_dump<Wide, gg::kNN, HOST_SIZES>(p, hs, stream)
                           : launch_dump<Wide, gg::kNT, HOST_SIZES>(p, hs, stream);
}

int check_common(const int64_t* batch_sizes, int64_t num_groups, int64_t tokens, int64_t hidden_in,
                 int64_t hidden_out, int trans_a, int trans_b) {
  if (trans_a && trans_b) return fail(GG_EINVAL, "trans_a and trans_b cannot both be set");
  if (num_groups < 0 || tokens < 0 || hidden_in < 0 || hidden_out < 0)
    return fail(GG_EINVAL, "negative dimension");
  if (num_groups > 0 && batch_sizes == nullptr) return fail(GG_EINVAL, "batch_sizes is null");
  if (hidden_in % 8 != 0 || hidden_out % 8 != 0)
    return fail(GG_ELIMIT, "hidden_in (%lld) and hidden_out (%lld) must be multiples of 8",
                (long long)hidden_in, (long long)hidden_out);
  if (hidden_in >= (1 << 22) || hidden_out >= (1 << 22))
    return fail(GG_ELIMIT, "hidden sizes must be below 2^22");
  if (tokens >= (int64_t(1) << 31)) return fail(GG_ELIMIT, "tokens must be below 2^31");
  return GG_OK;
}

// Upper bound of the tile count for any size vector (the device clips rows to `tokens`).
int64_t tile_bound(int64_t num_groups, int64_t tokens, int64_t hidden_in, int64_t hidden_out,
                   int trans_a, int bm, int bn) {
  const int64_t tiles_n = (hidden_out + bn - 1) / bn;
  if (trans_a) return num_groups * ((hidden_in + bm - 1) / bm) * tiles_n;
  return (tokens / bm + num_groups) * tiles_n;
}

int gmm_impl(const void* a, const void* b, void* c, bool out_f32, const int64_t* batch_sizes,
             int batch_sizes_on_device, int64_t num_groups, int64_t tokens, int64_t hidden_in,
             int64_t hidden_out, int trans_a, int trans_b, void* stream_);

}  // namespace

extern "C" {

const char* gg_last_error(void) { return g_err; }

int gg_version(void) { return 100; }

int gg_tile_shape(int64_t num_groups, int64_t tokens, int trans_a, int trans_b, int* bm, int* bn,
                  int* bk) {
  if (trans_a && trans_b) return fail(GG_EINVAL, "trans_a and trans_b cannot both be set");
  const bool s = use_short_shape(num_groups, tokens, trans_a);
  if (bm) *bm = s ? Short::BM : Wide::BM;
  if (bn) *bn = s ? Short::BN : Wide::BN;
  if (bk) *bk = BK;
  return GG_OK;
}

int gg_gmm_bf16(const void* a, const void* b, void* c, const int64_t* batch_sizes,
                int batch_sizes_on_device, int64_t num_groups, int64_t tokens, int64_t hidden_in,
                int64_t hidden_out, int trans_a, int trans_b, void* stream_) {
  return gmm_impl(a, b, c, /*out_f32=*/false, batch_sizes, batch_sizes_on_device, num_groups, tokens,
                  hidden_in, hidden_out, trans_a, trans_b, stream_);
}

int gg_gmm_bf16_acc_f32(const void* a, const void* b, float* c, const int64_t* batch_sizes,
                        int batch_sizes_on_device, int64_t num_groups, int64_t tokens,
                        int64_t hidden_in, int64_t hidden_out, void* stream_) {
  if (hidden_in >= (1 << 20) || hidden_out >= (1 << 20))
    return fail(GG_ELIMIT, "hidden sizes must be below 2^20 for the accumulating form");
  return gmm_impl(a, b, c, /*out_f32=*/true, batch_sizes, batch_sizes_on_device, num_groups, tokens,
                  hidden_in, hidden_out, /*trans_a=*/1, /*trans_b=*/0, stream_);
}

}  // extern "C"

namespace {

int gmm_impl(const void* a, const void* b, void* c, bool out_f32, const int64_t* batch_sizes,
             int batch_sizes_on_device, int64_t num_groups, int64_t tokens, int64_t hidden_in,
             int64_t hidden_out, int trans_a, int trans_b, void* stream_) {
  int rc = check_common(batch_sizes, num_groups, tokens, hidden_in, hidden_out, trans_a, trans_b);
  if (rc != GG_OK) return rc;
  if (num_groups == 0) return GG_OK;
  // nothing to write
  if (hidden_out == 0 || (trans_a ? hidden_in == 0 : tokens == 0)) return GG_OK;
  if (c == nullptr) return fail(GG_EINVAL, "c is null");
  if (tokens > 0 && (a == nullptr || b == nullptr)) return fail(GG_EINVAL, "a or b is null");
  // rows are fetched and stored 16 bytes at a time
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15)
    return fail(GG_ELIMIT, "a, b and c must be 16-byte aligned");
  if (batch_sizes_on_device && num_groups > GG_MAX_GROUPS_PER_LAUNCH)
    return fail(GG_ELIMIT, "at most %d groups are supported when batch_sizes is on the device, got %lld",
                GG_MAX_GROUPS_PER_LAUNCH, (long long)num_groups);

  DeviceInfo info;
  rc = device_info(&info);
  if (rc != GG_OK) return rc;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const int layout = trans_a ? gg::kTN : (trans_b ? gg::kNT : gg::kNN);

  gg::GmmParams p{};
  p.tokens = tokens;
  p.hidden_in = (int32_t)hidden_in;
  p.hidden_out = (int32_t)hidden_out;
  p.group_m = band_height(num_groups, tokens, trans_a);
  p.tail_split = tail_split();
  p.sched_out = nullptr;

  const bool short_shape = use_short_shape(num_groups, tokens, trans_a);
  const int bm = short_shape ? Short::BM : Wide::BM, bn = short_shape ? Short::BN : Wide::BN;
  if (batch_sizes_on_device) {
    if (tile_bound(num_groups, tokens, hidden_in, hidden_out, trans_a, bm, bn) >= (int64_t(1) << 31))
      return fail(GG_ELIMIT, "too many output tiles for one launch");
    p.a = static_cast<const char*>(a);
    p.b = static_cast<const char*>(b);
    p.c = static_cast<char*>(c);
    p.sizes_dev = batch_sizes;
    p.num_groups = (int32_t)num_groups;
    return dispatch<false>(short_shape, layout, out_f32, p, nullptr, info.cus, stream);
  }

  // Host-resident sizes: validated here, passed in the kernel argument block, at most
  // GG_MAX_GROUPS_PER_LAUNCH groups per launch.
  int64_t row = 0;
  for (int64_t e = 0; e < num_groups; ++e) {
    if (batch_sizes[e] < 0) return fail(GG_EINVAL, "batch_sizes[%lld] is negative", (long long)e);
    row += batch_sizes[e];
    if (row > tokens)
      return fail(GG_EINVAL, "batch_sizes sum past the %lld rows of a", (long long)tokens);
  }
  row = 0;
  for (int64_t first = 0; first < num_groups; first += GG_MAX_GROUPS_PER_LAUNCH) {
    const int64_t count = num_groups - first < GG_MAX_GROUPS_PER_LAUNCH
                              ? num_groups - first : GG_MAX_GROUPS_PER_LAUNCH;
    gg::HostSizes hs;
    int64_t rows_here = 0, tiles = 0;
    const int64_t tiles_n = (hidden_out + bn - 1) / bn;
    for (int64_t i = 0; i < count; ++i) {
      hs.v[i] = (int32_t)batch_sizes[first + i];
      rows_here += batch_sizes[first + i];
      tiles += trans_a ? ((hidden_in + bm - 1) / bm) * tiles_n
                       : ((batch_sizes[first + i] + bm - 1) / bm) * tiles_n;
    }
    if (tiles >= (int64_t(1) << 31)) return fail(GG_ELIMIT, "too many output tiles for one launch");
    // this launch sees its own groups as groups 0..count-1 of operands that start at `row`
    p.tokens = rows_here;
    p.num_groups = (int32_t)count;
    p.sizes_dev = nullptr;
    p.a = static_cast<const char*>(a) + row * hidden_in * 2;
    if (trans_a) {
      p.b = static_cast<const char*>(b) + row * hidden_out * 2;
      p.c = static_cast<char*>(c) + first * hidden_in * hidden_out * (out_f32 ? 4 : 2);
    } else {
      p.b = static_cast<const char*>(b) + first * hidden_in * hidden_out * 2;
      p.c = static_cast<char*>(c) + row * hidden_out * 2;
    }
    if (tiles > 0) {
      // the full grid also for few tiles: the last round's tiles may be cut into pieces for
      // the workgroups that would otherwise idle
      rc = dispatch<true>(short_shape, layout, out_f32, p, &hs, info.cus, stream);
      if (rc != GG_OK) return rc;
    }
    row += rows_here;
  }
  return GG_OK;
}

}  // namespace

extern "C" {

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
  p.tail_split = tail_split();
  p.num_groups = (int32_t)num_groups;
  p.sched_out = table_out;
  const int layout = trans_a ? gg::kTN : (trans_b ? gg::kNT : gg::kNN);
  const bool short_shape = use_short_shape(num_groups, tokens, trans_a);
  if (batch_sizes_on_device) {
    p.sizes_dev = batch_sizes;
    return dispatch_dump<false>(short_shape, layout, p, nullptr, stream);
  }
  gg::HostSizes hs;
  for (int64_t i = 0; i < num_groups; ++i) {
    if (batch_sizes[i] < 0 || batch_sizes[i] >= (int64_t(1) << 31))
      return fail(GG_EINVAL, "batch_sizes[%lld] out of range", (long long)i);
    hs.v[i] = (int32_t)batch_sizes[i];
  }
  return dispatch_dump<true>(short_shape, layout, p, &hs, stream);
}

}  // extern "C"
