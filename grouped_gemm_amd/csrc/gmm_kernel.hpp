// Grouped GEMM for gfx950 (MI355X): one persistent launch, scheduler on the device.
//
// Replaces the reference's CUTLASS grouped kernel and its argument builders
// (csrc/grouped_gemm.cu:38-81, 230-371; csrc/fill_arguments.cuh:34-131).
//
// Every workgroup first derives the same schedule from batch_sizes (prefix sums of
// rows and of tiles, kept in LDS), then walks tiles t = id, id + grid, ... .  A tile is
// up to BM x BN outputs of one group: a group's rows are split evenly over its tile rows,
// and a tile issues MFMAs only for the 32-row blocks that have rows.  Operand tiles go from
// HBM straight into LDS
// (buffer_load_dwordx4 ... lds, 16 bytes per lane), through a ring of STAGES buffers;
// rows past a group's end are cut off by the buffer descriptor's size, so they
// arrive as zeros and no lane ever touches memory outside its group.  Fragments are read
// from LDS with ds_read_b128 where the depth dimension is contiguous in memory and
// with the transposing ds_read_b64_tr_b16 where it is not, feed
// v_mfma_f32_32x32x16_bf16 with fp32 accumulators, and leave as bf16 through
// buffer stores that the descriptor clips at the group's last row (or are added to an fp32
// output, in the accumulating form of the weight-gradient layout).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

namespace gg {

constexpr int kMaxGroups = 512;
constexpr int kSchedCols = 14;

enum : int { kNN = 0, kNT = 1, kTN = 2 };
// Element types of a and b.  Two-byte types give a c of the same type; the one-byte (OCP fp8)
// types give a bf16 c.
enum : int { kBF16 = 0, kF16 = 1, kF8E4M3 = 2, kF8E5M2 = 3 };
constexpr bool is_f8(int dt) { return dt == kF8E4M3 || dt == kF8E5M2; }

using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;
using bf16x4 = __attribute__((ext_vector_type(4))) __bf16;
using f16x8 = __attribute__((ext_vector_type(8))) _Float16;
using f16x4 = __attribute__((ext_vector_type(4))) _Float16;
using f32x16 = __attribute__((ext_vector_type(16))) float;
using f32x4 = __attribute__((ext_vector_type(4))) float;
using u32x2 = __attribute__((ext_vector_type(2))) uint32_t;
using u32x4 = __attribute__((ext_vector_type(4))) uint32_t;
using i32x4 = __attribute__((ext_vector_type(4))) int;
using i32x8 = __attribute__((ext_vector_type(8))) int;

#define GG_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

struct GmmParams {
  const char* a;
  const char* b;
  char* c;
  const int64_t* sizes_dev;  // device-resident batch_sizes of ALL groups, or nullptr (then HostSizes)
  int64_t* sched_out;        // only read by the schedule dump kernel
  char* workspace;           // counters + fp32 partial tiles of depth pieces, or nullptr
  int64_t tokens;            // rows of a
  int64_t row_base;          // host-resident sizes: rows taken by the groups before first_group
  int32_t first_group;       // this launch schedules groups first_group .. first_group + num_groups - 1
  int32_t num_groups;        // at most kMaxGroups
  int32_t hidden_in;
  int32_t hidden_out;
  int32_t group_m;     // tile rows per band of the in-group tile order
  int32_t flags;       // kFlag* bits
  int32_t ws_slots;    // partial-tile slots the workspace holds (0: no depth pieces)
  int32_t b_cols;      // columns of one group's b in memory: hidden_out, or twice that for gate | up
  // the variants with row indices only:
  const int32_t* a_rows;   // row r of the left operand is row a_rows[r] of a, or nullptr (rows in place)
  const int32_t* c_rows;   // row r of the output goes to row c_rows[r] of c, or nullptr
  uint32_t a_bytes;        // bytes of a and of c in memory, below kOutOfRangeIndexed
  uint32_t c_bytes;
  uint32_t a_index_rows;   // rows of a and of c in memory: an index that names no row of them is a
  uint32_t c_index_rows;   // missing row (read as zeros, not stored)
  int32_t* status;         // device word that collects kStatus* bits about the sizes, or nullptr
};

enum : int {
  kStatusNegativeSize = 1,   // a batch size was negative (taken as 0)
  kStatusRowsPastEnd = 2,    // the sizes sum past `tokens` (the rows past the end were dropped)
};

enum : int {
  kEpiStore = 0,    // c in the operands' element type, overwritten
  kEpiAccF32 = 1,   // c in fp32, added to (weight-gradient layout only)
  kEpiSwiGLU = 2,   // b holds gate | up columns; c = silu(a @ gate) * (a @ up), half as wide
  // kEpiAccF32 with atomic additions instead of read, add, write: faster while the launch is bound
  // by the matrix pipe (deep groups: 3.35 -> 3.16 ms at 8 x 4096 rows, 4096 x 14336), much slower
  // when it is bound by the traffic of c itself (256 x 256 rows, 2048 x 7168: 7.0 -> 11.7 ms)
  kEpiAccF32Atomic = 3,
};

enum : int {   // debugging switches, for comparing the ways a call can be scheduled
  kFlagWholeTiles = 1,    // never cut the tiles of the last round into pieces
  kFlagOneClass = 2,      // hand out runt rows in place, not after all other tiles
  kFlagRowPieces = 4,     // ignore the workspace: cut along the rows only
  kFlagGroupOrder = 8,    // NN and NT layouts: never hand out the groups' tiles by tile rows
  kFlagByTileRows = 16,   // set by the host side (never by callers): hand them out by tile rows
};

// Workspace layout: kWsCounterBytes of int32 arrival counters (one per tile of the last round; all
// zero before a launch and all zero again after it), then ws_slots partial tiles of BM x BN floats.
constexpr int kWsCounterBytes = 4096;
// Depth pieces per tile: 2 or 4.  A piece's fix-up (a partial tile written, the last piece reading
// them all back) costs about as much as 20 depth slices, so only deep tiles are cut.
constexpr int kMaxDepthPieces = 4;
constexpr int kMinSlicesPerPiece = 48;

// The last round of a persistent grid is filled only partly: `tiles % grid` workgroups have a
// tile, the others idle.  When that rest is at most half of the grid, each of its tiles is cut
// into pieces that go to different workgroups.  With a workspace (and a deep product) the cut
// runs along the depth:
// every piece accumulates its share of the depth slices into an fp32 partial tile in the
// workspace, and the piece that arrives last adds the partial tiles up in piece order (so the sum
// does not depend on which piece that is) and stores the result.  Without a workspace the cut
// runs along the rows (2 or 4 pieces of whole 32-row blocks; not in the weight-gradient layout).
// A launch with fewer tiles than workgroups is all "last round".
struct TailPlan {
  int main_tiles;   // tiles before the last round, handed out whole
  int pieces;       // pieces per tile of the last round
  int total;        // indices to hand out: main_tiles + rest * pieces
  bool by_depth;
};
template <int LAYOUT, bool DEPTH_PIECES_ALLOWED = true>
__device__ __forceinline__ TailPlan plan_tail(int tiles, int grid, const GmmParams& p, int bk) {
  TailPlan t;
  const int rest = tiles % grid;
  t.pieces = 1;
  t.by_depth = false;
  if (rest > 0 && 2 * rest <= grid && !(p.flags & kFlagWholeTiles)) {
    int cand = grid / rest;
    cand = cand > kMaxDepthPieces ? kMaxDepthPieces : cand;
    if (DEPTH_PIECES_ALLOWED && p.ws_slots > 0 && !(p.flags & kFlagRowPieces)) {
      if (rest * cand > p.ws_slots) cand = p.ws_slots / rest;
      cand = cand >= 4 ? 4 : cand;
      {   // keep the pieces worth their fix-up
        // (the depth is the same for every tile, or, in the weight-gradient layout, the group's
        // row count: there the average over the groups stands for it)
        const int64_t depth = LAYOUT != kTN ? (int64_t)p.hidden_in : p.tokens / (p.num_groups > 0 ? p.num_groups : 1);
        const int nk = (int)((depth + bk - 1) / bk);
        if (cand > nk / kMinSlicesPerPiece) cand = nk / kMinSlicesPerPiece;
      }
      cand &= ~1;   // 2 or 4 (3 becomes 2): the fix-up sums two pieces per step
      if (cand >= 2) {
        t.pieces = cand;
        t.by_depth = true;
      }
    }
    if (!t.by_depth && LAYOUT != kTN) t.pieces = 4 * rest <= grid ? 4 : 2;
  }
  t.main_tiles = t.pieces > 1 ? tiles - rest : tiles;
  t.total = t.main_tiles + (tiles - t.main_tiles) * t.pieces;
  return t;
}

// Host-resident batch_sizes travel in the kernel argument block: no copy, no staging.
struct HostSizes {
  int32_t v[kMaxGroups];
};

// What every workgroup keeps in LDS about the groups.  Tiles come in two classes: first all
// tiles except each group's last, much shorter tile row ("runt" row: at most half the 32-row
// blocks of the group's other tile rows), then the runt rows.  Tiles of one class take about the
// same time, so workgroups that walk the classes in this order stay in step, and the cheap tiles
// fill the end of the launch.
struct Sched {
  int32_t row_start[kMaxGroups + 1];   // exclusive prefix sum of rows, clipped to tokens
  int32_t rows[kMaxGroups];            // rows of `a` the group uses
  int32_t tile_start[kMaxGroups + 1];  // exclusive prefix sum of the first class's tiles
  int32_t runt_start[kMaxGroups + 1];  // exclusive prefix sum of the runt rows' tiles
  int32_t arrived;                     // broadcast slot for the arrival count of a depth piece
  int32_t fix_tile[24];                // the tile whose depth pieces this workgroup adds up after its last tile
  // Weight-gradient layout (plan_deep_tiles): the first front_tiles tiles, the deepest ones, are
  // cut along the depth into front_pieces pieces each; tile indices 0 .. front_tiles *
  // front_pieces - 1 name those pieces, the tiles behind follow whole, and the last round is not
  // cut.  (Kept here, not in registers: the tile loop has no scalar registers to spare.)
  int32_t front_tiles, front_pieces;
  int32_t most_rows;                   // rows of the largest group
  // order[q] is the group whose tiles are handed out q-th.  Weight-gradient layout: by descending
  // depth.  Every group has the same number of tiles there and a tile's cost is its group's depth,
  // so the deepest groups go first and the shallow ones fill the end of the launch: what the
  // reference's sort by k does for its scheduler (csrc/grouped_gemm.cu:193-207,
  // csrc/fill_arguments.cuh:80-81).  Other layouts, with kFlagByTileRows: by ascending number of
  // tile rows (tile_start and runt_start then count in that order); without: not used.  Results
  // do not depend on it.
  int16_t order[kMaxGroups];
};

constexpr uint32_t kOutOfRange = 0x80000000u;  // beyond any descriptor size used here
// ... and for the descriptors that span a whole tensor (rows reached through an index)
constexpr uint32_t kOutOfRangeIndexed = 0xfffffff0u;
constexpr uint32_t kRsrcFlags = 0x00020000u;   // raw buffer, 32-bit data format
// Cache policy of the output stores: non-temporal.  The output is written once and never read by
// this kernel, so it should not push operand lines that other tiles still share out of L2.
constexpr int kStoreStreaming = 2;

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// Buffer descriptor of `bytes` bytes at `base`, as the four dwords the hardware reads.
// Both inputs are the same in every lane; reading them through the first lane tells the
// compiler so and keeps the descriptor in scalar registers.
using rsrc_words = __attribute__((ext_vector_type(4))) int;

__device__ __forceinline__ rsrc_words make_rsrc_words(const void* base, uint32_t bytes) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  rsrc_words r;
  r[0] = uniform((int)(uint32_t)b);
  r[1] = uniform((int)((uint32_t)(b >> 32) & 0xffffu));   // 48-bit base, stride 0
  r[2] = uniform((int)bytes);
  r[3] = (int)kRsrcFlags;
  return r;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  const uint64_t ub = (uint64_t)(uint32_t)uniform((int)(uint32_t)b) |
                      ((uint64_t)(uint32_t)uniform((int)(uint32_t)(b >> 32)) << 32);
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(ub), 0,
                                           (uint32_t)uniform((int)bytes), kRsrcFlags);
}

// 16 bytes per lane from global memory straight into LDS at lds_addr + lane * 16.
// Written as assembly on purpose: the compiler then keeps no record of pending writes
// into LDS, and does not put a full wait for them in front of later LDS reads that touch
// other buffers of the ring.  The waits that are needed are the explicit wait_vmcnt calls.
__device__ __forceinline__ void load_to_lds_16(const rsrc_words& rsrc_in, uint32_t voffset,
                                               uint32_t lds_addr) {
  // (the descriptor is the same in every lane; saying so again here keeps it in scalar registers
  // even where the compiler has parked it in vector registers for want of scalar ones)
  rsrc_words rsrc;
  rsrc[0] = uniform(rsrc_in[0]);
  rsrc[1] = uniform(rsrc_in[1]);
  rsrc[2] = uniform(rsrc_in[2]);
  rsrc[3] = uniform(rsrc_in[3]);
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %0, %1, 0 offen lds"
      :
      : "v"(voffset), "s"(rsrc), "s"(lds_addr)
      : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)reinterpret_cast<uintptr_t>(GG_LDS_PTR(p));
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void block_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// One 32x32x16 matrix instruction on fragments of 8 two-byte elements per lane (carried as
// bf16x8 whatever the element type; the type only selects the instruction).
template <int DT>
__device__ __forceinline__ f32x16 mfma_32x32x16(bf16x8 x, bf16x8 y, f32x16 acc) {
  if constexpr (DT == kBF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, x),
                                                  __builtin_bit_cast(f16x8, y), acc, 0, 0, 0);
  }
}

// One 32x32x64 matrix instruction on fp8 fragments: 32 one-byte elements per lane and operand,
// handed over as the two 16-byte halves they are read from LDS in.
template <int DT>
__device__ __forceinline__ f32x16 mfma_32x32x64_f8(bf16x8 x_lo, bf16x8 x_hi, bf16x8 y_lo, bf16x8 y_hi, f32x16 acc) {
  const i32x8 x = __builtin_shufflevector(__builtin_bit_cast(i32x4, x_lo), __builtin_bit_cast(i32x4, x_hi), 0, 1, 2,
                                          3, 4, 5, 6, 7);
  const i32x8 y = __builtin_shufflevector(__builtin_bit_cast(i32x4, y_lo), __builtin_bit_cast(i32x4, y_hi), 0, 1, 2,
                                          3, 4, 5, 6, 7);
  constexpr int FORMAT = DT == kF8E5M2 ? 1 : 0;   // e4m3 : e5m2, for both operands; no block scales
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, acc, FORMAT, FORMAT, 0, 0, 0, 0);
}

// Four fp32 values rounded (to nearest even) to the element type, as 8 bytes.
template <int DT>
__device__ __forceinline__ u32x2 round4(float v0, float v1, float v2, float v3) {
  if constexpr (DT == kBF16) {
    bf16x4 o = {(__bf16)v0, (__bf16)v1, (__bf16)v2, (__bf16)v3};
    return __builtin_bit_cast(u32x2, o);
  } else {
    f16x4 o = {(_Float16)v0, (_Float16)v1, (_Float16)v2, (_Float16)v3};
    return __builtin_bit_cast(u32x2, o);
  }
}

// ---------------------------------------------------------------------- schedule

// How a group's output is cut into tiles.
struct GroupTiles {
  int tiles_m, tiles_n;
  int height;       // rows per tile row (the last tile row takes what is left)
  int main_rows;    // tile rows of the first class
  int runt;         // 1: the last tile row is a runt row (second class)
};

// The rows of a group are split evenly over its tile rows, in whole 32-row blocks: 300 rows make
// two tile rows of 160 (5 blocks each), not one of 256 and one of 44.  Tile rows of a group then
// take the same time, and blocks without rows cost nothing.  What is left for the last tile row
// of a tall group can still be much less than the others' (4122 rows: 16 tile rows of 256 and one
// of 26): such a row goes to the second class.
template <int LAYOUT, int BM, int BN>
__device__ __forceinline__ GroupTiles group_tiles(int rows, int hidden_in, int hidden_out, int flags) {
  GroupTiles g;
  g.tiles_n = (hidden_out + BN - 1) / BN;
  g.runt = 0;
  if (LAYOUT == kTN) {
    g.tiles_m = (hidden_in + BM - 1) / BM;
    g.height = BM;
  } else {
    g.tiles_m = (rows + BM - 1) / BM;
    g.height = BM;
    if (g.tiles_m > 0) {
      g.height = ((rows + g.tiles_m - 1) / g.tiles_m + 31) / 32 * 32;
      const int last_blocks = (rows - (g.tiles_m - 1) * g.height + 31) / 32;
      g.runt = g.tiles_m >= 2 && 2 * last_blocks <= g.height / 32 && !(flags & kFlagOneClass) ? 1 : 0;
    }
  }
  g.main_rows = g.tiles_m - g.runt;
  return g;
}

// Run by the first wave of a workgroup.  Each lane owns up to 8 consecutive groups; one
// wave-wide scan of int64 row counts and one of the two int32 tile counts.  Every size is
// clamped to [0, tokens] before it enters a sum, so no size vector can make a sum overflow or a
// group start before row 0 or end past row `tokens`.
template <int LAYOUT, int BM, int BN>
__device__ __forceinline__ void build_schedule(Sched* s, const GmmParams& p, const HostSizes& hs) {
  const int lane = threadIdx.x;
  if (lane >= 64) return;
  const int E = p.num_groups;
  const int per = (E + 63) >> 6;
  const int e0 = lane * per;
  int bad = 0;   // kStatus* bits seen by this lane
  auto clamp = [&](int64_t v) {
    if (v < 0) bad |= kStatusNegativeSize;
    if (v > p.tokens) bad |= kStatusRowsPastEnd;
    return v < 0 ? (int64_t)0 : (v > p.tokens ? p.tokens : v);
  };
  // rows taken by the groups before this launch's first one
  int64_t base = p.row_base;
  if (p.sizes_dev != nullptr && p.first_group > 0) {
    int64_t part = 0;
    for (int i = lane; i < p.first_group; i += 64) part += clamp(p.sizes_dev[i]);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) part += __shfl_xor(part, d);
    base = part;
  }
  int64_t sz[8];
  int64_t sum = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = e0 + i;
    int64_t v = 0;
    if (i < per && e < E) {
      v = p.sizes_dev != nullptr ? p.sizes_dev[p.first_group + e] : (int64_t)hs.v[e];
      v = clamp(v);
    }
    sz[i] = v;
    sum += v;
  }
  int64_t incl = sum;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int64_t o = __shfl_up(incl, d);
    if (lane >= d) incl += o;
  }
  int64_t run = base + incl - sum;
  int rows[8];
  int tsum = 0, rsum = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = e0 + i;
    const int64_t start = run < p.tokens ? run : p.tokens;
    const int64_t left = p.tokens - start;
    const int r = (int)(sz[i] < left ? sz[i] : left);
    rows[i] = r;
    if (i < per && e < E) {
      s->row_start[e] = (int)start;
      s->rows[e] = r;
      const GroupTiles g = group_tiles<LAYOUT, BM, BN>(r, p.hidden_in, p.hidden_out, p.flags);
      tsum += g.main_rows * g.tiles_n;
      rsum += g.runt * g.tiles_n;
    }
    run += sz[i];
  }
  int tincl = tsum, rincl = rsum;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(tincl, d);
    const int o2 = __shfl_up(rincl, d);
    if (lane >= d) {
      tincl += o;
      rincl += o2;
    }
  }
  int trun = tincl - tsum, rrun = rincl - rsum;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = e0 + i;
    if (i < per && e < E) {
      s->tile_start[e] = trun;
      s->runt_start[e] = rrun;
      const GroupTiles g = group_tiles<LAYOUT, BM, BN>(rows[i], p.hidden_in, p.hidden_out, p.flags);
      trun += g.main_rows * g.tiles_n;
      rrun += g.runt * g.tiles_n;
    }
  }
  int most = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) most = rows[i] > most ? rows[i] : most;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const int o = __shfl_xor(most, d);
    most = o > most ? o : most;
  }
  if (lane == 63) {
    s->front_tiles = 0;
    s->front_pieces = 1;
    s->most_rows = most;
    s->row_start[E] = (int)(run < p.tokens ? run : p.tokens);
    s->tile_start[E] = tincl;
    s->runt_start[E] = rincl;
    if (run > p.tokens) bad |= kStatusRowsPastEnd;
  }
  // What the host would have rejected in host-resident sizes is reported for device-resident
  // ones: one workgroup ORs what its first wave saw into the caller's status word.
  if (p.status != nullptr && blockIdx.x == 0) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) bad |= __shfl_xor(bad, d);
    if (lane == 0 && bad != 0) atomicOr(p.status, bad);
  }
}

// Weight-gradient layout: the groups by descending depth, groups of equal depth in their own order
// (what the reference's stable sort gives).  Run by every thread of the workgroup after
// build_schedule and a barrier; ends with a barrier.  `keys` is scratch for kMaxGroups 64-bit
// words (the tile buffers are not in use yet).
__device__ __forceinline__ void order_groups_by_depth(Sched* s, int num_groups, uint64_t* keys) {
  // Up to a few hundred groups it is quicker to count, per group, the groups that go before it
  // (measured equal at 256 groups, 12 us slower than the sort at 512): straight from
  // Sched::rows, nothing written to `keys` (with the row counts copied there first the compiler
  // built a different and 4-6 % slower depth loop for this layout).
  if (num_groups <= 256) {
    for (int e = threadIdx.x; e < num_groups; e += blockDim.x) {
      const int mine = s->rows[e];
      int before = 0;
      for (int j = 0; j < num_groups; ++j) {
        const int other = s->rows[j];   // (the same address in every lane: a broadcast read)
        before += (other > mine || (other == mine && j < e)) ? 1 : 0;
      }
      s->order[before] = (int16_t)e;
    }
    __syncthreads();
    return;
  }
  // A bitonic sort in LDS of one 64-bit word per group, depth above and 0xffff - index below.
  int n = 2;
  while (n < num_groups) n <<= 1;
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    keys[i] = i < num_groups ? ((uint64_t)(uint32_t)s->rows[i] << 16) | (uint64_t)(0xffff - i) : 0;   // padding sorts last
  __syncthreads();
  for (int k = 2; k <= n; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int partner = i ^ j;
        if (partner > i) {
          const uint64_t x = keys[i], y = keys[partner];
          const bool descending = (i & k) == 0;
          if (descending ? x < y : x > y) {
            keys[i] = y;
            keys[partner] = x;
          }
        }
      }
      __syncthreads();
    }
  }
  for (int i = threadIdx.x; i < num_groups; i += blockDim.x) s->order[i] = (int16_t)(0xffff - (int)(keys[i] & 0xffff));
  __syncthreads();
}

// Weight-gradient layout with a workspace, after order_groups_by_depth: tiles go out by descending
// depth, one workgroup each, so a group much deeper than the others sets the length of the launch
// however its tiles are dealt (Zipf depths: the deepest tile 227 slices, 144 slices of work per
// workgroup).  When the deepest tile is longer than a workgroup's even share of all depth slices,
// the tiles deeper than half that share (and deep enough to pay for their fix-up) are cut into 2
// or 4 depth pieces, which are handed out first, one per workgroup.  Run by every thread; the
// same answer in each.
__device__ __forceinline__ void plan_deep_tiles(Sched* s, const GmmParams& p, int grid, int bk, TailPlan* plan) {
  const int E = p.num_groups;
  const int tiles = s->tile_start[E];
  if (E == 0 || tiles == 0 || p.ws_slots <= 0 || (p.flags & (kFlagWholeTiles | kFlagRowPieces))) return;
  const int per_group = tiles / E;   // (every group has the same number of tiles in this layout)
  // depth slices of all groups together: their rows, and half a slice per group for the rounding
  const int64_t slices = ((int64_t)s->row_start[E] - s->row_start[0] + (int64_t)E * (bk / 2)) / bk;
  const int64_t share = slices * per_group / grid;
  const int deepest = (s->most_rows + bk - 1) / bk;
  const int pieces = deepest >= 4 * kMinSlicesPerPiece ? 4 : (deepest >= 2 * kMinSlicesPerPiece ? 2 : 0);
  if (pieces == 0 || deepest <= share) return;
  int most = grid / pieces;
  most = most < p.ws_slots / pieces ? most : p.ws_slots / pieces;
  most = most < kWsCounterBytes / 4 ? most : kWsCounterBytes / 4;
  int front = 0;
  for (int q = 0; q < E && front < most; ++q) {
    const int depth = (s->rows[s->order[q]] + bk - 1) / bk;
    if (2 * (int64_t)depth <= share || depth < pieces * kMinSlicesPerPiece) break;
    front += per_group;
  }
  front = front < most ? front : most;
  if (front == 0) return;
  s->front_tiles = front;     // (every thread writes the same two values, and reads its own wave's)
  s->front_pieces = pieces;
  plan->pieces = 1;   // the last round stays whole: a workgroup has at most one tile to fix
  plan->by_depth = true;
  plan->main_tiles = plan->total = front * pieces + (tiles - front);
}

// NN and NT layouts with many short groups: the groups by ascending number of tile rows, groups
// of equal number in their own order.  Where group sizes straddle a multiple of the tile height,
// groups of k and of k + 1 tile rows alternate at random in group order; with equal groups side by
// side such launches measured 2-5 % faster (tile indices are dealt to the XCDs in runs of 32 and
// walk a group in bands of tile rows: runs and bands then cut every group the same way).  A
// launch with a group of more than kMaxTileRowsForOrder tile rows (Zipf-like sizes) keeps the
// group order: there it measured 1-2 % slower.  The tile prefix sums are counted again, in the
// new order (the first wave, as in build_schedule; the totals do not change).
constexpr int kMaxTileRowsForOrder = 8;

template <int LAYOUT, int BM, int BN>
__device__ __forceinline__ void order_groups_by_tile_rows(Sched* s, const GmmParams& p) {
  const int E = p.num_groups;
  // A counting sort with one bucket per number of tile rows, by the first wave: each lane owns up
  // to 8 consecutive groups, counts them by bucket, and one wave-wide scan per bucket gives every
  // group its place (about a microsecond, where ranking the groups one against the other took 12).
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    const int per = (E + 63) >> 6;
    const int e0 = lane * per;
    if (s->most_rows > kMaxTileRowsForOrder * BM) {
      for (int i = 0; i < per; ++i)
        if (e0 + i < E) s->order[e0 + i] = (int16_t)(e0 + i);
    } else {
      constexpr int BUCKETS = kMaxTileRowsForOrder + 1;
      int key[8], count[BUCKETS];
#pragma unroll
      for (int b = 0; b < BUCKETS; ++b) count[b] = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        key[i] = (i < per && e0 + i < E) ? (s->rows[e0 + i] + BM - 1) / BM : -1;
#pragma unroll
        for (int b = 0; b < BUCKETS; ++b) count[b] += key[i] == b ? 1 : 0;
      }
      int next[BUCKETS];   // where this lane's next group of a bucket goes
      int base = 0;
#pragma unroll
      for (int b = 0; b < BUCKETS; ++b) {
        int incl = count[b];
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int o = __shfl_up(incl, d);
          if (lane >= d) incl += o;
        }
        next[b] = base + incl - count[b];
        base += __shfl(incl, 63);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int at = -1;
#pragma unroll
        for (int b = 0; b < BUCKETS; ++b) {
          if (key[i] == b) {
            at = next[b];
            next[b] += 1;
          }
        }
        if (at >= 0) s->order[at] = (int16_t)(e0 + i);
      }
    }
  }
  __syncthreads();
  const int lane = threadIdx.x;
  if (lane < 64) {
    const int per = (E + 63) >> 6;
    const int q0 = lane * per;
    int tsum = 0, rsum = 0;
    for (int i = 0; i < per; ++i) {
      const int q = q0 + i;
      if (q < E) {
        const GroupTiles g = group_tiles<LAYOUT, BM, BN>(s->rows[s->order[q]], p.hidden_in, p.hidden_out, p.flags);
        tsum += g.main_rows * g.tiles_n;
        rsum += g.runt * g.tiles_n;
      }
    }
    int tincl = tsum, rincl = rsum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(tincl, d);
      const int o2 = __shfl_up(rincl, d);
      if (lane >= d) {
        tincl += o;
        rincl += o2;
      }
    }
    int trun = tincl - tsum, rrun = rincl - rsum;
    for (int i = 0; i < per; ++i) {
      const int q = q0 + i;
      if (q < E) {
        s->tile_start[q] = trun;
        s->runt_start[q] = rrun;
        const GroupTiles g = group_tiles<LAYOUT, BM, BN>(s->rows[s->order[q]], p.hidden_in, p.hidden_out, p.flags);
        trun += g.main_rows * g.tiles_n;
        rrun += g.runt * g.tiles_n;
      }
    }
  }
  __syncthreads();
}

// Element offsets of a group's A, B and C blocks, the quantities of the reference's
// problem table (csrc/fill_arguments.cuh:72-76) in int64.  The kernel addresses memory
// through these and the schedule dump prints these.
struct GroupGeom {
  int64_t a_off, b_off, c_off;
  int32_t m, n, k;
  int32_t row0;   // first row of the group in a (and in c, unless c is the weight gradient)
};

// `e` is the group's index among all groups of the call; `start` and `rows` are the group's
// entries of Sched::row_start and Sched::rows.
template <int LAYOUT>
__device__ __forceinline__ GroupGeom group_geometry(const GmmParams& p, int e, int64_t start,
                                                    int rows) {
  GroupGeom g;
  const int64_t hin = p.hidden_in, hout = p.hidden_out;
  g.row0 = (int32_t)start;
  if (LAYOUT == kTN) {
    g.m = p.hidden_in;
    g.n = p.hidden_out;
    g.k = rows;
    g.a_off = hin * start;
    g.b_off = start * hout;
    g.c_off = (int64_t)e * hin * hout;
  } else {
    g.m = rows;
    g.n = p.hidden_out;
    g.k = p.hidden_in;
    g.a_off = start * hin;
    g.b_off = (int64_t)e * hin * p.b_cols;
    g.c_off = start * hout;
  }
  return g;
}

// In-group tile order: bands of `group_m` tile rows, tile rows fastest inside a band, so
// that tiles running at the same time share A rows and B columns in L2.
__device__ __forceinline__ void tile_coords(int u, int tiles_m, int tiles_n, int group_m,
                                            int* tm, int* tn) {
  const int per_band = group_m * tiles_n;
  const int band = u / per_band;
  const int first_m = band * group_m;
  const int left = tiles_m - first_m;
  const int gsz = left < group_m ? left : group_m;
  const int r = u - band * per_band;
  *tm = first_m + r % gsz;
  *tn = r / gsz;
}

template <int LAYOUT, int BM, int BN>
__global__ __launch_bounds__(64) void schedule_dump_kernel(GmmParams p, HostSizes hs) {
  __shared__ Sched s;
  __shared__ uint64_t sort_keys[kMaxGroups];
  build_schedule<LAYOUT, BM, BN>(&s, p, hs);
  __syncthreads();
  const bool ordered = LAYOUT == kTN || (p.flags & kFlagByTileRows) != 0;
  if (LAYOUT == kTN) {
    order_groups_by_depth(&s, p.num_groups, sort_keys);
  } else if (ordered) {
    order_groups_by_tile_rows<LAYOUT, BM, BN>(&s, p);
  }
  for (int e = threadIdx.x; e < p.num_groups; e += 64) {
    const GroupGeom g = group_geometry<LAYOUT>(p, p.first_group + e, s.row_start[e], s.rows[e]);
    const GroupTiles gt = group_tiles<LAYOUT, BM, BN>(s.rows[e], p.hidden_in, p.hidden_out, p.flags);
    int64_t* row = p.sched_out + (int64_t)e * kSchedCols;
    row[0] = g.m;
    row[1] = g.n;
    row[2] = g.k;
    row[3] = LAYOUT == kTN ? g.m : g.k;  // lda: column-major A has ld = rows
    row[4] = LAYOUT == kNT ? g.k : g.n;  // ldb
    row[5] = g.n;                        // ldc
    row[6] = g.a_off;
    row[7] = g.b_off;
    row[8] = g.c_off;
    int position = e;   // where the group's tiles stand in the order they are handed out
    if (ordered) {
      for (int q = 0; q < p.num_groups; ++q)
        if (s.order[q] == e) position = q;
    }
    row[9] = s.tile_start[position];
    row[10] = gt.tiles_m * gt.tiles_n;
    row[11] = s.rows[e];
    row[12] = s.tile_start[p.num_groups] + s.runt_start[position];
    row[13] = gt.runt * gt.tiles_n;
  }
}

// ------------------------------------------------------------ operand tile movers
//
// Two kinds of operand tile, by which dimension is contiguous in memory.
//
// DepthMajor ("KC"): R rows (M or N index) of BK depth elements, depth contiguous.  LDS
// keeps row-major rows of BK*2 bytes; the 16-byte chunk c of row r sits at chunk slot
// c ^ ((r / RP) % CPR), which makes 16 consecutive rows at one depth hit 64 distinct
// banks for ds_read_b128.
//
// WidthMajor ("MC"): BK depth rows of W elements (M or N index contiguous).  LDS keeps
// row-major rows of W*2 bytes; 64-byte segment s of depth row k sits at segment slot
// s ^ g(k), g(k) = (k & 3) | ((k >> 1) & 4), so the 8 depth rows one transposing read
// touches land in distinct bank groups.
//
// A lane's LDS slot is fixed by the hardware (wave base + lane * 16), so the swizzle is
// applied by choosing which global chunk each lane fetches.

// GATHER: rows come through an index (or in place) at byte offsets kept per load, relative to
// the start of the whole tensor.  GATE_UP (B of the NT layout with gate | up rows): the tile's R
// rows are 32-row blocks taken alternately from the gate rows and, `up_step` bytes further, the
// up rows of b, so that a wave finds the gate and the up value of an output column side by side.
template <int R, int BK, int NT, bool GATHER = false, bool GATE_UP = false>
struct DepthMajor {
  static constexpr int CPR = BK / 8;                                  // chunks per row
  static constexpr int RP = (BK * 2 >= 256) ? 1 : 256 / (BK * 2);     // rows per 256 B
  static constexpr int ROWS_PER_INSTR = NT / CPR;
  static constexpr int NI = R * CPR / NT;                             // loads per lane per tile
  static constexpr int BYTES = R * BK * 2;
  static_assert(NT % CPR == 0 && (R * CPR) % NT == 0, "tile does not split over the block");
  static_assert(ROWS_PER_INSTR % (RP * CPR) == 0, "swizzle must not depend on the load index");

  const char* base;   // first row of the tile, depth 0
  int ld;             // elements between rows ( = depth extent )
  int span;           // elements from the tile's first row to its last existing row
  int depth;          // depth extent
  int my_chunk;       // depth chunk (of 8) this lane fetches
  uint32_t voff0;     // byte offset of this lane's chunk for load 0
  uint32_t vrow[GATHER ? NI : 1];   // GATHER: byte offset of this lane's chunk per load
  uint32_t total_bytes;             // GATHER: bytes of the whole tensor
  uint32_t up_step;                 // GATE_UP: bytes from a gate row to its up row

  __device__ __forceinline__ void setup(const char* tile_base, int ld_, int rows_valid_, int depth_) {
    base = tile_base;
    ld = ld_;
    span = rows_valid_ > 0 ? (rows_valid_ - 1) * ld_ : -(1 << 30);   // no rows: nothing in range
    depth = depth_;
    const int tid = threadIdx.x;
    const int row = tid / CPR, pos = tid % CPR;
    my_chunk = pos ^ ((row / RP) % CPR);
    voff0 = (uint32_t)(row * ld + my_chunk * 8) * 2u;
  }

  // GATHER: the tile's row r is row rows[r] of the tensor at `tensor_base` (of tensor_rows rows)
  // when `rows` is given, row first_row + r otherwise; rows past rows_valid_ are out of range.
  __device__ __forceinline__ void setup_gather(const char* tensor_base, uint32_t tensor_bytes,
                                               const int32_t* rows, uint32_t tensor_rows, int first_row, int ld_,
                                               int rows_valid_, int depth_) {
    base = tensor_base;
    ld = ld_;
    span = 0;
    depth = depth_;
    total_bytes = tensor_bytes;
    const int tid = threadIdx.x;
    const int row = tid / CPR, pos = tid % CPR;
    my_chunk = pos ^ ((row / RP) % CPR);
    voff0 = 0;
#pragma unroll
    for (int i = 0; i < (GATHER ? NI : 1); ++i) {
      const int r = row + i * ROWS_PER_INSTR;
      uint32_t v = kOutOfRangeIndexed;
      if (r < rows_valid_) {
        const uint32_t src = rows != nullptr ? (uint32_t)rows[r] : (uint32_t)(first_row + r);
        // (an index that names no row of the tensor, negative ones included: a row of zeros)
        if (src < tensor_rows) v = (src * (uint32_t)ld_ + (uint32_t)(my_chunk * 8)) * 2u;
      }
      vrow[i] = v;
    }
  }

  // GATE_UP: `tile_base` is the tile's first gate row; rows_valid_ counts rows to the end of the
  // up rows of the group, so that the descriptor ends where the group's b ends.
  __device__ __forceinline__ void setup_gate_up(const char* tile_base, int ld_, int rows_valid_, int depth_,
                                                int out_cols) {
    setup(tile_base, ld_, rows_valid_, depth_);
    up_step = (uint32_t)out_cols * (uint32_t)ld_ * 2u;
  }

  // Fetch depth slice [kt*BK, kt*BK+BK) into the LDS tile at `dst` (wave-uniform).
  // What all loads of depth slice kt share.
  struct Slice {
    rsrc_words rsrc;
    uint32_t v0;   // this lane's offset for load 0, or out of range in the depth tail
  };
  __device__ __forceinline__ Slice slice(int kt) const {
    const int left = uniform(depth - kt * BK);
    Slice sl;
    if constexpr (GATHER) {
      // the descriptor spans the tensor from this slice's first byte on; v0 is 0 for a chunk
      // inside the depth and out of range for one past it
      const uint32_t skip = (uint32_t)kt * (BK * 2);
      sl.rsrc = make_rsrc_words(base + skip, left > 0 && total_bytes > skip ? total_bytes - skip : 0u);
      sl.v0 = (left >= BK || my_chunk * 8 < left) ? 0u : kOutOfRangeIndexed;
    } else {
      const int elems = left > 0 ? span + left : 0;
      sl.rsrc = make_rsrc_words(base + (int64_t)kt * (BK * 2), elems > 0 ? (uint32_t)elems * 2u : 0u);
      sl.v0 = (left >= BK || my_chunk * 8 < left) ? voff0 : kOutOfRange;
    }
    return sl;
  }
  // Load I of the NI that make up one slice, into the LDS tile at `dst` (wave-uniform).
  template <int I>
  __device__ __forceinline__ void load(const Slice& sl, const char* dst, int wave) const {
    const uint32_t step = (uint32_t)(ROWS_PER_INSTR * ld) * 2u;
    uint32_t v;
    if constexpr (GATHER) {
      v = vrow[I] | sl.v0;   // either flag pushes the offset out of range
    } else if constexpr (GATE_UP) {
      static_assert(ROWS_PER_INSTR == 32, "one load instruction per 32-row block");
      v = sl.v0 + (I / 2) * step + (I % 2) * up_step;
    } else {
      v = sl.v0 + I * step;
    }
    load_to_lds_16(sl.rsrc, v, uniform(lds_address(dst) + (I * NT + wave * 64) * 16));
  }

  // A depth that is even but no multiple of 8: the 16-byte chunk that holds a row's last depth
  // values also holds the first values of the next row in memory (only behind the last row does the
  // descriptor end).  Once the slice with that chunk has landed, every thread clears the foreign
  // dwords of its rows' chunks in the LDS tile at `tile`, so that nothing of another row, not even
  // a NaN against a zero, reaches a sum.  tail = depth values of the slice that exist.
  __device__ static __forceinline__ void clear_depth_tail(char* tile, int tail) {
    const int chunk = tail >> 3, first_dword = (tail & 7) >> 1;
    for (int row = threadIdx.x; row < R; row += NT) {
      uint32_t* at = reinterpret_cast<uint32_t*>(tile + row * (BK * 2) + ((chunk ^ ((row / RP) % CPR)) << 4));
#pragma unroll
      for (int d = 1; d < 4; ++d)
        if (d >= first_dword) at[d] = 0u;
    }
  }
};

// F8 (one-byte elements, seen two to one as W two-byte elements per depth row): 32-byte segment
// s of depth row k sits at segment slot s ^ (k & 7), so the 8 depth rows one byte-wise
// transposing read touches land in 8 distinct groups of 8 banks.
template <int W, int BK, int NT, bool F8 = false>
struct WidthMajor {
  static constexpr int CPRW = W / 8;                  // chunks per depth row
  static constexpr int SEGS = W * 2 / 64;             // 64-byte segments per depth row
  static constexpr int ROWS_PER_INSTR = NT / CPRW;
  static constexpr int NI = BK * CPRW / NT;
  static constexpr int BYTES = W * BK * 2;
  static constexpr int PITCH = W * 2;
  static_assert(NT % CPRW == 0 && (BK * CPRW) % NT == 0, "tile does not split over the block");
  static_assert(SEGS >= 4, "needs at least 128 columns");

  __device__ static __forceinline__ int seg_swizzle(int krow) {
    return (krow & 3) | (SEGS >= 8 ? ((krow >> 1) & 4) : 0);
  }
  // which 16-byte chunk of depth row krow the lane whose LDS slot is chunk p fetches
  __device__ static __forceinline__ int chunk_for_slot(int p, int krow) {
    if constexpr (F8) {
      static_assert(!F8 || CPRW == 16, "8 segments of 32 bytes per depth row");
      return (((p >> 1) ^ (krow & 7)) << 1) | (p & 1);
    } else {
      return (((p >> 2) ^ seg_swizzle(krow)) << 2) | (p & 3);
    }
  }

  const char* base;      // depth row 0 of the group, column 0
  int ld;                // elements between depth rows
  int depth;             // depth rows of the group
  uint32_t voff[NI];     // byte offset of this lane's chunk per load (kOutOfRange past the width)

  __device__ __forceinline__ void setup(const char* group_base, int ld_, int depth_, int col0,
                                        int width) {
    base = group_base;
    ld = ld_;
    depth = depth_;
    const int tid = threadIdx.x;
    const int krow0 = tid / CPRW, p = tid % CPRW;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int krow = krow0 + i * ROWS_PER_INSTR;
      const int c = chunk_for_slot(p, krow);
      const int col = col0 + c * 8;
      voff[i] = col < width ? (uint32_t)(krow * ld + col) * 2u : kOutOfRange;
    }
  }

  // B of the NN layout with gate | up columns: the tile's W columns are 32-column blocks taken
  // alternately from the gate columns [0, out_cols) and the up columns [out_cols, 2 out_cols) of
  // the group's b; col0 is the tile's first output column, ld_ = 2 * out_cols.
  __device__ __forceinline__ void setup_gate_up(const char* group_base, int ld_, int depth_, int col0,
                                                int out_cols) {
    base = group_base;
    ld = ld_;
    depth = depth_;
    const int tid = threadIdx.x;
    const int krow0 = tid / CPRW, p = tid % CPRW;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int krow = krow0 + i * ROWS_PER_INSTR;
      static_assert(!F8, "gate | up columns are for two-byte elements");
      const int c = chunk_for_slot(p, krow);   // 16-byte chunk of the tile row
      const int block = c >> 2;                                        // 32-column block of the tile
      const int out = col0 + (block >> 1) * 32 + (c & 3) * 8;          // output column it belongs to
      const int col = (block & 1) * out_cols + out;
      voff[i] = out < out_cols ? (uint32_t)(krow * ld + col) * 2u : kOutOfRange;
    }
  }

  struct Slice {
    rsrc_words rsrc;
  };
  __device__ __forceinline__ Slice slice(int kt) const {
    int left = uniform(depth - kt * BK);
    left = left < 0 ? 0 : (left > BK ? BK : left);
    Slice sl;
    sl.rsrc = make_rsrc_words(base + (int64_t)kt * BK * ld * 2, (uint32_t)(left * ld) * 2u);
    return sl;
  }
  template <int I>
  __device__ __forceinline__ void load(const Slice& sl, const char* dst, int wave) const {
    load_to_lds_16(sl.rsrc, voff[I], uniform(lds_address(dst) + (I * NT + wave * 64) * 16));
  }
};

// ---------------------------------------------------------------- fragment readers
// A fragment is the operand of one 32x32x16 MFMA: lane l holds 8 depth values
// 8*(l/32) .. +7 of row (or column) l % 32.

// STRIDE: distance between the blocks a wave owns, in 32-wide blocks (the waves along a
// dimension take blocks alternately when STRIDE is their number, contiguously when it is 1).
// F8: one-byte elements.  A row of the tile is then 128 depth values, and the fragment of one
// 32x32x64 instruction is 32 consecutive bytes of it (depth 32 (l / 32) .. +31 of a 64-deep step),
// read as two 16-byte halves: "step" 2 s + h below is half h of 64-deep step s.
template <int BK, int STRIDE, bool F8 = false>
struct DepthMajorFrag {
  static constexpr int CPR = BK / 8;
  static constexpr int RP = (BK * 2 >= 256) ? 1 : 256 / (BK * 2);
  static_assert((32 / RP) % CPR == 0, "blocks must share the swizzle of block 0");
  uint32_t off[BK / 16];   // lane offset per 16-deep step, block 0

  __device__ __forceinline__ void setup(int first_row) {
    const int lane = threadIdx.x & 63;
    const int row = first_row + (lane & 31);
    const int sw = (row / RP) % CPR;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int chunk = F8 ? 4 * (ks / 2) + 2 * (lane >> 5) + ks % 2 : ks * 2 + (lane >> 5);
      off[ks] = (uint32_t)(row * (BK * 2) + ((chunk ^ sw) << 4));
    }
  }
  __device__ __forceinline__ bf16x8 read(const char* tile, int ks, int blk) const {
    return *reinterpret_cast<const bf16x8*>(tile + off[ks] + blk * (STRIDE * 32) * (BK * 2));
  }
};

template <int W, int BK, int NBLK, int STRIDE>
struct WidthMajorFrag {
  static constexpr int PITCH = W * 2;
  static constexpr int SEGS = W * 2 / 64;
  uint32_t off[NBLK];   // lane offset per 32-wide block, depth step 0

  __device__ __forceinline__ void setup(int first_col) {
    const int lane = threadIdx.x & 63;
    const int l16 = lane & 15;
    const int krow = 8 * (lane >> 5) + (l16 >> 2);
    const int g = (krow & 3) | (SEGS >= 8 ? ((krow >> 1) & 4) : 0);
#pragma unroll
    for (int j = 0; j < NBLK; ++j) {
      const int seg = (first_col >> 5) + j * STRIDE;
      off[j] = (uint32_t)(krow * PITCH + ((seg ^ g) << 6) + 32 * ((lane >> 4) & 1) + 8 * (l16 & 3));
    }
  }
  __device__ __forceinline__ bf16x8 read(const char* tile, int ks, int blk) const {
    const char* p = tile + off[blk] + ks * 16 * PITCH;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (__attribute__((address_space(3))) bf16x4*)GG_LDS_PTR(p));
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (__attribute__((address_space(3))) bf16x4*)GG_LDS_PTR(p + 4 * PITCH));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
};

// One-byte elements, width-major tile of W bytes per depth row (128 depth rows a slice).  The
// fragment of a 32x32x64 instruction is, per lane, 32 consecutive depth values of one column
// (depth 32 (l / 32) .. +31 of the 64-deep step, column l % 32), carried as two 16-byte halves
// like the depth-major one: "step" 2 s + h is half h of 64-deep step s.  ds_read_b64_tr_b8 gives
// a lane 8 consecutive depth values of its column: 16 lanes hand in the addresses of an 8 x 16
// byte block (lane i: depth row i / 2, bytes 8 (i % 2) .. +7) and lane j of them receives column
// j.  Two such reads make a half.
template <int W, int NBLK, int STRIDE>
struct WidthMajorFrag8 {
  static constexpr int PITCH = W;
  uint32_t off[NBLK];   // lane offset per 32-wide block, 64-deep step 0, half 0, first read

  __device__ __forceinline__ void setup(int first_col) {
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4, i = lane & 15;
    const int krow = 32 * (g >> 1) + (i >> 1);   // (+ multiples of 8: the swizzle sees i / 2 only)
#pragma unroll
    for (int j = 0; j < NBLK; ++j) {
      const int col = first_col + j * STRIDE * 32 + 16 * (g & 1) + 8 * (i & 1);
      off[j] = (uint32_t)(krow * PITCH + ((((col >> 5) ^ (krow & 7)) << 5) | (col & 31)));
    }
  }
  __device__ __forceinline__ bf16x8 read(const char* tile, int ks, int blk) const {
    using i32x2 = __attribute__((ext_vector_type(2))) int;
    using i32x4 = __attribute__((ext_vector_type(4))) int;
    const char* p = tile + off[blk] + (64 * (ks / 2) + 16 * (ks % 2)) * PITCH;
    const i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)GG_LDS_PTR(p));
    const i32x2 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
        (__attribute__((address_space(3))) i32x2*)GG_LDS_PTR(p + 8 * PITCH));
    return __builtin_bit_cast(bf16x8, i32x4{lo[0], lo[1], hi[0], hi[1]});
  }
};

// ------------------------------------------------------------------------ kernel

// Compile-time loop: f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N-1>{}).
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  [&]<int... I>(std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
  }(std::make_integer_sequence<int, N>{});
}

constexpr int kTileInfoDwords = 24;   // a tile's description on its way through LDS (pack_tile)

template <int LAYOUT, int BM, int BN, int BK, int STAGES, int WAVES_M, int WAVES_N>
struct GmmConfig {
  static constexpr int NT = WAVES_M * WAVES_N * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int MB = WTM / 32, NB = WTN / 32;
  static constexpr bool A_DEPTH_MAJOR = LAYOUT != kTN;
  static constexpr bool B_DEPTH_MAJOR = LAYOUT == kNT;
  static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  // after the tile buffers: the schedule, then one strip per wave for the epilogue
  static constexpr int SCHED_OFFSET = STAGES * STAGE_BYTES;
  static constexpr int EPILOGUE_OFFSET = (SCHED_OFFSET + (int)sizeof(Sched) + 15) / 16 * 16;
  static constexpr int EPILOGUE_PITCH = 64 * 2 + 16;            // 64 bf16 columns + padding
  static constexpr int EPILOGUE_WAVE_BYTES = 32 * EPILOGUE_PITCH;
  static constexpr bool STAGED_EPILOGUE =
      NB % 2 == 0 && EPILOGUE_OFFSET + WAVES_M * WAVES_N * EPILOGUE_WAVE_BYTES <= 160 * 1024;
  // last: per wave, the descriptions of the tiles between the fetch and the compute cursor
  static constexpr int TILE_RING_SLOTS = 4;
  static constexpr int TILE_RING_OFFSET =
      ((STAGED_EPILOGUE ? EPILOGUE_OFFSET + WAVES_M * WAVES_N * EPILOGUE_WAVE_BYTES
                        : SCHED_OFFSET + (int)sizeof(Sched)) + 15) / 16 * 16;
  static constexpr int LDS_BYTES = TILE_RING_OFFSET + WAVES_M * WAVES_N * TILE_RING_SLOTS * kTileInfoDwords * 4;
  static_assert(LDS_BYTES <= 160 * 1024, "a compute unit has 160 KiB of LDS");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile is made of 32x32 MFMA blocks");
  static_assert(BK % 16 == 0 && STAGES >= 2, "");
};

// One output tile (or one piece of a tile of the last round) as the scheduler hands it out.
struct TileInfo {
  GroupGeom g;
  int m0, n0;       // first row and column of the tile inside its group's output
  int rows_valid;   // rows of the tile that exist (0: no tile)
  int blocks;       // 32-row blocks the tile's rows take (MFMAs are issued for these only)
  int depth;        // depth to fetch (0: nothing to fetch, the tile multiplies zeros)
  int k0;           // first depth slice (not 0 only for a depth piece)
  int nk;           // depth slices, at least 1 so that an empty group still stores zeros
  int pieces;       // depth pieces this tile is cut into (1: whole depth, store directly)
  int piece;        // which of them this is
  int rank;         // index of the tile among the tiles of the last round
  bool valid;
};

// Where a tile cursor stands: group and class.  Tile indices only grow, so inside a class the
// group only moves forward; it starts over once, when the indices pass into the runt class.
struct TileCursor {
  int e = 0;
  int cls = 0;
};

// A tile's description as 24 dwords, for the trip through LDS from the fetch cursor, which works
// it out, to the compute cursor, which needs the same one or two tiles later.
__device__ __forceinline__ void pack_tile(const TileInfo& t, int32_t* w) {
  w[0] = (int32_t)t.g.a_off, w[1] = (int32_t)(t.g.a_off >> 32);
  w[2] = (int32_t)t.g.b_off, w[3] = (int32_t)(t.g.b_off >> 32);
  w[4] = (int32_t)t.g.c_off, w[5] = (int32_t)(t.g.c_off >> 32);
  w[6] = t.g.m, w[7] = t.g.n, w[8] = t.g.k, w[9] = t.g.row0;
  w[10] = t.m0, w[11] = t.n0, w[12] = t.rows_valid, w[13] = t.blocks, w[14] = t.depth, w[15] = t.k0;
  w[16] = t.nk, w[17] = t.pieces, w[18] = t.piece, w[19] = t.rank, w[20] = t.valid ? 1 : 0;
  w[21] = w[22] = w[23] = 0;
}
__device__ __forceinline__ TileInfo unpack_tile(const int32_t* w) {
  auto u = [&](int i) { return uniform(w[i]); };
  auto u64 = [&](int i) { return (int64_t)(((uint64_t)(uint32_t)u(i + 1) << 32) | (uint32_t)u(i)); };
  TileInfo t;
  t.g.a_off = u64(0), t.g.b_off = u64(2), t.g.c_off = u64(4);
  t.g.m = u(6), t.g.n = u(7), t.g.k = u(8), t.g.row0 = u(9);
  t.m0 = u(10), t.n0 = u(11), t.rows_valid = u(12), t.blocks = u(13), t.depth = u(14), t.k0 = u(15);
  t.nk = u(16), t.pieces = u(17), t.piece = u(18), t.rank = u(19), t.valid = u(20) != 0;
  return t;
}

// Smallest position e >= from with t < start[e + 1], for an exclusive prefix sum `start` of n
// positions with t < start[n] (so start[e] <= t: positions without tiles are passed over).  A
// gallop, then a bisection: two probes when the answer is the next position, the common case of a
// cursor that moves on, and about 2 log2 of the distance for a workgroup's first tile, where a
// walk position by position, one LDS round trip each, took 15 to 30 us of a launch with 256 to 512
// groups.
__device__ __forceinline__ int advance_to(const int32_t* start, int n, int from, int t) {
  if (t < uniform(start[from + 1])) return from;
  int lo = from + 1, step = 1;   // t >= start[lo]
  while (lo + step < n && t >= uniform(start[lo + step])) {
    lo += step;
    step <<= 1;
  }
  int hi = lo + step < n ? lo + step : n;   // t < start[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (t >= uniform(start[mid])) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  return lo;
}

// Tile index -> group and position.  Indices past plan.main_tiles name pieces of the last
// round's tiles: piece (t - main) % pieces of tile main + (t - main) / pieces.
template <int LAYOUT, int BM, int BN, int BK>
__device__ __forceinline__ TileInfo find_tile(const Sched* sched, const GmmParams& p, int t,
                                              const TailPlan& plan, TileCursor& cur) {
  TileInfo ti;
  ti.k0 = 0;
  ti.pieces = 1;
  ti.piece = 0;
  ti.rank = 0;
  if (t >= plan.total) {
    ti.g = GroupGeom{0, 0, 0, 0, 0, 0, 0};
    ti.m0 = ti.n0 = ti.rows_valid = ti.depth = 0;
    ti.blocks = 1;
    ti.nk = 1;
    ti.valid = false;
    return ti;
  }
  int piece = -1;
  int pieces = plan.pieces;
  const int front_tiles = LAYOUT == kTN ? uniform(sched->front_tiles) : 0;
  if (front_tiles > 0) {
    const int front_pieces = uniform(sched->front_pieces);
    const int cut = front_tiles * front_pieces;
    if (t < cut) {
      pieces = front_pieces;
      piece = t % pieces;
      ti.rank = t / pieces;
      t = ti.rank;
    } else {
      t = t - cut + front_tiles;
    }
  } else if (t >= plan.main_tiles) {
    const int r = t - plan.main_tiles;
    piece = r % plan.pieces;
    ti.rank = r / plan.pieces;
    t = plan.main_tiles + ti.rank;
  }
  const int first_class = uniform(sched->tile_start[p.num_groups]);
  int u;
  if (LAYOUT == kTN) {
    // (every group has the same number of tiles, tile_start[1], and there are no runt rows)
    const int per_group = uniform(sched->tile_start[1]);
    cur.e = t / per_group;
    u = t - cur.e * per_group;
  } else if (t < first_class) {
    cur.e = advance_to(sched->tile_start, p.num_groups, cur.e, t);
    u = t - uniform(sched->tile_start[cur.e]);
  } else {
    if (cur.cls == 0) {
      cur.cls = 1;
      cur.e = 0;
    }
    t -= first_class;
    cur.e = advance_to(sched->runt_start, p.num_groups, cur.e, t);
    u = t - uniform(sched->runt_start[cur.e]);
  }
  // (the cursor walks positions of the order the groups are handed out in.  Weight-gradient layout:
  // all groups have the same number of tiles, so the tile prefix sums serve positions as they are;
  // by tile rows: the prefix sums were counted in that order)
  const bool ordered = LAYOUT == kTN || (p.flags & kFlagByTileRows) != 0;
  const int e = ordered ? uniform((int)sched->order[cur.e]) : cur.e;
  // read through the first lane: everything derived from these stays in scalar registers
  const int rows = uniform(sched->rows[e]);
  ti.g = group_geometry<LAYOUT>(p, p.first_group + e, uniform(sched->row_start[e]), rows);
  const GroupTiles gt = group_tiles<LAYOUT, BM, BN>(rows, p.hidden_in, p.hidden_out, p.flags);
  int tm, tn;
  if (cur.cls == 0) {
    tile_coords(u, gt.main_rows, gt.tiles_n, p.group_m, &tm, &tn);
  } else {
    tm = gt.tiles_m - 1;
    tn = u;
  }
  ti.m0 = uniform(tm) * gt.height;
  ti.n0 = uniform(tn) * BN;
  ti.rows_valid = min(gt.height, ti.g.m - ti.m0);
  ti.depth = ti.g.k;
  const int nk = (ti.g.k + BK - 1) / BK;
  ti.nk = nk < 1 ? 1 : nk;
  if (piece >= 0 && plan.by_depth) {
    // this piece's share of the depth slices; a piece without slices contributes zeros
    const int first = piece * ti.nk / pieces, last = (piece + 1) * ti.nk / pieces;
    ti.pieces = pieces;
    ti.piece = piece;
    ti.k0 = first;
    ti.nk = last - first;
    if (ti.nk <= 0) {
      ti.k0 = 0;
      ti.nk = 1;
      ti.depth = 0;
    }
  } else if (piece >= 0) {
    // this piece's share of the tile's 32-row blocks; a piece past the rows is an empty tile
    const int all = (ti.rows_valid + 31) / 32;
    const int per = (all + pieces - 1) / pieces;
    const int skip = piece * per * 32;
    ti.m0 += skip;
    ti.rows_valid = min(per * 32, ti.rows_valid - skip);
    if (ti.rows_valid <= 0) {
      ti.rows_valid = 0;
      ti.depth = 0;
      ti.nk = 1;
    }
  }
  ti.blocks = LAYOUT == kTN ? BM / 32 : max(1, (ti.rows_valid + 31) / 32);
  ti.valid = true;
  return ti;
}

// DT: element type of a and b (and of c unless it is the fp32 accumulator).
// EPI: what happens to a finished tile (kEpi*): stored in the element type; added to an fp32 c
// (gradient accumulation, weight-gradient layout); or, with gate | up columns in b, combined to
// silu(gate) * up and stored half as wide.
// INDEXED: rows of a are fetched and rows of c stored through p.a_rows / p.c_rows (NN and NT).
// RAGGED_DEPTH: hidden_in is even but no multiple of 8 (NN and NT, two-byte elements, plain store).
template <int DT, int LAYOUT, int BM, int BN, int BK, int STAGES, int WAVES_M, int WAVES_N,
          int EPI = kEpiStore, bool INDEXED = false, bool RAGGED_DEPTH = false>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gmm_kernel(GmmParams p, HostSizes hs) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
  using Cfg = GmmConfig<LAYOUT, BM, BN, BK, STAGES, WAVES_M, WAVES_N>;
  constexpr int NT = Cfg::NT, MB = Cfg::MB, NB = Cfg::NB, KS = BK / 16;
  constexpr bool ACC_F32 = EPI == kEpiAccF32 || EPI == kEpiAccF32Atomic, GATE_UP = EPI == kEpiSwiGLU;
  // One-byte elements (NT layout only: both operands depth-contiguous).  The tile movers see them
  // as two-byte elements, two to one: same bytes per row and slice, BK_ELEMS depth values a slice.
  constexpr bool F8 = is_f8(DT);
  constexpr int ES = F8 ? 1 : 2, BK_ELEMS = BK * 2 / ES, OUT_DT = DT == kF16 ? kF16 : kBF16;
  static_assert(!F8 || !GATE_UP || LAYOUT == kNT, "fp8 with gate | up rows streams in the NT layout only");
  static_assert(!ACC_F32 || LAYOUT == kTN, "the fp32 accumulator is the weight gradient's");
  static_assert(!(GATE_UP || INDEXED) || LAYOUT != kTN, "row indices and gate | up are for the NN and NT layouts");
  static_assert(!GATE_UP || NB % 2 == 0, "a wave needs the gate and the up block of its columns");
  constexpr int BNS = GATE_UP ? BN / 2 : BN;   // output columns per tile, what the schedule counts in
  // (width-major tiles of one-byte elements: half as many two-byte elements per depth row, twice
  // the depth rows)
  using ALoad = std::conditional_t<Cfg::A_DEPTH_MAJOR, DepthMajor<BM, BK, NT, INDEXED>,
                                   WidthMajor<BM * ES / 2, BK_ELEMS, NT, F8>>;
  using BLoad = std::conditional_t<Cfg::B_DEPTH_MAJOR, DepthMajor<BN, BK, NT, false, GATE_UP>,
                                   WidthMajor<BN * ES / 2, BK_ELEMS, NT, F8>>;
  using AFrag = std::conditional_t<Cfg::A_DEPTH_MAJOR, DepthMajorFrag<BK, WAVES_M, F8>,
                                   std::conditional_t<F8, WidthMajorFrag8<BM, MB, WAVES_M>, WidthMajorFrag<BM, BK, MB, WAVES_M>>>;
  using BFrag = std::conditional_t<Cfg::B_DEPTH_MAJOR, DepthMajorFrag<BK, 1, F8>,
                                   std::conditional_t<F8, WidthMajorFrag8<BN, NB, 1>, WidthMajorFrag<BN, BK, NB, 1>>>;
  constexpr int LOADS_PER_STAGE = ALoad::NI + BLoad::NI;   // per lane, per depth slice
  constexpr int QUARTER_LOADS = LOADS_PER_STAGE / 4;
  static_assert(KS == 4 && STAGES == 2, "the step schedule below is written for BK = 64 and two buffers");
  static_assert(LOADS_PER_STAGE % 4 == 0 && LOADS_PER_STAGE < 32, "");
  constexpr int UNITS = MB + NB;    // fragments of one 16-deep step

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  Sched* sched = reinterpret_cast<Sched*>(smem + Cfg::SCHED_OFFSET);
  build_schedule<LAYOUT, BM, BNS>(sched, p, hs);
  __syncthreads();
  if constexpr (LAYOUT == kTN) {
    order_groups_by_depth(sched, p.num_groups, reinterpret_cast<uint64_t*>(smem));
  } else {
    if (p.flags & kFlagByTileRows) order_groups_by_tile_rows<LAYOUT, BM, BNS>(sched, p);
  }

  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  AFrag afrag;
  BFrag bfrag;
  afrag.setup(wm * 32);   // wave row wm owns row blocks wm, wm + WAVES_M, ...
  bfrag.setup(wn * Cfg::WTN);

  // (a tile that is combined or scattered on its way out is never cut along the depth: the
  // fix-up of the depth pieces stores plain tiles)
  constexpr bool DEPTH_PIECES = !(GATE_UP || INDEXED || RAGGED_DEPTH);
  TailPlan plan = plan_tail<LAYOUT, DEPTH_PIECES>(
      uniform(sched->tile_start[p.num_groups]) + uniform(sched->runt_start[p.num_groups]),
      (int)gridDim.x, p, BK_ELEMS);
  if constexpr (!DEPTH_PIECES) plan.by_depth = false;   // (known at compile time: no depth-piece code is kept)
  if constexpr (LAYOUT == kTN && DEPTH_PIECES) {
    plan_deep_tiles(sched, p, (int)gridDim.x, BK_ELEMS, &plan);
    plan.pieces = uniform(plan.pieces), plan.main_tiles = uniform(plan.main_tiles), plan.total = uniform(plan.total);
  }
  const int total_tiles = plan.total;

  // Workgroups are dealt to the 8 XCDs round-robin; give each XCD a contiguous run of
  // tile indices so that its private L2 sees neighbouring tiles.
  const int G = gridDim.x;
  const int w = blockIdx.x;
  const int vid = (G % 8 == 0) ? (w % 8) * (G / 8) + (w / 8) : w;
  if (vid >= total_tiles) return;

  // Two cursors walk this workgroup's tiles: the fetch cursor runs STAGES depth slices
  // ahead of the compute cursor and crosses into the next tile on its own, so the first
  // slices of a tile are already in flight while the previous tile is being stored.
  ALoad aload;
  BLoad bload;
  int fetch_t = vid, fetch_kt = 0;
  TileCursor fetch_cur;
  TileInfo fti;
  // The compute cursor does not look its tiles up again: the fetch cursor, which is one or two
  // tiles ahead, leaves each description in a ring in LDS (one ring per wave, written by its first
  // lane and read back by the same wave: no barrier involved).
  int32_t* tile_ring = reinterpret_cast<int32_t*>(smem + Cfg::TILE_RING_OFFSET) +
                       wave * (Cfg::TILE_RING_SLOTS * kTileInfoDwords);
  int fetch_n = 0;   // tiles the fetch cursor has set up
  auto fetch_setup = [&]() {
    fti = find_tile<LAYOUT, BM, BNS, BK_ELEMS>(sched, p, fetch_t, plan, fetch_cur);
    {
      int32_t words[kTileInfoDwords];
      pack_tile(fti, words);
      int32_t* slot = tile_ring + (fetch_n % Cfg::TILE_RING_SLOTS) * kTileInfoDwords;
      if (lane == 0) {
#pragma unroll
        for (int i = 0; i < kTileInfoDwords; i += 4)
          *reinterpret_cast<u32x4*>(slot + i) = u32x4{(uint32_t)words[i], (uint32_t)words[i + 1],
                                                      (uint32_t)words[i + 2], (uint32_t)words[i + 3]};
      }
      fetch_n = uniform(fetch_n + 1);
    }
    const int depth = fti.depth;
    if constexpr (INDEXED) {
      const int first = fti.g.row0 + fti.m0;
      aload.setup_gather(p.a, p.a_bytes, p.a_rows != nullptr ? p.a_rows + first : nullptr, p.a_index_rows, first,
                         fti.g.k * ES / 2, depth > 0 ? fti.rows_valid : 0, depth * ES / 2);
    } else if constexpr (Cfg::A_DEPTH_MAJOR) {
      aload.setup(p.a + (fti.g.a_off + (int64_t)fti.m0 * fti.g.k) * ES, fti.g.k * ES / 2, fti.rows_valid,
                  depth * ES / 2);
    } else {
      aload.setup(p.a + fti.g.a_off * ES, fti.g.m * ES / 2, depth, fti.m0 * ES / 2, fti.g.m * ES / 2);
    }
    if constexpr (GATE_UP && Cfg::B_DEPTH_MAJOR) {
      bload.setup_gate_up(p.b + (fti.g.b_off + (int64_t)fti.n0 * fti.g.k) * ES, fti.g.k * ES / 2,
                          fti.valid && depth > 0 ? 2 * fti.g.n - fti.n0 : 0, depth * ES / 2, fti.g.n);
    } else if constexpr (GATE_UP) {
      bload.setup_gate_up(p.b + fti.g.b_off * 2, 2 * fti.g.n, depth, fti.n0, fti.g.n);
    } else if constexpr (Cfg::B_DEPTH_MAJOR) {
      bload.setup(p.b + (fti.g.b_off + (int64_t)fti.n0 * fti.g.k) * ES, fti.g.k * ES / 2,
                  fti.valid && depth > 0 ? min(BN, fti.g.n - fti.n0) : 0, depth * ES / 2);
    } else {
      bload.setup(p.b + fti.g.b_off * ES, fti.g.n * ES / 2, depth, fti.n0 * ES / 2, fti.g.n * ES / 2);
    }
  };
  // Slices past the depth (or past the last tile) are fetched with an empty descriptor:
  // zeros, no traffic, and the number of loads in flight is the same at every step.
  typename ALoad::Slice a_slice;
  typename BLoad::Slice b_slice;
  auto fetch_begin = [&]() {   // descriptors of the cursor's slice
    a_slice = aload.slice(fti.k0 + fetch_kt);
    b_slice = bload.slice(fti.k0 + fetch_kt);
  };
  // Load J of the cursor's slice (A's loads first, then B's) into buffer `buf`.
  auto fetch_load = [&](auto j_tag, int buf) {
    constexpr int J = decltype(j_tag)::value;
    const char* st = smem + uniform(buf) * Cfg::STAGE_BYTES;
    if constexpr (J < ALoad::NI) {
      aload.template load<J>(a_slice, st, wave);
    } else {
      bload.template load<J - ALoad::NI>(b_slice, st + Cfg::A_BYTES, wave);
    }
  };
  auto fetch_advance = [&]() {
    // (said to be the same in every lane once more: where the compiler loses track of that, the
    // slice descriptors below are computed lane by lane and the branch becomes a masked one)
    fetch_kt = uniform(fetch_kt + 1);
    if (fetch_kt == uniform(fti.nk) && uniform((int)fti.valid) != 0) {
      fetch_t = uniform(fetch_t + G);
      fetch_kt = 0;
      fetch_setup();
    }
  };

  // Fragments: one register set per 16-deep step of a slice.  A "unit" is one fragment (one
  // ds_read_b128, or two transposing 64-bit reads): the first ML of A's, then B's NB.
  bf16x8 fa[KS][MB], fb[KS][NB];
  auto read_unit = [&](auto u_tag, auto set_tag, auto ml_tag, int buf) {   // set = 16-deep step it belongs to
    constexpr int U = decltype(u_tag)::value, SET = decltype(set_tag)::value, ML = decltype(ml_tag)::value;
    const char* sa = smem + buf * Cfg::STAGE_BYTES;
    if constexpr (U < ML) {
      fa[SET][U] = afrag.read(sa, SET, U);
    } else {
      fb[SET][U - ML] = bfrag.read(sa + Cfg::A_BYTES, SET, U - ML);
    }
  };

  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  using IMB = std::integral_constant<int, MB>;
  using IQ = std::integral_constant<int, QUARTER_LOADS>;
  using IQ2 = std::integral_constant<int, 2 * QUARTER_LOADS>;
  using IQ3 = std::integral_constant<int, 3 * QUARTER_LOADS>;

  // Both buffers are requested up front, except the last quarter of the second slice: every
  // step issues one quarter of a slice's loads, and step 0 issues the last quarter of the
  // slice that was begun in the steps before it.
  fetch_setup();
  fetch_begin();
  static_for<LOADS_PER_STAGE>([&](auto j) { fetch_load(j, 0); });
  fetch_advance();
  fetch_begin();
  static_for<3 * QUARTER_LOADS>([&](auto j) { fetch_load(j, 1); });

  int tile_t = vid;
  int tile_n = 0;   // tiles this workgroup has finished
  auto next_tile = [&]() {
    int32_t words[kTileInfoDwords];
    const int32_t* slot = tile_ring + (tile_n % Cfg::TILE_RING_SLOTS) * kTileInfoDwords;
#pragma unroll
    for (int i = 0; i < kTileInfoDwords; i += 4) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(slot + i);
      words[i] = (int32_t)v[0], words[i + 1] = (int32_t)v[1], words[i + 2] = (int32_t)v[2], words[i + 3] = (int32_t)v[3];
    }
    return unpack_tile(words);
  };
  TileInfo ti = next_tile();
  // RAGGED_DEPTH: hidden_in is even but no multiple of 8.  No depth pieces then (every tile starts at
  // depth 0), so the ragged chunks are in slice hidden_in / BK of every tile.  Once a buffer holds
  // that slice, complete for every wave, what its ragged chunks picked up from the rows behind is
  // cleared before any wave reads a fragment from it.
  static_assert(!RAGGED_DEPTH || (LAYOUT != kTN && !F8 && !GATE_UP && !INDEXED), "");
  const int tail_slice = RAGGED_DEPTH ? p.hidden_in / BK : -1;
  auto clear_tail = [&](int buf) {
    if constexpr (RAGGED_DEPTH) {
      char* st = smem + uniform(buf) * Cfg::STAGE_BYTES;
      const int tail = p.hidden_in % BK;
      if constexpr (Cfg::A_DEPTH_MAJOR) ALoad::clear_depth_tail(st, tail);
      if constexpr (Cfg::B_DEPTH_MAJOR) BLoad::clear_depth_tail(st + Cfg::A_BYTES, tail);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      block_barrier();
    }
  };
  wait_vmcnt<3 * QUARTER_LOADS>();   // the first slice is in
  block_barrier();
  if (RAGGED_DEPTH && tail_slice == 0) clear_tail(0);
  static_for<2 * UNITS>([&](auto u) {
    constexpr int uu = decltype(u)::value;
    read_unit(std::integral_constant<int, uu % UNITS>{}, std::integral_constant<int, uu / UNITS>{}, IMB{}, 0);
  });

  int x = 0;   // buffer of the slice being multiplied

  // Partial tile of depth piece `piece` of the tile `ti` names, as this thread sees it: a lane's
  // 16-byte group (i, j, q) sits at ((i * NB + j) * 4 + q) * NT + thread, so one instruction of a
  // wave moves 1 KiB of consecutive bytes.
  auto partial_slot = [&](const TileInfo& tile, int piece) {
    return reinterpret_cast<float*>(p.workspace + kWsCounterBytes) +
           (int64_t)(tile.rank * tile.pieces + piece) * (BM * BN) + threadIdx.x * 4;
  };
  bool fix_pending = false;   // this workgroup's depth piece was the last of its tile to arrive

  // One tile, for a wave that has ML row blocks with rows in them (the tile's row blocks go to
  // the wave rows alternately).  One copy of this body exists per value of ML; a tile picks
  // its copy once, so no accumulator ever lives across a choice.
  //
  // Per slice (buffer X, the other buffer Y holds the next slice):
  //   step 0  reads the fragments of steps 2 and 3 from X; after it nobody needs X any more
  //   step 1  barrier: X goes to the fetch cursor, which starts the slice two ahead into it
  //   step 3  barrier: Y is complete for every wave; reads the fragments of the next slice's
  //           steps 0 and 1 from Y (all MB of A's: the next slice may be the next tile's)
  // Every step issues a quarter of a slice's loads (step 0 the last quarter of the slice begun
  // in steps 1-3 before it), so the memory pipe sees a steady trickle, and X is released two
  // steps before Y is needed, so loads stay in flight across the hand-over.
  auto tile_body = [&](auto ml_tag) {
    constexpr int ML = decltype(ml_tag)::value;
    constexpr int SLOTS = ML * NB;    // MFMAs per 16-deep step
    f32x16 acc[ML][NB];
#pragma unroll
    for (int i = 0; i < ML; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // One 16-deep step: SLOTS slots of one MFMA each, with this step's LDS reads and global
    // loads placed behind the first MFMAs, in this order, so they run under the matrix pipe.
    //   RML     A fragments per set that are read (ML, or MB for the next slice's)
    //   SETS    sets read: 0 or 2, starting at READ_SET
    //   LOADS   global loads FIRST_LOAD .. of the fetch cursor's slice, into buffer `fill`
    auto step = [&](auto ks_tag, auto sets_tag, auto rml_tag, auto read_set_tag, auto first_load_tag,
                    auto loads_tag, int src, int fill) {
      constexpr int ks = decltype(ks_tag)::value, SETS = decltype(sets_tag)::value;
      constexpr int RML = decltype(rml_tag)::value, RUNITS = RML + NB, READS = SETS * RUNITS;
      constexpr int READ_SET = decltype(read_set_tag)::value;
      constexpr int FIRST_LOAD = decltype(first_load_tag)::value, LOADS = decltype(loads_tag)::value;
      // fp8: steps 2 s and 2 s + 1 share the 64-deep step s, half of the blocks each, and an
      // instruction takes the halves 2 s and 2 s + 1 of both fragments
      constexpr int STEP_SLOTS = F8 ? SLOTS / 2 : SLOTS;
      static_for<STEP_SLOTS>([&](auto m_tag) {
        constexpr int mm = decltype(m_tag)::value, m = F8 ? mm + (ks % 2) * STEP_SLOTS : mm;
        // serpentine over the blocks: consecutive MFMAs share one operand, also across rows
        constexpr int j = m / ML, i = (j % 2 == 0) ? m % ML : ML - 1 - m % ML;
        // operands swapped: the result block is held transposed, so a lane owns four
        // consecutive columns of one output row
        if constexpr (F8) {
          acc[i][j] = mfma_32x32x64_f8<DT>(fb[ks & ~1][j], fb[ks | 1][j], fa[ks & ~1][i], fa[ks | 1][i], acc[i][j]);
        } else {
          acc[i][j] = mfma_32x32x16<DT>(fb[ks][j], fa[ks][i], acc[i][j]);
        }
        constexpr int u0 = READS * mm / STEP_SLOTS, u1 = READS * (mm + 1) / STEP_SLOTS;
        static_for<u1 - u0>([&](auto d) {
          constexpr int u = u0 + decltype(d)::value;
          read_unit(std::integral_constant<int, u % RUNITS>{},
                    std::integral_constant<int, READ_SET + u / RUNITS>{}, rml_tag, src);
        });
        constexpr int l0 = LOADS * mm / STEP_SLOTS, l1 = LOADS * (mm + 1) / STEP_SLOTS;
        static_for<l1 - l0>([&](auto d) {
          fetch_load(std::integral_constant<int, FIRST_LOAD + l0 + decltype(d)::value>{}, fill);
        });
        __builtin_amdgcn_sched_barrier(0);
      });
    };

    for (int kt = 0; kt < ti.nk; ++kt) {
      const int y = uniform(x ^ 1);   // (the same in every lane: keeps the LDS addresses scalar)
      step(I0{}, I2{}, ml_tag, I2{}, IQ3{}, IQ{}, x, y);
      fetch_advance();
      // every wave has all fragments of this slice in registers
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      block_barrier();
      fetch_begin();
      step(I1{}, I0{}, ml_tag, I0{}, I0{}, IQ{}, x, x);
      step(I2{}, I0{}, ml_tag, I0{}, IQ{}, IQ{}, x, x);
      // the next slice has landed for every wave (only this slice's two quarters may be pending)
      wait_vmcnt<2 * QUARTER_LOADS>();
      block_barrier();
      if (RAGGED_DEPTH && uniform(kt + 1 == ti.nk ? 0 : kt + 1) == tail_slice) clear_tail(y);
      step(I3{}, I2{}, IMB{}, I0{}, IQ2{}, IQ{}, y, x);
      x = uniform(y);
    }

    // A depth piece of a tile of the last round: park the partial tile in the workspace and
    // count the arrival.  The piece that arrives last adds the partial tiles up and stores the
    // sum, after the tile loop (fix_up below), where no accumulator is live any more.
    if (DEPTH_PIECES && ti.pieces > 1) {
      float* mine = partial_slot(ti, ti.piece);
#pragma unroll
      for (int i = 0; i < ML; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            *reinterpret_cast<f32x4*>(mine + ((i * NB + j) * 4 + q) * (NT * 4)) = v;
          }
      __threadfence();   // the partial tile is visible device-wide before the arrival is counted
      block_barrier();
      if (threadIdx.x == 0) sched->arrived = atomicAdd(reinterpret_cast<int*>(p.workspace) + ti.rank, 1);
      block_barrier();
      fix_pending = uniform(sched->arrived) == ti.pieces - 1;
      if (fix_pending) {
        // Keep the tile's description for the fix-up after the tile loop (a piece of the last
        // round is this workgroup's last tile, one of a deep tile its first): copied from the
        // slot of the tile ring it was read from, which the fetch cursor, at most two tiles
        // ahead, has not reached again.  (Packing it from registers would keep every field live
        // through the depth loop, which has no scalar registers to spare.)
        static_assert(sizeof(sched->fix_tile) == kTileInfoDwords * 4 && kTileInfoDwords <= 64, "");
        if (threadIdx.x < kTileInfoDwords)
          sched->fix_tile[threadIdx.x] = tile_ring[(tile_n % Cfg::TILE_RING_SLOTS) * kTileInfoDwords + threadIdx.x];
      }
      return;
    }

    // Epilogue.  A lane owns row (l % 32) of each 32x32 block and columns 8q + 4(l/32) .. +3.
    // The accumulators stay in the accumulation registers; each value is moved out right
    // where it is converted, so the epilogue needs only a few vector registers.
    {
      constexpr int CE = ACC_F32 ? 4 : 2;   // bytes per element of c
      constexpr uint32_t OOR = INDEXED ? kOutOfRangeIndexed : kOutOfRange;
      // the descriptor covers the tile's rows of c, or all of c when rows go through an index
      const char* cbase = INDEXED ? p.c : p.c + (ti.g.c_off + (int64_t)ti.m0 * ti.g.n) * CE;
      const uint32_t cbytes = INDEXED ? p.c_bytes
                              : (ti.rows_valid > 0 ? (uint32_t)(ti.rows_valid * ti.g.n) * (uint32_t)CE : 0u);
      const __amdgpu_buffer_rsrc_t rc = make_rsrc(cbase, cbytes);
      // byte offset of row `row` of the tile in that descriptor (OOR: the row does not exist)
      auto row_offset = [&](int row) -> uint32_t {
        if constexpr (INDEXED) {
          if (row >= ti.rows_valid) return OOR;
          const int r = ti.g.row0 + ti.m0 + row;
          const uint32_t dst = p.c_rows != nullptr ? (uint32_t)p.c_rows[r] : (uint32_t)r;
          return dst < p.c_index_rows ? dst * (uint32_t)ti.g.n * 2u : OOR;   // no such row: not stored
        } else {
          return (uint32_t)(row * ti.g.n) * (uint32_t)CE;
        }
      };
      auto at = [&](uint32_t row_off, int col) -> uint32_t {
        return col < ti.g.n && (!INDEXED || row_off != OOR) ? row_off + (uint32_t)col * (uint32_t)CE : OOR;
      };
      auto take4 = [&](int i, int j, int q) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[r]) : "a"(acc[i][j][4 * q + r]));
        return round4<OUT_DT>(v[0], v[1], v[2], v[3]);
      };
      if constexpr (GATE_UP) {
        // Blocks 2 jp and 2 jp + 1 of a wave hold the gate and the up value of the same 32 output
        // columns, element for element: silu(gate) * up in fp32, one rounding, 8 bytes per lane.
#pragma unroll
        for (int i = 0; i < ML; ++i) {
          const uint32_t row_off = row_offset((wm + i * WAVES_M) * 32 + (lane & 31));
#pragma unroll
          for (int jp = 0; jp < NB / 2; ++jp) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              float o[4];
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float gate, up;
                asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(gate) : "a"(acc[i][2 * jp][4 * q + r]));
                asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(up) : "a"(acc[i][2 * jp + 1][4 * q + r]));
                o[r] = gate / (1.0f + __expf(-gate)) * up;
              }
              const int col = ti.n0 + wn * (Cfg::WTN / 2) + jp * 32 + 8 * q + 4 * (lane >> 5);
              __builtin_amdgcn_raw_buffer_store_b64(round4<OUT_DT>(o[0], o[1], o[2], o[3]), rc, at(row_off, col), 0,
                                                    kStoreStreaming);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      } else if constexpr (ACC_F32) {
        if constexpr (EPI == kEpiAccF32Atomic) {
          // c += product in fp32, by atomic additions that return nothing: the wave fires them and
          // moves on, where a read-add-write would wait for the reads (every element of c belongs
          // to one tile, so each gets exactly one addition per call and the result is the same).
          // One 32 x 32 block at a time goes through the wave's LDS strip, in as the 16-byte pieces
          // the lanes hold, out as one float per lane, 32 lanes to a row: an instruction then adds
          // to two complete 128-byte lines.
          static_assert(Cfg::STAGED_EPILOGUE, "the accumulating epilogue uses the waves' LDS strips");
          char* strip = smem + Cfg::EPILOGUE_OFFSET + wave * Cfg::EPILOGUE_WAVE_BYTES;
          constexpr int PITCH = Cfg::EPILOGUE_PITCH;   // 32 floats and 16 bytes of padding
          const int in_row = lane & 31, in_half = lane >> 5;
#pragma unroll
          for (int i = 0; i < ML; ++i) {
#pragma unroll
            for (int j = 0; j < NB; ++j) {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                f32x4 v;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[r]) : "a"(acc[i][j][4 * q + r]));
                *reinterpret_cast<f32x4*>(strip + in_row * PITCH + (8 * q + 4 * in_half) * 4) = v;
              }
              const int col = ti.n0 + wn * Cfg::WTN + j * 32 + (lane & 31);
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int srow = r * 2 + (lane >> 5);
                const float v = *reinterpret_cast<const float*>(strip + srow * PITCH + (lane & 31) * 4);
                const int row = (wm + i * WAVES_M) * 32 + srow;
                const uint32_t off = col < ti.g.n ? (uint32_t)(row * ti.g.n + col) * 4u : kOutOfRange;
                __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(v, rc, off, 0, 0);
              }
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        } else {
          // c += product in fp32.  The 4 consecutive columns a lane holds are 16 bytes of c:
          // read them, add, write them back; lanes l and l + 32 cover 32 contiguous bytes of a
          // row, four such instructions one 128-byte line.  All reads of a 32-row block row are
          // issued before the first addition: 16 in flight per lane measured faster than a
          // rolling 8 + 8.
#pragma unroll
          for (int i = 0; i < ML; ++i) {
            const int row = (wm + i * WAVES_M) * 32 + (lane & 31);
            uint32_t off[NB][4];
            u32x4 old[NB][4];
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const int col = ti.n0 + wn * Cfg::WTN + j * 32 + 8 * q + 4 * (lane >> 5);
                off[j][q] = col < ti.g.n ? (uint32_t)(row * ti.g.n + col) * 4u : kOutOfRange;
                old[j][q] = __builtin_amdgcn_raw_buffer_load_b128(rc, off[j][q], 0, 0);
              }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                f32x4 sum = __builtin_bit_cast(f32x4, old[j][q]);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                  float v;
                  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(acc[i][j][4 * q + r]));
                  sum[r] += v;
                }
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, sum), rc, off[j][q], 0, 0);
              }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      } else if constexpr (Cfg::STAGED_EPILOGUE) {
        // Through a strip of LDS private to the wave: 32 rows x 64 columns go in as the
        // 8-byte pieces the lanes hold and come out as 16 bytes per lane, 8 lanes per row, so
        // that one store instruction writes 8 complete 128-byte lines.
        char* strip = smem + Cfg::EPILOGUE_OFFSET + wave * Cfg::EPILOGUE_WAVE_BYTES;
        constexpr int PITCH = Cfg::EPILOGUE_PITCH;
        const int in_row = lane & 31, in_half = lane >> 5;
        const int out_row = lane >> 3, out_chunk = lane & 7;
        // an even width that is not a multiple of 8: rows of c then start on 4-byte boundaries
        // only, and the last 16-byte chunk of a row holds 2, 4 or 6 columns
        const bool ragged_width = uniform(ti.g.n & 7) != 0;
#pragma unroll
        for (int i = 0; i < ML; ++i) {
          uint32_t row_off[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) row_off[r] = row_offset((wm + i * WAVES_M) * 32 + r * 8 + out_row);
#pragma unroll
          for (int jp = 0; jp < NB / 2; ++jp) {
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
              for (int q = 0; q < 4; ++q)
                *reinterpret_cast<u32x2*>(strip + in_row * PITCH + (jj * 32 + 8 * q + 4 * in_half) * 2) =
                    take4(i, 2 * jp + jj, q);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const u32x4 v = *reinterpret_cast<const u32x4*>(strip + (r * 8 + out_row) * PITCH + out_chunk * 16);
              const int col = ti.n0 + wn * Cfg::WTN + jp * 64 + out_chunk * 8;
              // (whole chunks only: for widths that are multiples of 8 the same as col < n)
              __builtin_amdgcn_raw_buffer_store_b128(v, rc, col + 8 <= ti.g.n ? at(row_off[r], col) : OOR, 0,
                                                     kStoreStreaming);
              {
                if (ragged_width) {
                  const int valid = ti.g.n - col;   // columns of this lane's chunk that exist
                  const uint32_t off = at(row_off[r], col);
                  if (valid > 0 && valid < 8 && off != OOR) {
                    if (valid & 4) __builtin_amdgcn_raw_buffer_store_b64(u32x2{v[0], v[1]}, rc, off, 0, kStoreStreaming);
                    if (valid & 2)
                      __builtin_amdgcn_raw_buffer_store_b32((valid & 4) ? v[2] : v[0], rc, off + ((valid & 4) ? 8u : 0u), 0,
                                                            kStoreStreaming);
                  }
                }
              }
            }
            // keep the conversion of one strip from being hoisted over the stores of the
            // previous one: few accumulators are live in vector registers at a time
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < ML; ++i) {
          const uint32_t row_off = row_offset((wm + i * WAVES_M) * 32 + (lane & 31));
#pragma unroll
          for (int j = 0; j < NB; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int col = ti.n0 + wn * Cfg::WTN + j * 32 + 8 * q + 4 * (lane >> 5);
              __builtin_amdgcn_raw_buffer_store_b64(take4(i, j, q), rc, at(row_off, col), 0, kStoreStreaming);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
    }
  };

  while (true) {
    // row blocks of this tile that fall to this wave row: blocks wm, wm + WAVES_M, ...
    const int live = uniform((ti.blocks - wm + WAVES_M - 1) / WAVES_M);
    if constexpr (LAYOUT == kTN || MB == 1) {
      tile_body(IMB{});
    } else {
      static_assert(MB == 4, "one copy of the tile body per live block count 1..4");
      if (live >= 4) {
        tile_body(std::integral_constant<int, 4>{});
      } else if (live == 3) {
        tile_body(std::integral_constant<int, 3>{});
      } else if (live == 2) {
        tile_body(std::integral_constant<int, 2>{});
      } else {
        tile_body(std::integral_constant<int, 1>{});
      }
    }
    tile_t = uniform(tile_t + G);
    if (tile_t >= total_tiles) break;
    tile_n = uniform(tile_n + 1);
    ti = next_tile();
  }
  wait_vmcnt<0>();   // the zero-filling fetches past the last tile still write LDS

  // Fix-up of a tile that was cut along the depth: the tile this workgroup left in
  // Sched::fix_tile when its piece arrived last (a workgroup has at most one).  The partial tiles
  // are added up in piece order, two per step (their count is even), whichever piece does the
  // adding, so the result does not depend on timing.  One block row of 32 rows at a time: NB * 4
  // groups of 16 bytes per lane and piece.
  if (DEPTH_PIECES && fix_pending) {
    __syncthreads();   // (the description was written by the first threads of the workgroup)
    int32_t words[kTileInfoDwords];
#pragma unroll
    for (int i = 0; i < kTileInfoDwords; ++i) words[i] = sched->fix_tile[i];
    const TileInfo ft = unpack_tile(words);
    __threadfence();   // the other pieces' partial tiles are visible to this workgroup
    if (threadIdx.x == 0) reinterpret_cast<int*>(p.workspace)[ft.rank] = 0;   // leave the counters as they were found
    constexpr int CE = ACC_F32 ? 4 : 2;   // bytes per element of c
    const char* cbase = p.c + (ft.g.c_off + (int64_t)ft.m0 * ft.g.n) * CE;
    const uint32_t cbytes = ft.rows_valid > 0 ? (uint32_t)(ft.rows_valid * ft.g.n) * (uint32_t)CE : 0u;
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(cbase, cbytes);
    const int live = LAYOUT == kTN ? MB : (ft.blocks - wm + WAVES_M - 1) / WAVES_M;
    for (int i = 0; i < live; ++i) {
      f32x4 sum[NB][4];
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) sum[j][q] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      for (int piece = 0; piece < ft.pieces; piece += 2) {
        const float* from0 = partial_slot(ft, piece) + (i * NB * 4) * (NT * 4);
        const float* from1 = partial_slot(ft, piece + 1) + (i * NB * 4) * (NT * 4);
        f32x4 v0[NB][4], v1[NB][4];
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            v0[j][q] = *reinterpret_cast<const f32x4*>(from0 + (j * 4 + q) * (NT * 4));
            v1[j][q] = *reinterpret_cast<const f32x4*>(from1 + (j * 4 + q) * (NT * 4));
          }
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) sum[j][q] = (sum[j][q] + v0[j][q]) + v1[j][q];
      }
      // a lane owns row (l % 32) of each 32x32 block and columns 8q + 4(l/32) .. +3
      const int row = (wm + i * WAVES_M) * 32 + (lane & 31);
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = ft.n0 + wn * Cfg::WTN + j * 32 + 8 * q + 4 * (lane >> 5);
          const uint32_t off = col < ft.g.n ? (uint32_t)(row * ft.g.n + col) * (uint32_t)CE : kOutOfRange;
          if constexpr (ACC_F32) {
            const f32x4 old = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rc, off, 0, 0));
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, old + sum[j][q]), rc, off, 0, 0);
          } else {
            __builtin_amdgcn_raw_buffer_store_b64(
                round4<OUT_DT>(sum[j][q][0], sum[j][q][1], sum[j][q][2], sum[j][q][3]), rc, off, 0, kStoreStreaming);
          }
        }
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace gg
