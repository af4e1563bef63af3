// Grouped GEMM for the shapes and element types the streaming kernel (gmm_kernel.hpp) does not
// take: hidden sizes that are not multiples of 8, operands that do not start on a 16-byte
// boundary, one-byte (fp8) elements, and row indices on every layout.  The reference's default
// build runs any hidden size through cuBLAS (csrc/grouped_gemm.cu:373-394); this is that
// generality, not that speed.
//
// Same schedule (build_schedule / find_tile), same matrix instructions and fp32 accumulation as
// the streaming kernel; what differs is how operands reach LDS.  Here they go through
// registers, VEC elements at a time along whichever dimension is contiguous in memory (VEC is the
// largest of 8, 4, 2, 1 that divides both hidden sizes and fits the pointers' alignment), every
// vector checked against the group's bounds, and are laid down in LDS depth-contiguous whatever
// their layout in memory, so that one fragment reader serves all three layouts.
#pragma once

#include "gmm_kernel.hpp"

namespace gg {

template <int DT>
struct ElemTraits {
  static constexpr int BYTES = is_f8(DT) ? 1 : 2;
  static constexpr int OUT_DT = DT == kF16 ? kF16 : kBF16;   // element type of c
};

struct GenericParams {
  GmmParams p;
  const int32_t* a_rows;   // row r of `a` as the product sees it is row a_rows[r] in memory, or nullptr
  const int32_t* b_rows;   // the same for b (weight-gradient layout only), or nullptr
  const int32_t* c_rows;   // row r of the output goes to row c_rows[r] of c (not the weight gradient), or nullptr
  // rows of a, b and c in memory: an index that names no row of its tensor is a missing row (read
  // as zeros, not stored), as on the streaming kernels
  int64_t a_num_rows, b_num_rows, c_num_rows;
};

namespace generic {

constexpr int BM = 128, BN = 128, BK = 32, THREADS = 256;
constexpr int PAD = 8;   // elements; keeps 8-element chunks aligned and spreads rows over the banks

template <int BYTES>
struct Frag;
template <>
struct Frag<2> {
  using type = bf16x8;
};
template <>
struct Frag<1> {
  using type = long;
};

template <int DT>
__device__ __forceinline__ f32x16 mfma(typename Frag<ElemTraits<DT>::BYTES>::type x,
                                       typename Frag<ElemTraits<DT>::BYTES>::type y, f32x16 acc) {
  if constexpr (DT == kF8E4M3) {
    return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(x, y, acc, 0, 0, 0);
  } else if constexpr (DT == kF8E5M2) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(x, y, acc, 0, 0, 0);
  } else {
    return mfma_32x32x16<DT>(x, y, acc);
  }
}

// One operand tile: ROWS indices i (rows of A, columns of B) by BK depth values k.  In memory the
// element (i, k) sits at base + i * stride_i + k * stride_k (elements), one of the strides being 1;
// `rows` optionally redirects the index of the strided dimension through an index array.
// GATE_UP (B with gate | up columns): the tile's 128 indices are 32-index blocks taken alternately
// from the gate columns [0, out_cols) and the up columns [out_cols, 2 out_cols); i0 and i_end then
// count output columns.
template <int ES, int VEC, bool K_CONTIGUOUS, bool GATE_UP = false>
struct TileLoader {
  static constexpr int VECS = BM * BK / VEC;         // vectors per tile
  static constexpr int PER_THREAD = VECS / THREADS;
  static_assert(VECS % THREADS == 0, "");

  const char* base;      // group's element (0, 0)
  int64_t ld;            // elements between consecutive indices of the strided dimension
  int i0, i_end;         // the tile's first index and the group's index count
  int k_end;             // the group's depth
  const int32_t* index;  // rows of the strided dimension in memory, or nullptr
  int index_base;        // position of the group's first row in `index`
  int64_t index_rows;    // rows the indexed tensor has in memory
  int out_cols;          // GATE_UP: output columns of the group

  uint32_t regs[PER_THREAD][VEC * ES > 4 ? VEC * ES / 4 : 1];

  // where vector v of the tile sits: (i, k) of its first element
  __device__ __forceinline__ static void coords(int v, int* i, int* k) {
    if (K_CONTIGUOUS) {
      *i = v / (BK / VEC);
      *k = (v % (BK / VEC)) * VEC;
    } else {
      *k = v / (BM / VEC);
      *i = (v % (BM / VEC)) * VEC;
    }
  }

  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int n = 0; n < PER_THREAD; ++n) {
      int i, k;
      coords(threadIdx.x + n * THREADS, &i, &k);
      int gi = i0 + i;
      const int gk = k0 + k;
      bool inside = gi < i_end;
      if constexpr (GATE_UP) {
        const int block = i >> 5, out = i0 + (block >> 1) * 32 + (i & 31);
        inside = out < i_end;
        gi = (block & 1) * out_cols + out;
      }
#pragma unroll
      for (int w = 0; w < (VEC * ES > 4 ? VEC * ES / 4 : 1); ++w) regs[n][w] = 0;
      bool present = inside && gk < k_end;   // extents are multiples of VEC: a vector is all in or all out
      int64_t strided = K_CONTIGUOUS ? gi : gk;
      if (present && index != nullptr) {
        strided = index[index_base + strided];
        present = strided >= 0 && strided < index_rows;   // an index that names no row: zeros
      }
      if (present) {
        const char* src = base + (strided * ld + (K_CONTIGUOUS ? gk : gi)) * ES;
        constexpr int NB = VEC * ES;
        if constexpr (NB == 1) {
          regs[n][0] = *reinterpret_cast<const uint8_t*>(src);
        } else if constexpr (NB == 2) {
          regs[n][0] = *reinterpret_cast<const uint16_t*>(src);
        } else if constexpr (NB == 4) {
          regs[n][0] = *reinterpret_cast<const uint32_t*>(src);
        } else if constexpr (NB == 8) {
          const u32x2 t = *reinterpret_cast<const u32x2*>(src);
          regs[n][0] = t[0], regs[n][1] = t[1];
        } else {
          const u32x4 t = *reinterpret_cast<const u32x4*>(src);
          regs[n][0] = t[0], regs[n][1] = t[1], regs[n][2] = t[2], regs[n][3] = t[3];
        }
      }
    }
  }

  // LDS keeps T[i][k] with k contiguous, rows of (BK + PAD) elements.
  __device__ __forceinline__ void stash(char* tile) const {
    constexpr int PITCH = (BK + PAD) * ES;
#pragma unroll
    for (int n = 0; n < PER_THREAD; ++n) {
      int i, k;
      coords(threadIdx.x + n * THREADS, &i, &k);
      if (K_CONTIGUOUS) {
        char* dst = tile + i * PITCH + k * ES;
        constexpr int NB = VEC * ES;
        if constexpr (NB == 1) {
          *reinterpret_cast<uint8_t*>(dst) = (uint8_t)regs[n][0];
        } else if constexpr (NB == 2) {
          *reinterpret_cast<uint16_t*>(dst) = (uint16_t)regs[n][0];
        } else if constexpr (NB == 4) {
          *reinterpret_cast<uint32_t*>(dst) = regs[n][0];
        } else if constexpr (NB == 8) {
          *reinterpret_cast<u32x2*>(dst) = u32x2{regs[n][0], regs[n][1]};
        } else {
          *reinterpret_cast<u32x4*>(dst) = u32x4{regs[n][0], regs[n][1], regs[n][2], regs[n][3]};
        }
      } else {
        // the vector runs along i: its elements go to VEC different rows of the LDS tile
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const uint32_t word = regs[n][e * ES / 4];
          char* dst = tile + (i + e) * PITCH + k * ES;
          if constexpr (ES == 2) {
            *reinterpret_cast<uint16_t*>(dst) = (uint16_t)(word >> (16 * (e % 2)));
          } else {
            *reinterpret_cast<uint8_t*>(dst) = (uint8_t)(word >> (8 * (e % 4)));
          }
        }
      }
    }
  }
};

// DT element type; VEC elements per memory access; the output is c in ElemTraits<DT>::OUT_DT, or
// fp32 added to when ACC_F32.
template <int DT, int LAYOUT, int VEC, int EPI>
__global__ __launch_bounds__(THREADS) void gmm_generic_kernel(GenericParams gp, HostSizes hs) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr bool ACC_F32 = EPI == kEpiAccF32, GATE_UP = EPI == kEpiSwiGLU;
  constexpr int BNS = GATE_UP ? BN / 2 : BN;   // output columns per tile
  constexpr int ES = ElemTraits<DT>::BYTES;
  constexpr int OUT_DT = ElemTraits<DT>::OUT_DT;
  constexpr int PITCH = (BK + PAD) * ES;
  using FragT = typename Frag<ES>::type;
  const GmmParams& p = gp.p;

  __shared__ Sched sched;
  __shared__ __attribute__((aligned(16))) char tile_a[BM * PITCH];
  __shared__ __attribute__((aligned(16))) char tile_b[BN * PITCH];
  build_schedule<LAYOUT, BM, BNS>(&sched, p, hs);
  __syncthreads();
  static_assert(sizeof(tile_a) >= kMaxGroups * sizeof(uint64_t), "the sort keys borrow a tile buffer");
  if constexpr (LAYOUT == kTN) order_groups_by_depth(&sched, p.num_groups, reinterpret_cast<uint64_t*>(tile_a));

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;   // 2 x 2 waves of 64 x 64 outputs

  TailPlan plan;   // whole tiles only
  plan.main_tiles = plan.total = sched.tile_start[p.num_groups] + sched.runt_start[p.num_groups];
  plan.pieces = 1;
  plan.by_depth = false;

  TileLoader<ES, VEC, LAYOUT != kTN> aload;
  TileLoader<ES, VEC, LAYOUT == kNT, GATE_UP> bload;
  TileCursor cur;
  for (int t = blockIdx.x; t < plan.total; t += gridDim.x) {
    const TileInfo ti = find_tile<LAYOUT, BM, BNS, BK>(&sched, p, t, plan, cur);
    const int group_row = (int)(ti.g.a_off / p.hidden_in);   // first row of the group in `a`
    // A: NN / NT rows of `a` (depth contiguous); weight gradient: columns of a^T (rows contiguous)
    if (LAYOUT != kTN) {
      aload.base = gp.a_rows ? p.a : p.a + ti.g.a_off * ES;
      aload.ld = ti.g.k;
      aload.i0 = ti.m0, aload.i_end = ti.m0 + ti.rows_valid;
    } else {
      aload.base = gp.a_rows ? p.a : p.a + ti.g.a_off * ES;
      aload.ld = ti.g.m;
      aload.i0 = ti.m0, aload.i_end = ti.g.m;
    }
    aload.k_end = ti.depth;
    aload.index = gp.a_rows;
    aload.index_base = group_row;
    aload.index_rows = gp.a_num_rows;
    // B: NN rows of b[e] are depth rows (columns contiguous); NT rows are output columns (depth
    // contiguous); weight gradient: rows of b are depth rows
    if (LAYOUT == kTN) {
      bload.base = gp.b_rows ? p.b : p.b + ti.g.b_off * ES;
      bload.index = gp.b_rows;
      bload.index_base = group_row;
      bload.index_rows = gp.b_num_rows;
    } else {
      bload.base = p.b + ti.g.b_off * ES;
      bload.index = nullptr;
      bload.index_base = 0;
      bload.index_rows = 0;
    }
    bload.ld = LAYOUT == kNT ? ti.g.k : (GATE_UP ? 2 * ti.g.n : ti.g.n);
    bload.i0 = ti.n0, bload.i_end = ti.g.n;
    bload.out_cols = ti.g.n;
    bload.k_end = ti.depth;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    aload.fetch(0);
    bload.fetch(0);
    for (int kt = 0; kt < ti.nk; ++kt) {
      __syncthreads();   // everybody is done reading the previous slice
      aload.stash(tile_a);
      bload.stash(tile_b);
      __syncthreads();
      if (kt + 1 < ti.nk) {   // the next slice travels while this one is multiplied
        aload.fetch((kt + 1) * BK);
        bload.fetch((kt + 1) * BK);
      }
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        FragT fa[2], fb[2];
        const int koff = (ks * 16 + 8 * (lane >> 5)) * ES;
#pragma unroll
        for (int i = 0; i < 2; ++i)
          fa[i] = *reinterpret_cast<const FragT*>(tile_a + (wm * 64 + i * 32 + (lane & 31)) * PITCH + koff);
#pragma unroll
        for (int j = 0; j < 2; ++j)
          fb[j] = *reinterpret_cast<const FragT*>(tile_b + (wn * 64 + j * 32 + (lane & 31)) * PITCH + koff);
        // operands swapped: a lane ends up with four consecutive columns of one output row
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = mfma<DT>(fb[j], fa[i], acc[i][j]);
      }
    }

    // Epilogue: a lane owns row (l % 32) of each 32 x 32 block and columns 8q + 4 (l / 32) .. +3.
    constexpr int CE = ACC_F32 ? 4 : 2;
    char* cbase = p.c + (gp.c_rows ? (int64_t)0 : ti.g.c_off * CE);
    const int out_row0 = LAYOUT == kTN ? 0 : (int)(ti.g.c_off / ti.g.n);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = ti.m0 + wm * 64 + i * 32 + (lane & 31);
      if (row >= ti.m0 + ti.rows_valid) continue;
      int64_t mem_row = row;
      if (gp.c_rows) {
        mem_row = gp.c_rows[out_row0 + row];
        if (mem_row < 0 || mem_row >= gp.c_num_rows) continue;   // an index that names no row: not stored
      }
      char* crow = cbase + mem_row * ti.g.n * CE;
      if constexpr (GATE_UP) {
        // blocks 0 and 1 of the wave hold the gate and the up value of the same 32 output columns
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = ti.n0 + wn * 32 + 8 * q + 4 * (lane >> 5);
          uint16_t* dst = reinterpret_cast<uint16_t*>(crow) + col;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float gate = acc[i][0][4 * q + r], up = acc[i][1][4 * q + r];
            const u32x2 one = round4<OUT_DT>(gate / (1.0f + __expf(-gate)) * up, 0.0f, 0.0f, 0.0f);
            if (col + r < ti.g.n) dst[r] = (uint16_t)one[0];
          }
        }
        continue;
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = ti.n0 + wn * 64 + j * 32 + 8 * q + 4 * (lane >> 5);
          if (col >= ti.g.n) continue;   // n is a multiple of VEC: a group of VEC columns is all in or all out
          if constexpr (ACC_F32) {
            float* dst = reinterpret_cast<float*>(crow) + col;
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (VEC >= 4 || col + r < ti.g.n) dst[r] += acc[i][j][4 * q + r];
          } else {
            const u32x2 packed = round4<OUT_DT>(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                                acc[i][j][4 * q + 3]);
            char* dst = crow + col * 2;
            if constexpr (VEC >= 4) {
              *reinterpret_cast<u32x2*>(dst) = packed;
            } else if constexpr (VEC == 2) {
              *reinterpret_cast<uint32_t*>(dst) = packed[0];
              if (col + 2 < ti.g.n) *reinterpret_cast<uint32_t*>(dst + 4) = packed[1];
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r)
                if (col + r < ti.g.n)
                  *reinterpret_cast<uint16_t*>(dst + 2 * r) = (uint16_t)(packed[r / 2] >> (16 * (r % 2)));
            }
          }
        }
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace generic
}  // namespace gg
