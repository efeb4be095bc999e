// MFMA tile machinery shared by the implicit-GEMM convolution and the matmul
// kernels (gfx950, wave64).
//
// A work-group of 256 lanes (4 waves, one per SIMD) owns a BM x BN output tile
// and walks the reduction in chunks of BK = 32.  Both operand tiles are staged
// in LDS in one of two layouts, chosen so that the global->LDS copy is always
// a 16-byte load and a 16-byte LDS store along the dimension that is
// contiguous in memory (no transposes anywhere):
//
//   K-inner   tile[row][BK + 4]    reduction index contiguous.  A lane fetches
//                                  four consecutive k with one ds_read_b128;
//                                  the +4 word pad makes eight consecutive rows
//                                  cover all 32 banks exactly once.
//   row-inner tile[BK][rows + 4]   row (m or n) index contiguous.  A lane
//                                  fetches one word per k; 32 consecutive lanes
//                                  read 32 consecutive words.
//
// The contraction runs on v_mfma_f32_32x32x2_f32: per instruction lane l
// supplies A[row = l % 32][k = l / 32] and B[k = l / 32][col = l % 32] and the
// 32x32 result tile lives in 16 accumulator registers per lane
// (row = 8 * (v / 4) + 4 * (l / 32) + v % 4, col = l % 32).  Any assignment of
// reduction indices to (instruction, lane half) is valid as long as A and B
// agree; here sub-step s of a BK chunk and instruction t in it use
// k = 8 * s + 4 * (l / 32) + t, which is what makes the ds_read_b128 fetch of
// a K-inner operand line up with four consecutive MFMAs.
#ifndef PORTDNN_AMD_CSRC_GEMM_TILE_H_
#define PORTDNN_AMD_CSRC_GEMM_TILE_H_

#include <hip/hip_runtime.h>

namespace snn {
namespace gemm {

constexpr int kBK = 32;        // reduction chunk per LDS stage
constexpr int kThreads = 256;  // 4 waves
constexpr int kPad = 4;        // words of padding per LDS row

typedef float float16v __attribute__((ext_vector_type(16)));

// LDS footprint (floats) of one stage of an operand tile with `rows` rows.
constexpr int k_inner_floats(int rows) { return rows * (kBK + kPad); }
constexpr int row_inner_floats(int rows) { return kBK * (rows + kPad); }

// Fetch the four A (or B) values lane `lane` needs for sub-step `s` from a
// K-inner tile; `row` is the tile row this lane serves.
__device__ inline float4 fetch_k_inner(const float* tile, int row, int s,
                                       int lane) {
  return *reinterpret_cast<const float4*>(
      tile + row * (kBK + kPad) + 8 * s + 4 * (lane >> 5));
}

// Same for a row-inner tile with `rows` rows.
template <int ROWS>
__device__ inline float4 fetch_row_inner(const float* tile, int row, int s,
                                         int lane) {
  const float* p = tile + (8 * s + 4 * (lane >> 5)) * (ROWS + kPad) + row;
  float4 v;
  v.x = p[0];
  v.y = p[ROWS + kPad];
  v.z = p[2 * (ROWS + kPad)];
  v.w = p[3 * (ROWS + kPad)];
  return v;
}

__device__ inline float comp(const float4& v, int t) {
  return t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
}

// One BK chunk of MFMA work for a wave tile of TM x TN 32x32 blocks.
// a_tile / b_tile point at the current LDS stage; a_row0 / b_row0 are the
// first tile rows (m resp. n) of this wave.  Every operand of the chunk is
// fetched from LDS up front (the fetches of the second half overlap the MFMAs
// of the first), so the matrix pipe is not gated by one LDS round trip per
// instruction pair.
template <int TM, int TN, bool A_K_INNER, bool B_K_INNER, int A_ROWS,
          int B_ROWS>
__device__ inline void mma_chunk(const float* a_tile, const float* b_tile,
                                 int a_row0, int b_row0, int lane,
                                 float16v (&acc)[TM][TN]) {
  constexpr int S = kBK / 8;  // sub-steps of 8 reduction indices
  const int l32 = lane & 31;
  float4 a[S][TM], b[S][TN];
#pragma unroll
  for (int s = 0; s < S; ++s) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      a[s][i] = A_K_INNER
                    ? fetch_k_inner(a_tile, a_row0 + 32 * i + l32, s, lane)
                    : fetch_row_inner<A_ROWS>(a_tile, a_row0 + 32 * i + l32, s,
                                              lane);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      b[s][j] = B_K_INNER
                    ? fetch_k_inner(b_tile, b_row0 + 32 * j + l32, s, lane)
                    : fetch_row_inner<B_ROWS>(b_tile, b_row0 + 32 * j + l32, s,
                                              lane);
    }
  }
  // Keep the compiler's scheduler from sinking the fetches back down between
  // the MFMAs (it would, to save registers).
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < S; ++s) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              comp(a[s][i], t), comp(b[s][j], t), acc[i][j], 0, 0, 0);
        }
      }
    }
  }
}

// Work-groups are handed to the 8 XCDs round-robin (group b runs on XCD b % 8)
// and each XCD has its own L2.  This maps the hardware group id to a logical
// tile id so that every XCD works on one contiguous run of logical tiles:
// neighbouring tiles (which share operand rows) then share an L2.
__device__ inline unsigned xcd_remap(unsigned b, unsigned n_blocks) {
  constexpr unsigned kXcds = 8;
  const unsigned per = n_blocks / kXcds;  // full rounds
  const unsigned main = per * kXcds;
  if (b >= main) return b;  // ragged tail keeps its id
  return (b % kXcds) * per + b / kXcds;
}

}  // namespace gemm
}  // namespace snn

#endif  // PORTDNN_AMD_CSRC_GEMM_TILE_H_
