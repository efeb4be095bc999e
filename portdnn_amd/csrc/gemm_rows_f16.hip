// Row-major binary16 GEMM  Y[m][n] = sum_k X[m][k] W[k][n]  with fp32
// accumulation on v_mfma_f32_32x32x16_f16 (gfx950): the 1x1 stride-1
// convolution in NHWC / HWCF (m = pixels, k = channels, n = features) and the
// plain row-major matmul.  No filter re-layout launch and no barrier in the
// main loop:
//
//   * A work-group keeps a slab W[0..K)[n0..n0+BN) of the filter in LDS in its
//     natural layout (feature index contiguous) for its whole life, filled
//     with global-to-LDS loads, and walks a range of 32- or 64-row blocks of
//     X; the waves take their work from a counter in LDS, so they never wait
//     for one another.
//   * The matrix instruction wants 8 consecutive reduction indices per lane
//     for both operands.  X has them contiguous in memory, so its operand is
//     one 16-byte buffer load per lane straight into registers.  W does not:
//     a lane reads TJ consecutive features of 8 consecutive reduction rows
//     (8 ds_read_b64 for TJ = 4) and transposes them in registers with
//     v_perm_b32 into the operands of TJ matrix instructions whose feature
//     index is interleaved, n = n0 + TJ * i + j for row i of instruction j.
//   * W is the instruction's A operand and X its B operand, so a lane ends up
//     with one output row and runs of 8 consecutive features: the result is
//     written with 16-byte stores, the two half-waves side by side.
//   * Reductions of 64 or 128 channels keep a row block's X in registers for
//     every 128-column group of the slab while the next block's X loads (8
//     waves); longer ones stream X a 64-channel chunk ahead of the multiplies
//     (16 waves, tasks = row block x column group).  A direct-to-register
//     operand load touches 32 cache lines per instruction, which is what
//     bounds the deep, small layers; the large ones are bound by the HBM
//     writes of Y.
//
// portDNN runs these layers through its matmul kernel
// (src/conv2d/im2col/launch.cc and src/matmul/kernels.h:26-133 for 1x1
// windows); accumulating in fp32 instead of half stays inside the 1e-2
// relative bar against it.
#include "snn_kernels.h"

namespace snn {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));

constexpr int kMaxGroups = 8;   // column groups per slab at most
constexpr int kChunk = 64;      // reduction indices per chunk of X operands
constexpr int kSteps = kChunk / 16;
constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;
constexpr size_t kMaxLdsBytes = 144 * 1024;
constexpr int kCUs = 256;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}

struct RowsGeom {
  int m_total, k_total, n_total;
  int slab_cols;       // BN: columns of W a work-group keeps in LDS
  int pitch;           // bytes per slab row in LDS (2 * BN)
  int n_slabs;
  int wgs_per_slab;
  int n_row_tasks;     // ceil(m_total / (32 * TM))
};

// TJ: 32-column blocks per column group (interleaved features).  TM: 32-row
// blocks per row task.  NCH == 0: X streams through a ring of register sets
// one 64-index chunk at a time and a task is (row task, column group).  NCH > 0
// (k_total == 64 * NCH): a register set holds a row task's X for the whole
// reduction, the wave walks all column groups of the slab with it and the
// next row task's X loads meanwhile, so X goes through the vector memory
// pipeline once per row task instead of once per column group.
template <int TJ, int TM, int NCH, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
    gemm_rows_f16_kernel(const _Float16* __restrict__ x,
                         const _Float16* __restrict__ w,
                         _Float16* __restrict__ y, RowsGeom g,
                         unsigned x_bytes, unsigned w_bytes,
                         unsigned y_bytes) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  __shared__ int lds_next_task;
  constexpr int kTaskRows = 32 * TM;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int c = lane & 31;   // X row / W operand row inside a block
  const int h = lane >> 5;   // which 8 of the 16 reduction indices of a step
  // Operand row c of a matrix instruction stands for the features
  // TJ * c_sw + j.  For TJ = 4 bits 1 and 2 of c are exchanged: accumulator
  // register v = 4 a + r of lane (c, h) then holds feature 4 * (8 a + 4 (r / 2)
  // + 2 h + r % 2) + j, so the 16-byte pieces the two half-waves store lie side
  // by side.  For TJ = 2 they already do (feature 2 * (8 a + 4 h + r) + j).
  const int c_sw = TJ == 4 ? (c & ~6) | ((c & 2) << 1) | ((c & 4) >> 1) : c;

  // Work-groups that share a slab sit on the same XCD (work-group b runs on
  // XCD b % 8), so one L2 serves all readers of that slab.
  const int n_wgs = static_cast<int>(gridDim.x);
  int lin = static_cast<int>(blockIdx.x);
  if (n_wgs % 8 == 0) lin = (lin & 7) * (n_wgs >> 3) + (lin >> 3);
  const int slab = lin / g.wgs_per_slab;
  const int rank = lin % g.wgs_per_slab;
  const int task_row_lo =
      static_cast<int>(static_cast<long>(rank) * g.n_row_tasks / g.wgs_per_slab);
  const int task_row_hi = static_cast<int>(static_cast<long>(rank + 1) *
                                           g.n_row_tasks / g.wgs_per_slab);
  const int n_row_tasks = task_row_hi - task_row_lo;
  const int col_groups = g.slab_cols / (32 * TJ);

  if (tid == 0) lds_next_task = 0;

  // ---- the slab: K rows of BN halves, no padding, loaded straight into LDS
  // (lane l of a wave load fills bytes 16 l .. 16 l + 15 of a 1 KiB block), all
  // of a wave's blocks in flight at once.
  {
    typedef __attribute__((address_space(3))) void* lds_ptr;
    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(w, w_bytes);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_blocks = g.k_total * g.pitch / 1024;
    const unsigned col0_bytes = static_cast<unsigned>(slab * g.slab_cols) * 2u;
    const unsigned row_bytes = static_cast<unsigned>(g.n_total) * 2u;
    const unsigned pitch = static_cast<unsigned>(g.pitch);
    for (int block = wave; block < n_blocks; block += WAVES) {
      const unsigned pos = static_cast<unsigned>(block) * 1024u + 16u * lane;
      const unsigned row = pos / pitch;
      const unsigned voff = row * row_bytes + col0_bytes + (pos - row * pitch);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          w_rsrc, (lds_ptr)(lds_raw + block * 1024), 16, voff, 0, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's blocks landed
  }
  __syncthreads();

  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t y_rsrc = make_rsrc(y, y_bytes);
  const unsigned x_row_bytes = static_cast<unsigned>(g.k_total) * 2u;
  const unsigned y_row_bytes = static_cast<unsigned>(g.n_total) * 2u;

  auto grab = [&]() -> int {
    int t = 0;
    if (lane == 0) t = atomicAdd(&lds_next_task, 1);
    return __builtin_amdgcn_readfirstlane(t);
  };
  // X operands of one 64-index chunk of row task `rt`: block b, step s ->
  // reduction indices 64 * chunk + 16 * s + 8 * h .. + 7 of row 32 b + c.
  auto load_x = [&](int rt, int chunk, uint4v (&dst)[TM][kSteps]) {
    const int row0 = (task_row_lo + rt) * kTaskRows;
    const unsigned soff = static_cast<unsigned>(chunk * kChunk) * 2u;
#pragma unroll
    for (int b = 0; b < TM; ++b) {
      const int row = row0 + 32 * b + c;
      const unsigned voff =
          row < g.m_total ? static_cast<unsigned>(row) * x_row_bytes +
                                static_cast<unsigned>(h) * 16u
                          : kOob;
#pragma unroll
      for (int s = 0; s < kSteps; ++s)
        dst[b][s] = __builtin_amdgcn_raw_buffer_load_b128(
            x_rsrc, voff + 32u * s, soff, 0);
    }
  };

  float16v acc[TM][TJ];
  auto zero_acc = [&]() {
#pragma unroll
    for (int b = 0; b < TM; ++b)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][j][v] = 0.f;
  };

  // One chunk of the reduction for column group cg.
  auto compute = [&](int cg, int chunk, const uint4v (&xr)[TM][kSteps]) {
    const unsigned char* const w_lane =
        lds_raw + (chunk * kChunk + 8 * h) * g.pitch +
        (cg * 32 * TJ + TJ * c_sw) * 2;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      // rows[t] = W[16 s + 8 h + t][TJ c_sw .. TJ c_sw + TJ - 1]
      unsigned rows[8][TJ / 2];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const unsigned char* p = w_lane + (16 * s + t) * g.pitch;
        if constexpr (TJ == 4) {
          const uint2v r = *reinterpret_cast<const uint2v*>(p);
          rows[t][0] = r[0];
          rows[t][1] = r[1];
        } else {
          rows[t][0] = *reinterpret_cast<const unsigned*>(p);
        }
      }
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        // operand of instruction j: feature TJ c_sw + j, 8 reduction indices
        uint4v f;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          f[q] = __builtin_amdgcn_perm(rows[2 * q + 1][j / 2],
                                       rows[2 * q][j / 2],
                                       (j & 1) ? 0x07060302u : 0x05040100u);
        const half8 wf = __builtin_bit_cast(half8, f);
#pragma unroll
        for (int b = 0; b < TM; ++b)
          acc[b][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
              wf, __builtin_bit_cast(half8, xr[b][s]), acc[b][j], 0, 0, 0);
      }
    }
  };

  // Lane (c, h) holds output row c; per group a of four accumulator registers
  // its values are consecutive features (see c_sw above): for TJ = 4 two runs
  // of 8 (r / 2 = 0, 1) at 32 a + 16 (r / 2) + 8 h, for TJ = 2 one run of 8 at
  // 16 a + 8 h.
  auto store_tile = [&](int rt, int cg) {
    const int row0 = (task_row_lo + rt) * kTaskRows;
    const int col0 = slab * g.slab_cols + cg * 32 * TJ;
#pragma unroll
    for (int b = 0; b < TM; ++b) {
      const int row = row0 + 32 * b + c;
      const unsigned voff =
          row < g.m_total ? static_cast<unsigned>(row) * y_row_bytes +
                                static_cast<unsigned>(col0 + 8 * h) * 2u
                          : kOob;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int e = 0; e < TJ / 2; ++e) {
          half8 v8;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int r = TJ == 4 ? 2 * e + i / 4 : i / 2;
            v8[i] = static_cast<_Float16>(acc[b][i % TJ][4 * a + r]);
          }
          __builtin_amdgcn_raw_buffer_store_b128(
              __builtin_bit_cast(uint4v, v8), y_rsrc,
              voff + static_cast<unsigned>(a * 16 * TJ + e * 32), 0, 0);
        }
      }
    }
  };

  if constexpr (NCH == 0) {
    // ---- streaming: tasks are (row task, column group); two register sets,
    // the X loads run one chunk ahead of the multiplies.
    const int n_tasks = n_row_tasks * col_groups;
    const int n_chunks = g.k_total / kChunk;
    int task = grab();
    if (task >= n_tasks) return;
    int chunk = 0;
    int next_task = grab();
    uint4v xa[TM][kSteps], xb[TM][kSteps];
    load_x(task / col_groups, 0, xa);
    zero_acc();
    // One (task, chunk) step: start the loads of the step after it, multiply,
    // and finish the task after its last chunk.  Returns false after the last
    // step of the wave.
    auto step = [&](const uint4v (&cur)[TM][kSteps],
                    uint4v (&nxt)[TM][kSteps]) -> bool {
      const bool last_chunk = chunk + 1 == n_chunks;
      const bool more = !last_chunk || next_task < n_tasks;
      if (more)
        load_x((last_chunk ? next_task : task) / col_groups,
               last_chunk ? 0 : chunk + 1, nxt);
      compute(task % col_groups, chunk, cur);
      if (!last_chunk) {
        ++chunk;
        return true;
      }
      store_tile(task / col_groups, task % col_groups);
      if (!more) return false;
      zero_acc();
      task = next_task;
      chunk = 0;
      next_task = grab();
      return true;
    };
    for (;;) {
      if (!step(xa, xb)) break;
      if (!step(xb, xa)) break;
    }
  } else {
    // ---- X resident: a job is a row task with a range of column groups.  The
    // first n_full jobs (a multiple of the wave count) take all column groups
    // of a row task; the row tasks left over are dealt one column group at a
    // time so that the last round of the work-group's waves is even.
    const int n_full = n_row_tasks / WAVES * WAVES;
    const int n_jobs = n_full + (n_row_tasks - n_full) * col_groups;
    auto job_row = [&](int job) {
      return job < n_full ? job : n_full + (job - n_full) / col_groups;
    };
    int job = grab();
    if (job >= n_jobs) return;
    int next_job = grab();
    uint4v xa[NCH][TM][kSteps], xb[NCH][TM][kSteps];
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) load_x(job_row(job), ch, xa[ch]);
    auto run_job = [&](const uint4v (&cur)[NCH][TM][kSteps],
                       uint4v (&nxt)[NCH][TM][kSteps]) -> bool {
      const bool more = next_job < n_jobs;
      if (more) {
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) load_x(job_row(next_job), ch, nxt[ch]);
      }
      const int rt = job_row(job);
      const int cg_lo = job < n_full ? 0 : (job - n_full) % col_groups;
      const int cg_hi = job < n_full ? col_groups : cg_lo + 1;
      for (int cg = cg_lo; cg < cg_hi; ++cg) {
        zero_acc();
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) compute(cg, ch, cur[ch]);
        store_tile(rt, cg);
      }
      if (!more) return false;
      job = next_job;
      next_job = grab();
      return true;
    };
    for (;;) {
      if (!run_job(xa, xb)) break;
      if (!run_job(xb, xa)) break;
    }
  }
}

struct RowsPlan {
  int tj, tm, nch;
  RowsGeom g;
  size_t lds_bytes;
  int n_wgs;
};

bool plan_rows(int m, int k, int n, RowsPlan* plan) {
  if (m < 1 || k < kChunk || k % kChunk != 0 || n % 64 != 0) return false;
  if (static_cast<size_t>(m) * k * 2 > kMaxBufferBytes ||
      static_cast<size_t>(m) * n * 2 > kMaxBufferBytes ||
      static_cast<size_t>(k) * n * 2 > kMaxBufferBytes)
    return false;
  for (int tj = 4; tj >= 2; tj -= 2) {
    for (int groups = kMaxGroups; groups >= 1; --groups) {
      const int bn = groups * 32 * tj;
      if (n % bn != 0) continue;
      const size_t lds = static_cast<size_t>(k) * 2 * bn;
      if (lds > kMaxLdsBytes) continue;
      // X stays in registers for the whole reduction when that is one or two
      // chunks; longer reductions stream it.
      plan->nch = k <= 2 * kChunk ? k / kChunk : 0;
      plan->tm = plan->nch == 1 ? 2 : 1;
      RowsGeom& g = plan->g;
      g.m_total = m; g.k_total = k; g.n_total = n;
      g.slab_cols = bn;
      g.pitch = 2 * bn;
      g.n_slabs = n / bn;
      g.n_row_tasks = ceil_div(m, 32 * plan->tm);
      g.wgs_per_slab = kCUs / g.n_slabs;
      if (g.wgs_per_slab < 1) g.wgs_per_slab = 1;
      if (g.wgs_per_slab > g.n_row_tasks) g.wgs_per_slab = g.n_row_tasks;
      plan->tj = tj;
      plan->lds_bytes = lds;
      plan->n_wgs = g.n_slabs * g.wgs_per_slab;
      return true;
    }
  }
  return false;
}

template <int TJ, int TM, int NCH, int WAVES>
int launch_rows_as(const _Float16* x, const _Float16* w, _Float16* y,
                   const RowsPlan& plan, hipStream_t stream) {
  auto kernel = gemm_rows_f16_kernel<TJ, TM, NCH, WAVES>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize,
      static_cast<int>(kMaxLdsBytes));
  if (attr != hipSuccess) return report_hip_error(attr, "gemm_rows_f16_kernel");
  const RowsGeom& g = plan.g;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(
      kernel, dim3(static_cast<unsigned>(plan.n_wgs)), dim3(64 * WAVES),
      plan.lds_bytes, stream, x, w, y, g,
      static_cast<unsigned>(static_cast<size_t>(g.m_total) * g.k_total * 2),
      static_cast<unsigned>(static_cast<size_t>(g.k_total) * g.n_total * 2),
      static_cast<unsigned>(static_cast<size_t>(g.m_total) * g.n_total * 2));
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

template <int TJ>
int launch_rows_tj(const _Float16* x, const _Float16* w, _Float16* y,
                   const RowsPlan& plan, hipStream_t stream) {
  if (plan.nch == 1) return launch_rows_as<TJ, 2, 1, 8>(x, w, y, plan, stream);
  if (plan.nch == 2) return launch_rows_as<TJ, 1, 2, 8>(x, w, y, plan, stream);
  return launch_rows_as<TJ, 1, 0, 16>(x, w, y, plan, stream);
}

}  // namespace

bool gemm_rows_f16_supports(int m, int k, int n) {
  static const bool off = SNN_TUNING_ENV("SNN_HIP_F16_ROWS_OFF") != nullptr;
  RowsPlan plan;
  return !off && (gemm_wreg_f16_supports(m, k, n) || plan_rows(m, k, n, &plan));
}

int launch_gemm_rows_f16(const _Float16* x, const _Float16* w, _Float16* y,
                         int m, int k, int n, hipStream_t stream) {
  if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
        reinterpret_cast<uintptr_t>(y)) & 15u) != 0)
    return SNN_HIP_INVALID_PARAMETER;
  // short reductions: the kernel that keeps the filter in registers
  if (gemm_wreg_f16_supports(m, k, n)) {
    launch_gemm_wreg_f16(x, w, y, m, k, n, stream);
    return SNN_HIP_OK;
  }
  RowsPlan plan;
  if (!plan_rows(m, k, n, &plan)) return SNN_HIP_INVALID_ALGORITHM;
  return plan.tj == 4 ? launch_rows_tj<4>(x, w, y, plan, stream)
                      : launch_rows_tj<2>(x, w, y, plan, stream);
}

}  // namespace snn
