// Products of some dozens to about a thousand rows on the matrix cores: y = x . w^T, bfloat16
// operands, float32 accumulation.  The reference leaves every product to its vendor library
// (yalis/external/model.py:449, 462-466, 717-722), and so does this engine for many rows; between
// the few-row product and those, the vendor library's tiles are few on the narrow matrices of a
// layer (512 rows x 3,072 columns: 24 to 48 tiles for 256 compute units), which this kernel
// answers with tiles of 128 x 128 cut along K as well (the unreduced K slices go to the same
// consumers that add the few-row product's slices).  What it wins, and so what it is used for
// (HipOps.mid_rows_product): 65 to 256 rows against matrices at least twice as long as wide,
// the down projections (us at 128 rows, vendor library's first candidate / few-row kernel / this:
// 8B shape 57.9 / 35.4 / 27.0, 3B 32.9 / 19.6 / 17.7, 70B 200 / 167 / 110).  From 384 rows on, and
// for gate/up at any number of rows, the library is faster (8B shape at 512 rows, library / this:
// qkv 31.3 / 48.4, o-proj 24.8 / 29.0, gate/up 85.8 / 152, down 74.4 / 81.8): a step of this
// kernel moves 96 KiB through LDS for 64 products, and the LDS, not the matrix cores, bounds it
// (writes of 16 bytes a lane run at about a third of the nominal 128 bytes a clock).
//
// A workgroup of four waves owns a tile of 128 rows of w (output features) x 128 rows of x
// (tokens) over one slice of K, walked in steps of 64.  Each wave owns 64 x 64 of it as 2 x 2
// products of v_mfma_f32_32x32x16_bf16 (A = 32 rows of w, B = 32 rows of x; see the wide form of
// the few-row product for the operand layout).  Both operands of a step are fetched with 16-byte
// loads (eight lanes a row of 128 bytes), parked in LDS in rows padded to 144 bytes (operand reads
// of 16 bytes a lane then meet no bank twice) and read from there by all four waves.  The loads
// of the step after next are in flight while a step is multiplied (two register sets by turns,
// two LDS buffers by turns, one barrier a step).  Rows beyond M or N are read from the last row
// and never stored; K beyond the slice is read from valid places and meets zeros of x.
//
// Workgroup i of a launch runs on die i % 8: the tiles that share 128 rows of w (all row blocks of
// x) are given numbers 8 apart, so that they meet in one die's L2.
#include <algorithm>

#include "common.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

union Frag8 {
  u32x4_t u;
  bf16x8_t v;
};

constexpr int GT_BM = 128;          // rows of x a tile
constexpr int GT_BN = 128;          // rows of w a tile
constexpr int GT_BK = 64;           // K elements a step
constexpr int GT_ROW = GT_BK + 8;   // an LDS row (bf16 elements): 144 bytes
constexpr int GT_DIES = 8;
constexpr int GT_PIECES = GT_BN * (GT_BK / 8) / 256;  // 16-byte pieces of one operand's step a thread fetches: 4

struct TilePlan {
  int m_tiles, n_tiles, splits, k_block;
};

template <typename TO>
__global__ __launch_bounds__(256, 2) void gemm_tile_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, float* __restrict__ part, TO* __restrict__ y,
    int M, int N, int K, int ldx, int ldw, int ldy, TilePlan plan) {
  extern __shared__ __attribute__((aligned(16))) bf16_t lds_raw[];
  bf16_t(*lds)[GT_ROW] = reinterpret_cast<bf16_t(*)[GT_ROW]>(lds_raw);  // two buffers of [GT_BN + GT_BM][GT_ROW]
  const int lane = threadIdx.x % 64;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int c = lane % 32, hl = lane / 32;
  // tile of this workgroup: the row blocks of x that share a block of w sit on one die
  const int die = blockIdx.x % GT_DIES, j = blockIdx.x / GT_DIES;
  const int n_tile = (j / plan.m_tiles) * GT_DIES + die, m_tile = j % plan.m_tiles;
  if (n_tile >= plan.n_tiles) return;  // (the grid is padded to whole groups of eight)
  const int n0 = n_tile * GT_BN, m0 = m_tile * GT_BM;
  const int kb0 = blockIdx.y * plan.k_block;
  const int kb1 = min(K, kb0 + plan.k_block);
  const int wn = wave % 2, wm = wave / 2;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][jj][v] = 0.f;

  // what this thread fetches of a step: piece p is row (tid + 256 p) / 8, bytes 16 * ((tid + 256 p) % 8)
  const int prow = threadIdx.x / 8, pk = 8 * (threadIdx.x % 8);
  const bf16_t* wsrc[GT_PIECES];
  const bf16_t* xsrc[GT_PIECES];
  bool x_in[GT_PIECES];
#pragma unroll
  for (int p = 0; p < GT_PIECES; ++p) {
    wsrc[p] = w + static_cast<size_t>(min(n0 + prow + 32 * p, N - 1)) * ldw;
    x_in[p] = m0 + prow + 32 * p < M;
    xsrc[p] = x + static_cast<size_t>(min(m0 + prow + 32 * p, M - 1)) * ldx;
  }
  const int k_last = K - 8;
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  u32x4_t wr[2][GT_PIECES], xr[2][GT_PIECES];
#define GT_LOAD(SET, K0)                                                                     \
  {                                                                                           \
    const int kk_ = min((K0) + pk, k_last);                                                   \
    _Pragma("unroll") for (int p = 0; p < GT_PIECES; ++p) {                                   \
      wr[SET][p] = *reinterpret_cast<const u32x4_t*>(wsrc[p] + kk_);                          \
      xr[SET][p] = *reinterpret_cast<const u32x4_t*>(xsrc[p] + kk_);                          \
    }                                                                                         \
  }
  // (x is zeroed where it lies beyond M or beyond the slice: at the store, not at the load, so
  // that no select sits behind a load that is still on its way)
#define GT_PARK(SET, BUF, K0)                                                                \
  {                                                                                           \
    bf16_t(*dst_)[GT_ROW] = lds + (BUF) * (GT_BN + GT_BM);                                    \
    if (m_edge || (K0) + GT_BK > kb1) { /* the same in every thread of the workgroup */      \
      const bool k_in_ = (K0) + pk < kb1;                                                     \
      _Pragma("unroll") for (int p = 0; p < GT_PIECES; ++p) {                                 \
        *reinterpret_cast<u32x4_t*>(&dst_[prow + 32 * p][pk]) = wr[SET][p];                   \
        *reinterpret_cast<u32x4_t*>(&dst_[GT_BN + prow + 32 * p][pk]) = (k_in_ && x_in[p]) ? xr[SET][p] : zero; \
      }                                                                                       \
    } else {                                                                                  \
      _Pragma("unroll") for (int p = 0; p < GT_PIECES; ++p) {                                 \
        *reinterpret_cast<u32x4_t*>(&dst_[prow + 32 * p][pk]) = wr[SET][p];                   \
        *reinterpret_cast<u32x4_t*>(&dst_[GT_BN + prow + 32 * p][pk]) = xr[SET][p];           \
      }                                                                                       \
    }                                                                                         \
  }
  // One step: put the step after next in flight (into the register set that the parked step has
  // left), multiply what the buffer holds, park the next step in the other buffer (last read a
  // step ago, before the barrier every wave has passed since).  The loads are unconditional: past
  // the slice they read valid places whose x is parked as zeros; a load under a condition would
  // make the compiler wait for everything in flight where the paths meet.  The fences keep the
  // compiler from moving the loads down to where their data is parked (it would, and wait for
  // them at once).
#define GT_STEP(BUF, S)                                                                      \
  {                                                                                           \
    GT_LOAD(BUF, kb0 + ((S) + 2) * GT_BK)                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                        \
    const bf16_t(*ws)[GT_ROW] = lds + (BUF) * (GT_BN + GT_BM) + 64 * wn;                      \
    const bf16_t(*xs)[GT_ROW] = lds + (BUF) * (GT_BN + GT_BM) + GT_BN + 64 * wm;              \
    Frag8 a[4][2], b[4][2];                                                                   \
    _Pragma("unroll") for (int u = 0; u < 4; ++u)                                             \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                           \
      a[u][i].u = *reinterpret_cast<const u32x4_t*>(&ws[32 * i + c][16 * u + 8 * hl]);        \
      b[u][i].u = *reinterpret_cast<const u32x4_t*>(&xs[32 * i + c][16 * u + 8 * hl]);        \
    }                                                                                         \
    _Pragma("unroll") for (int u = 0; u < 4; ++u)                                             \
    _Pragma("unroll") for (int i = 0; i < 2; ++i)                                             \
    _Pragma("unroll") for (int jj = 0; jj < 2; ++jj)                                          \
        acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u][i].v, b[u][jj].v, acc[i][jj], 0, 0, 0); \
    __builtin_amdgcn_sched_barrier(0);                                                        \
    GT_PARK(1 - (BUF), 1 - (BUF), kb0 + ((S) + 1) * GT_BK)                                    \
    __syncthreads();                                                                          \
  }
  // (an odd number of steps is rounded up: the step beyond the slice multiplies zeros of x)
  const int n_steps = (kb1 - kb0 + GT_BK - 1) / GT_BK;
  const bool m_edge = m0 + GT_BM > M;
  GT_LOAD(0, kb0)
  GT_LOAD(1, kb0 + GT_BK)
  __builtin_amdgcn_sched_barrier(0);
  GT_PARK(0, 0, kb0)
  __syncthreads();
  for (int s = 0; s < n_steps; s += 2) {
    GT_STEP(0, s)
    GT_STEP(1, s + 1)
  }
#undef GT_STEP
#undef GT_LOAD
#undef GT_PARK

  // accumulator v of acc[i][jj] is y[token m0 + 64 wm + 32 jj + c][feature n0 + 64 wn + 32 i + 8 (v / 4) + 4 hl + v % 4]
  float* pout = part ? part + static_cast<size_t>(blockIdx.y) * M * N : nullptr;
  // four features at once where every row of the result starts on a 16-byte boundary
  const bool vec = pout ? N % 4 == 0 : (ldy % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0);
#pragma unroll
  for (int jj = 0; jj < 2; ++jj) {
    const int m = m0 + 64 * wm + 32 * jj + c;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + 64 * wn + 32 * i + 8 * q + 4 * hl;
        if (n >= N) continue;
        const float v0 = acc[i][jj][4 * q], v1 = acc[i][jj][4 * q + 1], v2 = acc[i][jj][4 * q + 2], v3 = acc[i][jj][4 * q + 3];
        if (vec && n + 3 < N) {
          if (pout) {
            *reinterpret_cast<f32x4_t*>(pout + static_cast<size_t>(m) * N + n) = f32x4_t{v0, v1, v2, v3};
          } else if (sizeof(TO) == 2) {
            u32x2_t out;
            out[0] = pack_bf16x2(v0, v1);
            out[1] = pack_bf16x2(v2, v3);
            *reinterpret_cast<u32x2_t*>(reinterpret_cast<bf16_t*>(y) + static_cast<size_t>(m) * ldy + n) = out;
          } else {
            *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(y) + static_cast<size_t>(m) * ldy + n) = f32x4_t{v0, v1, v2, v3};
          }
        } else {
          const float vs[4] = {v0, v1, v2, v3};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) {
              if (pout)
                pout[static_cast<size_t>(m) * N + n + e] = vs[e];
              else
                y[static_cast<size_t>(m) * ldy + n + e] = from_f32<TO>(vs[e]);
            }
        }
      }
  }
}

int g_force_splits = 0;

// Tiles of 128 x 128; K is cut where the tiles alone leave compute units idle (the slices are
// added by whoever consumes the product), as far as a slice keeps at least 512 elements of K.
TilePlan tile_plan(int M, int N, int K) {
  TilePlan p;
  p.m_tiles = (M + GT_BM - 1) / GT_BM;
  p.n_tiles = (N + GT_BN - 1) / GT_BN;
  const int tiles = p.m_tiles * p.n_tiles;
  int splits = 1;
  // two workgroups fit a compute unit: cut K while the launch has fewer than one a unit
  while (splits < 8 && tiles * splits * 2 <= 256 && K / (splits * 2) >= 512) splits *= 2;
  if (g_force_splits > 0) splits = std::max(1, std::min(g_force_splits, K / GT_BK));
  const int steps = (K + GT_BK - 1) / GT_BK;
  p.k_block = (steps + splits - 1) / splits * GT_BK;
  p.splits = (K + p.k_block - 1) / p.k_block;
  return p;
}

template <typename TO>
int launch_tile(const bf16_t* x, const bf16_t* w, float* part, TO* y, int M, int N, int K, int ldx, int ldw, int ldy,
                const TilePlan& plan, hipStream_t stream) {
  const int groups = (plan.n_tiles + GT_DIES - 1) / GT_DIES;
  dim3 grid(groups * plan.m_tiles * GT_DIES, plan.splits);
  constexpr size_t lds_bytes = 2 * static_cast<size_t>(GT_BN + GT_BM) * GT_ROW * sizeof(bf16_t);  // 72 KiB: two workgroups a unit
  static bool raised = false;  // more than the default 64 KiB of dynamic LDS, once per kernel form
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tile_kernel<TO>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024) != hipSuccess)
      return yk_fail("gemm_tile: cannot raise the LDS limit");
    raised = true;
  }
  gemm_tile_kernel<TO><<<grid, dim3(256), lds_bytes, stream>>>(x, w, part, y, M, N, K, ldx, ldw, ldy, plan);
  return yk_check_launch("gemm_tile");
}

}  // namespace

// For tests and measurements: force the number of K slices (0: the library decides).
extern "C" int yk_gemm_tile_force(int splits) {
  YK_REQUIRE(splits >= 0, "gemm_tile_force: bad slice count");
  g_force_splits = splits;
  return 0;
}

// The K slices the plan makes for these sizes (a caller that keeps them needs slices * M * N floats).
extern "C" int yk_gemm_tile_splits(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K < 8) return 1;
  return tile_plan(M, N, K).splits;
}

// y [M, N] = x [M, K] . w [N, K]^T.  Where the plan cuts K (yk_gemm_tile_splits > 1) the slices
// stay unreduced in `workspace` ([slices][M][N] float32) for a consumer that adds them, and y is
// not written; returns the number of slices left there (0: y holds the result), negative on error.
extern "C" int yk_gemm_tile(const void* x, const void* w, void* y, int y_dtype, float* workspace, size_t workspace_floats,
                            int M, int N, int K, int ldx, int ldw, int ldy, hipStream_t stream) {
  YK_REQUIRE(M >= 0 && N > 0 && K >= 8, "gemm_tile: bad sizes");
  YK_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "gemm_tile: K and the leading dimensions must be multiples of 8");
  YK_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
             "gemm_tile: operands must be 16-byte aligned");
  YK_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "gemm_tile: leading dimensions too small");
  YK_REQUIRE(y_dtype == YK_F32 || y_dtype == YK_BF16, "gemm_tile: unsupported output dtype");
  if (M == 0) return 0;
  const TilePlan plan = tile_plan(M, N, K);
  YK_REQUIRE(static_cast<long>(plan.m_tiles) * ((plan.n_tiles + 7) / 8) * 8 <= 0x7fffffffL / 2, "gemm_tile: too many tiles");
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  if (plan.splits == 1) {
    YK_REQUIRE(y != nullptr, "gemm_tile: no result given");
    if (y_dtype == YK_F32) return launch_tile<float>(xp, wp, nullptr, static_cast<float*>(y), M, N, K, ldx, ldw, ldy, plan, stream);
    return launch_tile<bf16_t>(xp, wp, nullptr, static_cast<bf16_t*>(y), M, N, K, ldx, ldw, ldy, plan, stream);
  }
  YK_REQUIRE(workspace && reinterpret_cast<uintptr_t>(workspace) % 16 == 0 &&
                 workspace_floats >= static_cast<size_t>(plan.splits) * M * N,
             "gemm_tile: workspace too small or misaligned for the K slices");
  if (launch_tile<float>(xp, wp, workspace, nullptr, M, N, K, ldx, ldw, ldy, plan, stream)) return -1;
  return plan.splits;
}
