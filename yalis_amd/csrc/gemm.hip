// Contractions y[M, N] = x[M, K] . w[N, K]^T (the weight layout of a checkpoint).
//
// Two kernels:
//  * gemm_fma: float32 fused multiply-add accumulation for any mix of float32 /
//    bfloat16 operands and any sizes.  This is the whole true-32-bit path (no matrix
//    core mode with reduced-precision inputs is used) and the fallback for operands
//    the matrix-core kernel does not take.
//  * gemm_mfma_skinny: bfloat16 operands on the gfx950 matrix cores
//    (v_mfma_f32_16x16x32_bf16), float32 accumulation, for few rows of x (decode and
//    the output head): the weight is streamed once, straight from memory into the
//    matrix-core A operand, x sits in the B operand; K is split over workgroups so
//    that small weights still fill the chip, partial sums are combined in float32 in a
//    fixed order by a second kernel.
// The reference runs these products through nn.Linear / cuBLAS
// (yalis/external/model.py:63-65, 449, 462-466, 717-722).
#include <algorithm>

#include "common.h"

// ------------------------------------------------------------------ float32 FMA GEMM
constexpr int FT = 64;  // output tile FT x FT
constexpr int FK = 16;  // K step

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_fma_kernel(const TX* __restrict__ x,
                                                       const TW* __restrict__ w,
                                                       TO* __restrict__ y, int M, int N, int K,
                                                       int ldx, int ldw, int ldy) {
  __shared__ float xs[FK][FT + 1];
  __shared__ float ws[FK][FT + 1];
  const int m0 = blockIdx.y * FT, n0 = blockIdx.x * FT;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;  // 16 x 16 threads, 4 x 4 outputs each
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += FK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread
    for (int e = threadIdx.x; e < FT * FK; e += 256) {
      const int r = e / FK, kk = e % FK;
      const int k = k0 + kk;
      const int m = m0 + r, n = n0 + r;
      xs[kk][r] = (m < M && k < K) ? to_f32<TX>(x[static_cast<size_t>(m) * ldx + k]) : 0.f;
      ws[kk][r] = (n < N && k < K) ? to_f32<TW>(w[static_cast<size_t>(n) * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < FK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) y[static_cast<size_t>(m) * ldy + n] = from_f32<TO>(acc[i][j]);
    }
  }
}

template <typename TX, typename TW>
static int launch_fma(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K,
                      int ldx, int ldw, int ldy, hipStream_t stream) {
  dim3 grid((N + FT - 1) / FT, (M + FT - 1) / FT), block(256);
  if (y_dtype == YK_F32)
    gemm_fma_kernel<TX, TW, float><<<grid, block, 0, stream>>>(
        static_cast<const TX*>(x), static_cast<const TW*>(w), static_cast<float*>(y), M, N, K, ldx, ldw, ldy);
  else if (y_dtype == YK_BF16)
    gemm_fma_kernel<TX, TW, bf16_t><<<grid, block, 0, stream>>>(
        static_cast<const TX*>(x), static_cast<const TW*>(w), static_cast<bf16_t*>(y), M, N, K, ldx, ldw, ldy);
  else
    return yk_fail("gemm_fma: unsupported output dtype");
  return yk_check_launch("gemm_fma");
}

extern "C" int yk_gemm_fma(const void* x, int x_dtype, const void* w, int w_dtype, void* y,
                           int y_dtype, int M, int N, int K, int ldx, int ldw, int ldy,
                           hipStream_t stream) {
  YK_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_fma: bad sizes");
  YK_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "gemm_fma: leading dimensions too small");
  YK_REQUIRE((M + FT - 1) / FT <= 65535, "gemm_fma: too many rows for one launch");
  if (M == 0) return 0;
  if (x_dtype == YK_F32 && w_dtype == YK_F32) return launch_fma<float, float>(x, w, y, y_dtype, M, N, K, ldx, ldw, ldy, stream);
  if (x_dtype == YK_BF16 && w_dtype == YK_F32) return launch_fma<bf16_t, float>(x, w, y, y_dtype, M, N, K, ldx, ldw, ldy, stream);
  if (x_dtype == YK_F32 && w_dtype == YK_BF16) return launch_fma<float, bf16_t>(x, w, y, y_dtype, M, N, K, ldx, ldw, ldy, stream);
  if (x_dtype == YK_BF16 && w_dtype == YK_BF16) return launch_fma<bf16_t, bf16_t>(x, w, y, y_dtype, M, N, K, ldx, ldw, ldy, stream);
  return yk_fail("gemm_fma: unsupported operand dtypes");
}

// -------------------------------------------------------------- matrix-core skinny GEMM
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

union Frag8 {
  u32x4_t u;
  bf16x8_t v;
};

// Operand layout of v_mfma_f32_16x16x32_bf16 (64 lanes, r = lane % 16, g = lane / 16):
//   A (16 x 32): lane holds A[r][8g .. 8g+7];  B (32 x 16): lane holds B[8g .. 8g+7][r];
//   C (16 x 16): lane holds C[4g .. 4g+3][r].
// Here A = 16 rows of the weight (output features), B = 16 rows of x (tokens), so that
// C[i][r] = y[token r][feature 4g + i].
constexpr int SK_WAVES = 4;

template <int MT>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_mfma_skinny_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, float* __restrict__ part, int M,
    int N, int K, int ldx, int ldw, int k_chunk) {
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int r = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.x * SK_WAVES + wave) * 16;
  const int m0 = blockIdx.y * (16 * MT);
  const int ks = blockIdx.z * k_chunk;
  const int ke = min(K, ks + k_chunk);
  if (n0 >= N) return;
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const bool row_ok = (n0 + r) < N;
  const bf16_t* wrow = w + static_cast<size_t>(row_ok ? n0 + r : 0) * ldw;
  const bf16_t* xrow[MT];
  bool x_ok[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = m0 + 16 * t + r;
    x_ok[t] = m < M;
    xrow[t] = x + static_cast<size_t>(x_ok[t] ? m : 0) * ldx;
  }
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  for (int kb = ks; kb < ke; kb += 32) {
    // each lane group takes 8 of the step's 32; a chunk beyond ke feeds zeros
    const int k = kb + 8 * g;
    const bool k_ok = k < ke;
    Frag8 a;
    a.u = (row_ok && k_ok) ? *reinterpret_cast<const u32x4_t*>(wrow + k) : zero;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      Frag8 b;
      b.u = (x_ok[t] && k_ok) ? *reinterpret_cast<const u32x4_t*>(xrow[t] + k) : zero;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[t], 0, 0, 0);
    }
  }
  // part[split][m][n]
  float* out = part + static_cast<size_t>(blockIdx.z) * M * N;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = m0 + 16 * t + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g + i;
      if (n < N) out[static_cast<size_t>(m) * N + n] = acc[t][i];
    }
  }
}

// y[m][n] = sum over splits of part[s][m][n], in the order of s
template <typename TO>
__global__ void reduce_splits_kernel(const float* __restrict__ part, TO* __restrict__ y, int M,
                                     int N, int ldy, int splits) {
  const size_t total = static_cast<size_t>(M) * N;
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float s = 0.f;
    for (int k = 0; k < splits; ++k) s += part[k * total + i];
    y[(i / N) * ldy + i % N] = from_f32<TO>(s);
  }
}

// How the skinny kernel would split K for these sizes (also tells the caller how much
// workspace it needs: splits * M * N floats).
extern "C" int yk_gemm_skinny_splits(int M, int N, int K) {
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const long tiles = static_cast<long>((N + 16 * SK_WAVES - 1) / (16 * SK_WAVES)) * ((M + 16 * mt - 1) / (16 * mt));
  // aim at about 8 workgroups (32 waves) per compute unit, at least 256 of K per split
  long want = (256L * 8 + tiles - 1) / tiles;
  long max_by_k = std::max(1, K / 256);
  long s = std::max(1L, std::min(want, max_by_k));
  return static_cast<int>(std::min(s, 64L));
}

extern "C" int yk_gemm_mfma_skinny(const void* x, const void* w, void* y, int y_dtype,
                                   float* workspace, size_t workspace_floats, int M, int N, int K,
                                   int ldx, int ldw, int ldy, hipStream_t stream) {
  YK_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_mfma_skinny: bad sizes");
  YK_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_mfma_skinny: K and the leading dimensions must be multiples of 8");
  YK_REQUIRE((reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0),
             "gemm_mfma_skinny: operands must be 16-byte aligned");
  YK_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "gemm_mfma_skinny: leading dimensions too small");
  if (M == 0) return 0;
  const int splits = yk_gemm_skinny_splits(M, N, K);
  int k_chunk = (K + splits - 1) / splits;
  k_chunk = (k_chunk + 31) / 32 * 32;
  const int real_splits = (K + k_chunk - 1) / k_chunk;
  const bool direct = real_splits == 1 && y_dtype == YK_F32 && ldy == N;
  YK_REQUIRE(direct || workspace_floats >= static_cast<size_t>(real_splits) * M * N,
             "gemm_mfma_skinny: workspace too small");
  float* part = direct ? static_cast<float*>(y) : workspace;
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  dim3 grid((N + 16 * SK_WAVES - 1) / (16 * SK_WAVES), (M + 16 * mt - 1) / (16 * mt), real_splits);
  YK_REQUIRE(grid.y <= 65535, "gemm_mfma_skinny: too many rows for one launch");
  dim3 block(SK_WAVES * 64);
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  if (mt == 1)
    gemm_mfma_skinny_kernel<1><<<grid, block, 0, stream>>>(xp, wp, part, M, N, K, ldx, ldw, k_chunk);
  else if (mt == 2)
    gemm_mfma_skinny_kernel<2><<<grid, block, 0, stream>>>(xp, wp, part, M, N, K, ldx, ldw, k_chunk);
  else
    gemm_mfma_skinny_kernel<4><<<grid, block, 0, stream>>>(xp, wp, part, M, N, K, ldx, ldw, k_chunk);
  if (yk_check_launch("gemm_mfma_skinny")) return -1;
  if (direct) return 0;
  const size_t total = static_cast<size_t>(M) * N;
  const int rb = 256;
  const int rg = static_cast<int>(std::min<size_t>((total + rb - 1) / rb, 65535));
  if (y_dtype == YK_F32)
    reduce_splits_kernel<float><<<rg, rb, 0, stream>>>(part, static_cast<float*>(y), M, N, ldy, real_splits);
  else if (y_dtype == YK_BF16)
    reduce_splits_kernel<bf16_t><<<rg, rb, 0, stream>>>(part, static_cast<bf16_t*>(y), M, N, ldy, real_splits);
  else
    return yk_fail("gemm_mfma_skinny: unsupported output dtype");
  return yk_check_launch("reduce_splits");
}
