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
    // the K step's 16 products are summed on their own and then added to the running sum: a sum
    // of K terms carries the rounding of about sqrt(K / 16) + 4 additions instead of sqrt(K)
    float part[4][4] = {};
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
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] += part[i][j];
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
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

union Frag8 {
  u32x4_t u;
  bf16x8_t v;
};

// Operand layout of v_mfma_f32_16x16x32_bf16 (64 lanes, r = lane % 16, g = lane / 16):
//   A (16 x 32): lane holds A[r][8g .. 8g+7];  B (32 x 16): lane holds B[8g .. 8g+7][r];
//   C (16 x 16): lane holds C[4g .. 4g+3][r].
// Here A = 16 rows of the weight (output features), B = 16 rows of x (tokens), so that
// C[i][r] = y[token r][feature 4g + i].
//
// A workgroup of W waves (W = blockDim.x / 64, chosen per shape by the host) owns 16*W
// weight rows (16 per wave) and 16*MT rows of x over one slice of K (blockIdx.z).  K is
// walked in chunks of KC = 256 or 128 (skinny_chunk).  The chunk of x is staged in LDS once for all
// waves.  Every wave streams its own 16 weight rows with loads that cover two rows x 512 contiguous
// bytes (four x 256 with the short chunks)
// each (measured on MI355X: that pattern reads about a fifth faster than the 16 rows x 64
// bytes the matrix-core operand layout would ask of memory directly), parks the chunk in a
// wave-private piece of LDS and reads it back in operand layout; the next chunk's loads
// are in flight while the current one is multiplied.  Nothing is conditional in the loop:
// rows beyond N are read from the last row and never stored, K beyond the slice is read
// from valid places and meets zeros of x.
constexpr int SK_KC = 256;            // K elements per chunk
constexpr int SK_PAD = 8;             // bf16 elements of padding per LDS row (keeps 16-byte reads conflict-free)
constexpr int SK_ROW = SK_KC + SK_PAD;

// x is parked in two buffers by turns where that costs no resident workgroup (up to 16 rows
// of x): then one barrier a chunk is enough.  Measured: 2 to 5 % on the 8B shapes.
static constexpr int skinny_x_buffers(int mt, int kc) { return mt == 1 || kc < SK_KC ? 2 : 1; }
static size_t skinny_lds_bytes(int mt, int waves, int kc) {
  return static_cast<size_t>(16 * mt * skinny_x_buffers(mt, kc) + 16 * waves) * (kc + SK_PAD) * sizeof(bf16_t);
}
// Chunks are 256 or 128 elements of K long (with 128 a load covers four weight rows x 256
// bytes).  Short chunks leave room for the two buffers of x and for three workgroups a compute
// unit at any number of rows, and a workgroup gets going sooner, which counts where a
// workgroup walks a short slice of K; long chunks keep more bytes in flight per wave, which
// counts where it walks a long one (gate/up, the output head, the slices of the 70B shape).
// Measured on the 8B shapes (us, chunks of 256 / 128): 64 rows: qkv 17.0 / 15.3, o-proj 12.4 /
// 11.1, down 29.0 / 27.3, gate/up 59 / 56.7; 32 rows: qkv 12.8 / 11.5, o-proj 9.7 / 9.2, down
// 24.0 / 22.3, but gate/up 46.2 / 48.2; 8 rows: qkv 11.0 / 10.1, o-proj 8.1 / 8.0, down 21.0 / 20.4,
// but gate/up 40.2 / 46.6; the 70B shape's decode step at 64 rows (slices of 2,048 to 8,192):
// 36.9 / 37.7 ms, and its o-proj at 8 rows (slices of 2,048) is faster with long chunks too.  So:
// short chunks for slices of up to 1,792, up to 4,096 with 64 rows of x.
// What yk_gemm_skinny_force set (0: the library decides): for tests and measurements only.
static int g_force_chunk = 0, g_force_waves = 0, g_force_slices = 0;
// 33 to 64 rows of x against a K of 8,192 and more that one workgroup walks whole (no K slices:
// in practice gate/up with the activation in its epilogue): the wide form (32 x 32 x 16
// products, two waves of 32 weight rows a workgroup).  Measured (us, 16-row form / wide form):
// the 70B shape's gate/up (57,344 x 8,192) at 64 / 48 / 33 rows of x 200 / 186, 191 / 167,
// 187 / 161.  Elsewhere it does not pay: the same shape's sliced products at 64 rows, down-proj
// 97.4 / 98.4, qkv 33.8 / 43.5, o-proj 33.6 / 36.5; at a K of 4,096 (the 8B shape at 64 rows)
// gate/up 50.2 / 52.2 with four waves of 32 rows and 57.4 with two, down-proj 23.7 / 26.1, qkv
// 14.2 / 15.9.  The wide form halves the reads of x from LDS per weight byte, but a workgroup
// has half the waves to keep loads in flight, which counts for more wherever a workgroup's walk
// over K is short.  yk_gemm_skinny_wide: 0 never, 1 by this rule, 2 always (tests, measurements).
static int g_wide = 1;
constexpr int SK_WIDE_MIN_K = 8192;

static int skinny_chunk(int mt, int k_block) {
  if (g_force_chunk) return g_force_chunk;
  return k_block <= (mt == 4 ? 16 : 7) * SK_KC ? 128 : SK_KC;
}

// Where the rows of x come from when they are the output of an attention whose keys were
// split across workgroups and not yet merged (FROM_SPLITS): row m, column head * head_dim + d
// is the merged value of column token_col[m] % 16 * heads_per_tile + (head's place in its
// chunk) of tile token_col[m] / 16 (attn_merge_splits), rounded to bfloat16 as the merging
// kernel would have stored it.
struct AttnSplits {
  const float* o;
  const float* ml;
  const int32_t* token_col;
  int n_splits, n_heads, n_kv, head_dim, hpt, chunks;
};
constexpr int SK_SPLITS_MAX_K_BLOCK = 1024;  // a workgroup's whole slice of x then fits beside the weights

template <int MT, int W, typename TO, int GATED, bool FROM_SPLITS, int KC, int DEPTH = 1>
__global__ __launch_bounds__(W * 64) void gemm_mfma_skinny_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, float* __restrict__ part,
    TO* __restrict__ y, int M, int N, int K, int ldx, int ldw, int ldy, int k_block, AttnSplits xa) {
  static_assert(!FROM_SPLITS || (MT == 1 && GATED == 0), "unmerged attention feeds plain products of up to 16 rows");
  extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
  constexpr int STEPS = KC / 32;               // matrix-core steps per chunk
  constexpr int ROW = KC + SK_PAD;             // an LDS row
  constexpr int LPR = KC / 8, RPL = 64 / LPR;  // lanes that load one weight row's chunk; rows per load
  constexpr int XB = skinny_x_buffers(MT, KC);
  bf16_t(*xs0)[ROW] = reinterpret_cast<bf16_t(*)[ROW]>(lds);  // XB x [16 * MT][ROW]
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  // FROM_SPLITS: the workgroup's whole slice of x, [16][k_block + SK_PAD], merged once before the loop
  const int x_all_row = k_block + SK_PAD;
  bf16_t* x_all = lds;
  bf16_t(*wl)[ROW] = reinterpret_cast<bf16_t(*)[ROW]>(
      lds + (FROM_SPLITS ? static_cast<size_t>(16) * x_all_row : static_cast<size_t>(16 * MT * XB) * ROW) +
      static_cast<size_t>(16 * wave) * ROW);  // this wave's [16][ROW]
  const int r = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.x * W + wave) * 16;
  const int m0 = blockIdx.y * (16 * MT);
  const int kb0 = blockIdx.z * k_block;
  const int kb1 = min(K, kb0 + k_block);

  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // weights: load j of a chunk covers rows RPL * j .. RPL * j + RPL - 1 (two rows x 512 bytes with chunks
  // of 256, four x 256 bytes with chunks of 128), 16 bytes a lane
  const int half = lane / LPR, l32 = lane % LPR;
  const bf16_t* wrow[STEPS];
#pragma unroll
  for (int j = 0; j < STEPS; ++j) wrow[j] = w + static_cast<size_t>(min(n0 + RPL * j + half, N - 1)) * ldw;
  const int k_last = K - 8;
  // DEPTH chunks are in flight per wave, each in a register set of its own
  u32x4_t regs[DEPTH][STEPS];
#define SK_LOAD_W(S, KC0)                                                                   \
  {                                                                                          \
    const int kk_ = min((KC0) + 8 * l32, k_last);                                            \
    _Pragma("unroll") for (int j = 0; j < STEPS; ++j)                                     \
        regs[S][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wrow[j] + kk_)); \
  }
  // x: the chunk's 16*MT rows x 32 pieces of 16 bytes are spread over the threads, XP each;
  // what lies outside M or the slice is loaded from a clamped address and parked as zero
  constexpr int XP = 16 * MT * (KC / 8) / (W * 64);
  static_assert(XP * W * 64 == 16 * MT * (KC / 8), "x pieces must divide evenly over the threads");
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  u32x4_t xr[DEPTH][XP];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
#pragma unroll
    for (int p = 0; p < XP; ++p) xr[d][p] = zero;
#define SK_LOAD_X(S, KC0)                                                                   \
  _Pragma("unroll") for (int p = 0; p < XP; ++p) {                                           \
    const int e_ = threadIdx.x + p * W * 64;                                                 \
    const int m_ = m0 + e_ / (KC / 8), k_ = (KC0) + 8 * (e_ % (KC / 8));               \
    if (m_ < M) xr[S][p] = *reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(m_) * ldx + min(k_, k_last)); \
  }

  // The workgroups of a launch do not all start at the same place of their slices: workgroup b
  // starts b units of 256 into its slice and wraps round.  Row blocks started together would
  // otherwise ask for addresses a whole number of rows apart at every moment, which crowd onto
  // few memory channels: where the rows are a multiple of 4 KiB apart, that is (measured at the 8B
  // shape, 8 rows: gate/up 40.2 -> 37.6 us; the decode step 3.60 -> 3.53 ms, that of the 70B shape
  // 25.9 -> 25.1; with rows 6 KiB apart, the 3B shape, it cost half a percent; with 64 rows of x,
  // where every workgroup stages as many bytes of x as of the weight and those reads are shared only
  // by workgroups at the same place, gate/up went 56.9 -> 59.4 us, so not there).  (The unit does not
  // depend on the chunk length, so the order of the sums does not either.)
  const int n_chunks = (kb1 - kb0 + KC - 1) / KC;
  constexpr int PER_UNIT = SK_KC / KC;              // chunks in a unit of 256
  const int n_units = (kb1 - kb0 + SK_KC - 1) / SK_KC;
  const int slots = PER_UNIT * n_units;             // the last one may lie beyond the slice
  const int first_slot = MT < 4 && ldw % 2048 == 0 ? static_cast<int>(blockIdx.x % n_units) * PER_UNIT : 0;
  const bool last_missing = slots > n_chunks;
  const int missing_at = slots - 1 - first_slot;    // where the last slot comes in this workgroup's order
  auto chunk_start = [&](int i) {
    int j = i + (last_missing && i >= missing_at ? 1 : 0) + first_slot;
    if (j >= slots) j -= slots;
    return kb0 + j * KC;
  };
  SK_LOAD_W(0, chunk_start(0))
  if (FROM_SPLITS) {
    // (the first chunk of the weights is in flight meanwhile)
    const int pieces = k_block / 4;
    const int qpk = xa.n_heads / xa.n_kv;
    // rows beyond M stand as zeros
    for (int e = M * pieces + threadIdx.x; e < 16 * pieces; e += W * 64)
      *reinterpret_cast<u32x2_t*>(x_all + static_cast<size_t>(e / pieces) * x_all_row + (e % pieces) * 4) = u32x2_t{0u, 0u};
    // (unrolled: the loads of four pieces are in flight together)
#pragma unroll 4
    for (int e = threadIdx.x; e < M * pieces; e += W * 64) {
      const int m = e / pieces, kk = (e % pieces) * 4, k = kb0 + kk;
      u32x2_t piece = {0u, 0u};
      if (k < K) {
        const int tc = xa.token_col[m];
        const int head = k / xa.head_dim, d = k % xa.head_dim;
        const int hq = head % qpk;
        const size_t group = static_cast<size_t>(tc / 16) * (xa.n_kv * xa.chunks) + (head / qpk) * xa.chunks + hq / xa.hpt;
        float merged[4];
        attn_merge_splits(xa.o, xa.ml, group * xa.n_splits * 16 + (tc % 16) * xa.hpt + hq % xa.hpt, xa.n_splits, xa.head_dim, d, merged);
        piece[0] = pack_bf16x2(merged[0], merged[1]);
        piece[1] = pack_bf16x2(merged[2], merged[3]);
      }
      *reinterpret_cast<u32x2_t*>(x_all + static_cast<size_t>(m) * x_all_row + kk) = piece;
    }
  } else {
    SK_LOAD_X(0, chunk_start(0))
  }
#pragma unroll
  for (int d = 1; d < DEPTH; ++d)
    if (d < n_chunks) {
      SK_LOAD_W(d, chunk_start(d))
      if (!FROM_SPLITS) {
        SK_LOAD_X(d, chunk_start(d))
      }
    }
  int turn = 0;
  for (int ci0 = 0; ci0 < n_chunks; ci0 += DEPTH) {
#pragma unroll
   for (int d = 0; d < DEPTH; ++d) {
    const int ci = ci0 + d;
    if (DEPTH > 1 && ci >= n_chunks) continue;  // (the same in every wave)
    const int kc = chunk_start(ci);
    // With one buffer every wave must have read the previous chunk of x before it is
    // overwritten.  With two, the buffer written now was last read two chunks ago, and every
    // wave finished that before it passed the previous chunk's barrier.
    if (XB == 1) __syncthreads();
    bf16_t(*xs)[ROW] = xs0 + (XB == 2 ? turn * 16 * MT : 0);
    // park what has arrived, then put the next chunk's loads in flight
#pragma unroll
    for (int j = 0; j < STEPS; ++j) *reinterpret_cast<u32x4_t*>(&wl[RPL * j + half][8 * l32]) = regs[d][j];
    if (!FROM_SPLITS) {
#pragma unroll
      for (int p = 0; p < XP; ++p) {
        // (zeroed here, not at the load: a select right behind the load would make the wave
        // wait for everything it has just put in flight)
        const int e = threadIdx.x + p * W * 64;
        const bool outside = m0 + e / (KC / 8) >= M || kc + 8 * (e % (KC / 8)) >= kb1;
        *reinterpret_cast<u32x4_t*>(&xs[e / (KC / 8)][8 * (e % (KC / 8))]) = outside ? zero : xr[d][p];
      }
    }
    if (ci + DEPTH < n_chunks) {
      const int kc_next = chunk_start(ci + DEPTH);
      SK_LOAD_W(d, kc_next)
      if (!FROM_SPLITS) {
        SK_LOAD_X(d, kc_next)
      }
    }
    __syncthreads();
    // The operands of the steps are read from LDS ahead of the products that take them (all
    // of the chunk's at once where the registers allow, else two steps ahead): written the
    // plain way, one read then its product, the compiler reuses one register set and every
    // product waits for an LDS round trip.
    constexpr int AHEAD = MT >= 4 ? 2 : (MT == 2 ? 3 : STEPS);
    Frag8 a[STEPS], b[STEPS][MT];
#define SK_READ(U)                                                                          \
  {                                                                                          \
    a[U].u = *reinterpret_cast<const u32x4_t*>(&wl[r][32 * (U) + 8 * g]);                    \
    _Pragma("unroll") for (int t = 0; t < MT; ++t)                                           \
        b[U][t].u = FROM_SPLITS                                                              \
            ? *reinterpret_cast<const u32x4_t*>(x_all + static_cast<size_t>(16 * t + r) * x_all_row + (kc - kb0) + 32 * (U) + 8 * g) \
            : *reinterpret_cast<const u32x4_t*>(&xs[16 * t + r][32 * (U) + 8 * g]);          \
  }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) SK_READ(u)
    __builtin_amdgcn_sched_barrier(0);  // (the scheduler would otherwise move the reads back to their products)
#pragma unroll
    for (int u = 0; u < STEPS; ++u) {
      if (u + AHEAD < STEPS) {
        SK_READ(u + AHEAD)
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u].v, b[u][t].v, acc[t], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
#undef SK_READ
    turn ^= 1;
   }
  }
#undef SK_LOAD_W
#undef SK_LOAD_X

  if (GATED) {
    // The weight's rows alternate: 8 gate rows, then the 8 up rows that belong to them.  A
    // wave's tile holds one such pair of groups: lane groups 0 and 1 have the gate features
    // 0..7 of a token, groups 2 and 3 the up features, 32 lanes further.  Both are rounded
    // as the product's output would have been, then out = act(gate) * up, 8 columns a tile.
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      f32x4_t up;
#pragma unroll
      for (int e = 0; e < 4; ++e) up[e] = __shfl_xor(acc[t][e], 32, 64);
      const int m = m0 + 16 * t + r;
      if (g < 2 && m < M && n0 < N) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          y[static_cast<size_t>(m) * ldy + n0 / 2 + 4 * g + e] =
              from_f32<TO>(act_apply(as_output(acc[t][e], 1), GATED - 1) * as_output(up[e], 1));
      }
    }
    return;
  }
  const bool to_part = part != nullptr;
  float* pout = to_part ? part + static_cast<size_t>(blockIdx.z) * M * N : nullptr;
  const int n = n0 + 4 * g;
  if (n >= N) return;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = m0 + 16 * t + r;
    if (m >= M) continue;
    if (to_part && n + 3 < N && N % 4 == 0) {
      *reinterpret_cast<f32x4_t*>(pout + static_cast<size_t>(m) * N + n) = acc[t];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (n + e < N) {
          if (to_part)
            pout[static_cast<size_t>(m) * N + n + e] = acc[t][e];
          else
            y[static_cast<size_t>(m) * ldy + n + e] = from_f32<TO>(acc[t][e]);
        }
      }
    }
  }
}

// The wide form, for 33 to 64 rows of x: v_mfma_f32_32x32x16_bf16 (64 lanes, c = lane % 32,
// hl = lane / 32):
//   A (32 x 16): lane holds A[c][8 hl .. 8 hl + 7];  B (16 x 32): lane holds B[8 hl .. 8 hl + 7][c];
//   C (32 x 32): lane holds C[8 (v / 4) + 4 hl + v % 4][c] in accumulator v = 0 .. 15.
// A = 32 rows of the weight, B = 32 rows of x, two B tiles a wave: every weight fragment read
// from LDS meets two fragments of x, where the 16-row form reads four (and half as large a
// piece of the weight) - at 64 rows of x those reads are what the workgroup's time goes to.
// A workgroup of W waves owns 32 W weight rows and 64 rows of x over one slice of K; all else
// (chunks, loads of two rows x 512 bytes or four x 256, parking in wave-private LDS, x staged
// once a workgroup, clamped addresses instead of conditions) is the 16-row form's.
typedef float f32x16_t __attribute__((ext_vector_type(16)));

template <int W, typename TO, int GATED, int KC, int DEPTH = 1>
__global__ __launch_bounds__(W * 64) void gemm_mfma_skinny_wide_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, float* __restrict__ part,
    TO* __restrict__ y, int M, int N, int K, int ldx, int ldw, int ldy, int k_block) {
  extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
  constexpr int STEPS = KC / 16;               // matrix-core steps per chunk
  constexpr int ROW = KC + SK_PAD;             // an LDS row
  constexpr int LOADS = KC / 16;               // 16-byte loads a lane makes for a chunk of the wave's 32 rows
  constexpr int LPR = KC / 8, RPL = 64 / LPR;  // lanes that load one weight row's chunk; rows per load
  constexpr int XB = skinny_x_buffers(4, KC);
  bf16_t(*xs0)[ROW] = reinterpret_cast<bf16_t(*)[ROW]>(lds);  // XB x [64][ROW]
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  bf16_t(*wl)[ROW] = reinterpret_cast<bf16_t(*)[ROW]>(lds + static_cast<size_t>(64 * XB) * ROW + static_cast<size_t>(32 * wave) * ROW);
  const int c = lane % 32, hl = lane / 32;
  const int n0 = (blockIdx.x * W + wave) * 32;
  const int m0 = blockIdx.y * 64;
  const int kb0 = blockIdx.z * k_block;
  const int kb1 = min(K, kb0 + k_block);

  f32x16_t acc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

  const int half = lane / LPR, l32 = lane % LPR;
  const bf16_t* wrow[LOADS];
#pragma unroll
  for (int j = 0; j < LOADS; ++j) wrow[j] = w + static_cast<size_t>(min(n0 + RPL * j + half, N - 1)) * ldw;
  const int k_last = K - 8;
  u32x4_t regs[DEPTH][LOADS];  // DEPTH chunks in flight per wave, a register set each
#define SKW_LOAD_W(S, KC0)                                                                  \
  {                                                                                          \
    const int kk_ = min((KC0) + 8 * l32, k_last);                                            \
    _Pragma("unroll") for (int j = 0; j < LOADS; ++j)                                        \
        regs[S][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wrow[j] + kk_)); \
  }
  constexpr int XP = 64 * (KC / 8) / (W * 64);
  static_assert(XP * W * 64 == 64 * (KC / 8), "x pieces must divide evenly over the threads");
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  u32x4_t xr[DEPTH][XP];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
#pragma unroll
    for (int p = 0; p < XP; ++p) xr[d][p] = zero;
#define SKW_LOAD_X(S, KC0)                                                                  \
  _Pragma("unroll") for (int p = 0; p < XP; ++p) {                                           \
    const int e_ = threadIdx.x + p * W * 64;                                                 \
    const int m_ = m0 + e_ / (KC / 8), k_ = (KC0) + 8 * (e_ % (KC / 8));                     \
    if (m_ < M) xr[S][p] = *reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(m_) * ldx + min(k_, k_last)); \
  }
  const int n_chunks = (kb1 - kb0 + KC - 1) / KC;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (d < n_chunks) {
      SKW_LOAD_W(d, kb0 + d * KC)
      SKW_LOAD_X(d, kb0 + d * KC)
    }
  int turn = 0;
  for (int ci0 = 0; ci0 < n_chunks; ci0 += DEPTH) {
#pragma unroll
   for (int d = 0; d < DEPTH; ++d) {
    const int ci = ci0 + d;
    if (DEPTH > 1 && ci >= n_chunks) continue;  // (the same in every wave)
    const int kc = kb0 + ci * KC;
    if (XB == 1) __syncthreads();
    bf16_t(*xs)[ROW] = xs0 + (XB == 2 ? turn * 64 : 0);
#pragma unroll
    for (int j = 0; j < LOADS; ++j) *reinterpret_cast<u32x4_t*>(&wl[RPL * j + half][8 * l32]) = regs[d][j];
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int e = threadIdx.x + p * W * 64;
      const bool outside = m0 + e / (KC / 8) >= M || kc + 8 * (e % (KC / 8)) >= kb1;
      *reinterpret_cast<u32x4_t*>(&xs[e / (KC / 8)][8 * (e % (KC / 8))]) = outside ? zero : xr[d][p];
    }
    if (ci + DEPTH < n_chunks) {
      SKW_LOAD_W(d, kc + DEPTH * KC)
      SKW_LOAD_X(d, kc + DEPTH * KC)
    }
    __syncthreads();
    constexpr int AHEAD = 3;
    Frag8 a[STEPS], b[STEPS][2];
#define SKW_READ(U)                                                                         \
  {                                                                                          \
    a[U].u = *reinterpret_cast<const u32x4_t*>(&wl[c][16 * (U) + 8 * hl]);                   \
    b[U][0].u = *reinterpret_cast<const u32x4_t*>(&xs[c][16 * (U) + 8 * hl]);                \
    b[U][1].u = *reinterpret_cast<const u32x4_t*>(&xs[32 + c][16 * (U) + 8 * hl]);           \
  }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) SKW_READ(u)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < STEPS; ++u) {
      if (u + AHEAD < STEPS) {
        SKW_READ(u + AHEAD)
        __builtin_amdgcn_sched_barrier(0);
      }
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u].v, b[u][0].v, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u].v, b[u][1].v, acc[1], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
#undef SKW_READ
    turn ^= 1;
   }
  }
#undef SKW_LOAD_W
#undef SKW_LOAD_X

  if (GATED) {
    // The weight's rows alternate 8 gate rows / their 8 up rows: of a wave's 32 rows, 0-7 and
    // 16-23 are gates, 8-15 and 24-31 their ups.  Accumulators 0-3 of a lane are four gate
    // features (4 hl .. 4 hl + 3) of one token, accumulators 4-7 the up features that belong
    // to them; 8-11 and 12-15 the second pair of groups.
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int m = m0 + 32 * t + c;
      if (m >= M) continue;
#pragma unroll
      for (int pair = 0; pair < 2; ++pair) {
        if (n0 + 16 * pair >= N) continue;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          y[static_cast<size_t>(m) * ldy + n0 / 2 + 8 * pair + 4 * hl + e] =
              from_f32<TO>(act_apply(as_output(acc[t][8 * pair + e], 1), GATED - 1) * as_output(acc[t][8 * pair + 4 + e], 1));
      }
    }
    return;
  }
  const bool to_part = part != nullptr;
  float* pout = to_part ? part + static_cast<size_t>(blockIdx.z) * M * N : nullptr;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int m = m0 + 32 * t + c;
    if (m >= M) continue;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + 8 * q + 4 * hl;
      if (n >= N) continue;
      if (to_part && n + 3 < N && N % 4 == 0) {
        *reinterpret_cast<f32x4_t*>(pout + static_cast<size_t>(m) * N + n) =
            f32x4_t{acc[t][4 * q], acc[t][4 * q + 1], acc[t][4 * q + 2], acc[t][4 * q + 3]};
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (n + e < N) {
            if (to_part)
              pout[static_cast<size_t>(m) * N + n + e] = acc[t][4 * q + e];
            else
              y[static_cast<size_t>(m) * ldy + n + e] = from_f32<TO>(acc[t][4 * q + e]);
          }
        }
      }
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

static int skinny_mt(int M) { return M <= 16 ? 1 : (M <= 32 ? 2 : 4); }

// How the skinny kernel cuts the work for these sizes: waves per workgroup (each wave owns
// 16 weight rows), the number of K slices and the length of one (a multiple of 256).
// All workgroups do the same amount of work, so the time is that of the busiest compute
// unit: (workgroups on it) x (waves each) x (K chunks each, plus a start-up of about one
// and a half chunks), stretched when the unit has too few waves to keep memory busy.  The
// plan minimises that over 4 or 8 waves and the slice counts that leave at least two chunks
// per workgroup, with a small charge for narrow workgroups (every workgroup stages its own
// copy of x) and for many slices (the consumer adds them).
// A caller that takes the slices unreduced needs splits * M * N floats.
constexpr int SK_CUS = 256;

static int skinny_plan(int M, int N, int K, bool gated, int* waves_out, int* k_block_out) {
  const int mt = skinny_mt(M);
  const long mtiles = (M + 16 * mt - 1) / (16 * mt);
  const long ntiles = (N + 15) / 16;
  const long chunks = (K + SK_KC - 1) / SK_KC;
  // A product with the activation in its epilogue cannot split K; where its row blocks alone
  // occupy every compute unit it is not split (the fused epilogue saves a kernel and a pass over
  // the slices: the decode step of the 3B shape went 2.17 -> 2.10 ms at 8 rows, that of the 70B
  // shape 26.1 -> 25.8).
  const long max_s = gated && (ntiles + 3) / 4 * mtiles >= SK_CUS ? 1 : std::max(1L, std::min(32L, chunks / 2));
  double best = 1e300;
  int best_w = 4;
  long best_s = 1;
  // Four waves a workgroup beat eight at up to 32 rows of x on every shape tried.  With 64 rows
  // a workgroup stages as many bytes of x as of the weight, and eight waves share one copy:
  // measured on the 8B shapes at 64 rows (us, four / eight waves): gate/up 57.5 / 49.4, down
  // 27.0 / 23.7, o-proj 11.3 / 10.5, but qkv 15.4 / 16.3 (its 384 workgroups of eight waves
  // fill the compute units one and a half times); the model below tells these apart.
  for (int w : {4, 8}) {
    if (w == 8 && mt != 4) continue;
    const long rblocks = (ntiles + w - 1) / w;
    const double resident = std::min(20.0, static_cast<double>(160 * 1024 / skinny_lds_bytes(mt, w, SK_KC)) * w);
    for (long s = 1; s <= max_s; ++s) {
      const long per = (chunks + s - 1) / s;          // chunks per workgroup
      const long real = (chunks + per - 1) / per;     // slices that are not empty
      const long blocks = rblocks * mtiles * real;
      const double busiest = static_cast<double>((blocks + SK_CUS - 1) / SK_CUS) * w * (per + 1.5);
      // a compute unit streams at full rate only with about 6 waves' loads in flight
      const double waves_cu = std::min(resident, static_cast<double>(blocks) * w / SK_CUS);
      const double starved = std::max(1.0, 6.0 / waves_cu);
      const double cost = busiest * starved * (1.0 + 0.25 * mt / w) * (1.0 + 0.01 * real);
      if (cost < best * 0.999) {
        best = cost;
        best_w = w;
        best_s = real;
      }
    }
  }
  if (g_force_waves) best_w = g_force_waves == 8 && mt != 4 ? 4 : g_force_waves;
  if (g_force_slices) best_s = std::min<long>(g_force_slices, chunks);
  int k_block = static_cast<int>((chunks + best_s - 1) / best_s) * SK_KC;
  if (waves_out) *waves_out = best_w;
  if (k_block_out) *k_block_out = k_block;
  return static_cast<int>((K + k_block - 1) / k_block);
}

// For tests and measurements: force the few-row product's chunk length (128 or 256), its waves a
// workgroup (4; 8 count only with more than 32 rows of x) and its number of K slices; 0 leaves a choice to the library.  Process-wide:
// set it before the products it is meant for and clear it after (a caller that remembers
// yk_gemm_skinny_splits must ask again).
extern "C" int yk_gemm_skinny_force(int chunk, int waves, int slices) {
  YK_REQUIRE(chunk == 0 || chunk == 128 || chunk == 256, "gemm_skinny_force: chunks are 128 or 256 long");
  YK_REQUIRE(waves == 0 || waves == 4 || waves == 8, "gemm_skinny_force: a workgroup has 4 waves, or 8 (with more than 32 rows of x)");
  YK_REQUIRE(slices >= 0, "gemm_skinny_force: bad slice count");
  g_force_chunk = chunk;
  g_force_waves = waves;
  g_force_slices = slices;
  return 0;
}

extern "C" int yk_gemm_skinny_wide(int mode) {
  YK_REQUIRE(mode >= 0 && mode <= 2, "gemm_skinny_wide: 0 never, 1 by the library's rule, 2 always");
  g_wide = mode;
  return 0;
}

// gated != 0: the plan of a product with the activation in its epilogue (1: it can be fused).
extern "C" int yk_gemm_skinny_splits(int M, int N, int K, int gated) { return skinny_plan(M, N, K, gated != 0, nullptr, nullptr); }

template <typename TO>
static int launch_skinny(const bf16_t* x, const bf16_t* w, float* part, TO* y, int M, int N, int K,
                         int ldx, int ldw, int ldy, int waves, int k_block, int splits, int gated, hipStream_t stream,
                         const AttnSplits* from_splits = nullptr) {
  const int mt = skinny_mt(M);
  if (from_splits) {
    // x is attention's unmerged splits: one kernel form (up to 16 rows, four waves, no activation)
    if (mt != 1 || waves != 4 || gated || k_block > SK_SPLITS_MAX_K_BLOCK)
      return yk_fail("gemm_mfma_skinny: unmerged attention feeds plain products of up to 16 rows only");
    dim3 grid((N + 16 * waves - 1) / (16 * waves), 1, splits);
    const size_t lds = (static_cast<size_t>(16) * (k_block + SK_PAD) + static_cast<size_t>(16 * waves) * SK_ROW) * sizeof(bf16_t);
    static bool raised = false;
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_mfma_skinny_kernel<1, 4, TO, 0, true, SK_KC>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
        return yk_fail("gemm_mfma_skinny: cannot raise the LDS limit");
      raised = true;
    }
    gemm_mfma_skinny_kernel<1, 4, TO, 0, true, SK_KC><<<grid, dim3(256), lds, stream>>>(nullptr, w, part, y, M, N, K, 0, ldw, ldy, k_block, *from_splits);
    return yk_check_launch("gemm_mfma_skinny (from attention splits)");
  }
  dim3 grid((N + 16 * waves - 1) / (16 * waves), (M + 16 * mt - 1) / (16 * mt), splits);
  YK_REQUIRE(grid.y <= 65535, "gemm_mfma_skinny: too many rows for one launch");
  dim3 block(waves * 64);
  int kc = skinny_chunk(mt, k_block);
  // Long slices with 64 rows of x and eight waves: short chunks, two of them in flight per wave
  // (a register set each), in place of one long chunk: the same bytes in flight with half the
  // LDS a workgroup parks them in and a finer walk.  Measured on the 70B shape's down projection
  // (8,192 x 28,672 in four slices of 7,168; us, one long chunk / two short ones): 97.8 / 82.8 at
  // 64 rows of x, 96.7 / 80.2 at 48.  Where the slices are short enough for short chunks anyway,
  // a second chunk in flight costs 2 to 5 % (8B shape at 64 rows: gate/up 45.5 -> 46.6 us, down
  // 23.5 -> 24.5, qkv 13.9 -> 15.0), and four cost 8 to 10 %: the kernel is not short of bytes in
  // flight there.
  const bool wide = mt == 4 && (g_wide == 2 || (g_wide == 1 && K >= SK_WIDE_MIN_K && splits == 1));
  int depth = 1;
  if (!wide && mt == 4 && waves == 8 && !gated && !g_force_chunk && kc == SK_KC) {
    kc = 128;
    depth = 2;
  }
  const size_t lds = skinny_lds_bytes(mt, waves, kc);
  if (wide) {
    // waves of 32 weight rows: two of them (64 rows a workgroup) by the rule, half the plan's
    // number (the plan's rows a workgroup) when forced
    const int ww = g_wide == 2 ? waves / 2 : 2;
    dim3 wblock(ww * 64);
    grid.x = (N + 32 * ww - 1) / (32 * ww);
    const size_t lds = skinny_lds_bytes(mt, 2 * ww, kc);
#define SKW_GO(W_, G_) SKW_GO_KC(W_, G_, 128, 1) SKW_GO_KC(W_, G_, 256, 1)
#define SKW_GO_KC(W_, G_, KC_, D_)                                                                      \
  if (ww == W_ && gated == G_ && kc == KC_ && wdepth == D_) {                                           \
    static bool raised = false;                                                                         \
    if (!raised) {                                                                                      \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_mfma_skinny_wide_kernel<W_, TO, G_, KC_, D_>), \
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)    \
        return yk_fail("gemm_mfma_skinny: cannot raise the LDS limit");                                 \
      raised = true;                                                                                    \
    }                                                                                                   \
    gemm_mfma_skinny_wide_kernel<W_, TO, G_, KC_, D_><<<grid, wblock, lds, stream>>>(x, w, part, y, M, N, K, ldx, ldw, ldy, k_block); \
    return yk_check_launch("gemm_mfma_skinny (wide)");                                                  \
  }
    // With more than 48 rows of x the rule's two waves keep two long chunks in flight each (the 70B
    // shape's gate/up, us, one / two: 186.5 / 176 at 64 rows; 170 / 172 at 48 and 164 / 165 at 33,
    // so not there).
    const int wdepth = g_wide == 1 && !g_force_chunk && M > 48 && kc == SK_KC ? 2 : 1;
    SKW_GO_KC(2, 0, 256, 2)
    if constexpr (sizeof(TO) == 2) {
      SKW_GO_KC(2, 1, 256, 2) SKW_GO_KC(2, 2, 256, 2)
    }
    SKW_GO(2, 0) SKW_GO(4, 0)
    if constexpr (sizeof(TO) == 2) {
      SKW_GO(2, 1) SKW_GO(4, 1) SKW_GO(2, 2) SKW_GO(4, 2)
    }
#undef SKW_GO
#undef SKW_GO_KC
    return yk_fail("gemm_mfma_skinny: no wide kernel for this plan");
  }
#define SK_GO(MT_, W_, G_) SK_GO_KC(MT_, W_, G_, 128, 1) SK_GO_KC(MT_, W_, G_, 256, 1)
#define SK_GO_KC(MT_, W_, G_, KC_, D_)                                                                   \
  if (mt == MT_ && waves == W_ && gated == G_ && kc == KC_ && depth == D_) {                            \
    static bool raised = false; /* allow more than the default 64 KB of dynamic LDS, once */           \
    if (!raised) {                                                                                      \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_mfma_skinny_kernel<MT_, W_, TO, G_, false, KC_, D_>), \
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)    \
        return yk_fail("gemm_mfma_skinny: cannot raise the LDS limit");                                 \
      raised = true;                                                                                    \
    }                                                                                                   \
    gemm_mfma_skinny_kernel<MT_, W_, TO, G_, false, KC_, D_><<<grid, block, lds, stream>>>(x, w, part, y, M, N, K, ldx, ldw, ldy, k_block, AttnSplits{}); \
    return yk_check_launch("gemm_mfma_skinny");                                                         \
  }
  SK_GO_KC(4, 8, 0, 128, 2)
  SK_GO(1, 4, 0) SK_GO(2, 4, 0) SK_GO(4, 4, 0) SK_GO(4, 8, 0)
  if constexpr (sizeof(TO) == 2) {  // gated results are bfloat16 only
    SK_GO(1, 4, 1) SK_GO(2, 4, 1) SK_GO(4, 4, 1) SK_GO(4, 8, 1) SK_GO(1, 4, 2) SK_GO(2, 4, 2) SK_GO(4, 4, 2) SK_GO(4, 8, 2)
  }
#undef SK_GO
#undef SK_GO_KC
  return yk_fail("gemm_mfma_skinny: no kernel for this plan");
}

// The few-row product for checked arguments: plan, launch, and the reduction of the K slices
// unless the caller keeps them.  x, or (from_splits) attention's unmerged splits in its place.
static int skinny_product(const bf16_t* xp, const AttnSplits* from_splits, const bf16_t* wp, void* y, int y_dtype,
                          float* workspace, size_t workspace_floats, int M, int N, int K, int ldx, int ldw, int ldy,
                          int keep_splits, int gated, hipStream_t stream) {
  int k_block = 0, waves = 4;
  const int splits = skinny_plan(M, N, K, gated != 0, &waves, &k_block);
  YK_REQUIRE(!gated || splits == 1, "gemm_mfma_skinny: a gated product cannot split K");
  if (splits == 1 && !keep_splits) {
    int rc = y_dtype == YK_F32
                 ? launch_skinny<float>(xp, wp, nullptr, static_cast<float*>(y), M, N, K, ldx, ldw, ldy, waves, k_block, 1, gated, stream, from_splits)
                 : launch_skinny<bf16_t>(xp, wp, nullptr, static_cast<bf16_t*>(y), M, N, K, ldx, ldw, ldy, waves, k_block, 1, gated, stream, from_splits);
    return rc;
  }
  YK_REQUIRE(workspace && workspace_floats >= static_cast<size_t>(splits) * M * N,
             "gemm_mfma_skinny: workspace too small");
  if (launch_skinny<float>(xp, wp, workspace, nullptr, M, N, K, ldx, ldw, ldy, waves, k_block, splits, 0, stream, from_splits)) return -1;
  if (keep_splits) return splits;
  const size_t total = static_cast<size_t>(M) * N;
  const int rb = 256;
  const int rg = static_cast<int>(std::min<size_t>((total + rb - 1) / rb, 65535));
  if (y_dtype == YK_F32)
    reduce_splits_kernel<float><<<rg, rb, 0, stream>>>(workspace, static_cast<float*>(y), M, N, ldy, splits);
  else
    reduce_splits_kernel<bf16_t><<<rg, rb, 0, stream>>>(workspace, static_cast<bf16_t*>(y), M, N, ldy, splits);
  return yk_check_launch("reduce_splits");
}

// keep_splits != 0: leave the K slices unreduced in `workspace` ([splits][M][N] float32) for
// a consumer that sums them itself (y is not written unless there is a single slice and
// y is given).  Returns the number of slices written to the workspace (0: y holds the
// result), or a negative number on error.
// gated: 0 = y is the product [M, N].  1 (silu) or 2 (gelu-tanh): the rows of w alternate in
// groups of 8 gate rows and their 8 up rows, and y [M, N / 2] = act(gate) * up; only where the
// plan does not split K (yk_gemm_skinny_splits == 1), and N a multiple of 16.
extern "C" int yk_gemm_mfma_skinny(const void* x, const void* w, void* y, int y_dtype,
                                   float* workspace, size_t workspace_floats, int M, int N, int K,
                                   int ldx, int ldw, int ldy, int keep_splits, int gated,
                                   hipStream_t stream) {
  YK_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_mfma_skinny: bad sizes");
  YK_REQUIRE(K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_mfma_skinny: K and the leading dimensions must be multiples of 8");
  YK_REQUIRE((reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0),
             "gemm_mfma_skinny: operands must be 16-byte aligned");
  YK_REQUIRE(gated >= 0 && gated <= 2, "gemm_mfma_skinny: unknown activation");
  YK_REQUIRE(ldx >= K && ldw >= K && ldy >= (gated ? N / 2 : N), "gemm_mfma_skinny: leading dimensions too small");
  YK_REQUIRE(!gated || (N % 16 == 0 && y_dtype == YK_BF16 && !keep_splits), "gemm_mfma_skinny: a gated product needs N % 16 == 0 and a bfloat16 result");
  YK_REQUIRE(y_dtype == YK_F32 || y_dtype == YK_BF16, "gemm_mfma_skinny: unsupported output dtype");
  if (M == 0) return 0;
  return skinny_product(static_cast<const bf16_t*>(x), nullptr, static_cast<const bf16_t*>(w), y, y_dtype, workspace,
                        workspace_floats, M, N, K, ldx, ldw, ldy, keep_splits, gated, stream);
}

// Whether yk_gemm_mfma_skinny_from_attention takes a product of these sizes: up to 16 rows, and
// a plan whose K slices are short enough for a workgroup to hold its whole slice of x.
extern "C" int yk_gemm_skinny_from_attention_ok(int M, int N, int K) {
  if (M <= 0 || M > 16 || N <= 0 || K < 8 || K % 8) return 0;
  int k_block = 0, waves = 4;
  skinny_plan(M, N, K, false, &waves, &k_block);
  return waves == 4 && k_block <= SK_SPLITS_MAX_K_BLOCK;
}

// yk_gemm_mfma_skinny with x = the output of a yk_attn_mfma launch that left its splits in
// `attn_workspace` (leave_splits): the product merges them while it stages x, rounding to
// bfloat16 as yk_attn_combine would have stored them.  M tokens (at most 16), K = n_heads *
// head_dim; token_col[m] = 16 * (the token's tile in that launch) + (its place in the tile).
extern "C" int yk_gemm_mfma_skinny_from_attention(const float* attn_workspace, size_t attn_workspace_floats,
                                                  const int32_t* token_col, int n_tiles, int n_splits,
                                                  int n_heads, int n_kv, int head_dim, const void* w, void* y,
                                                  int y_dtype, float* workspace, size_t workspace_floats, int M,
                                                  int N, int ldw, int ldy, int keep_splits, hipStream_t stream) {
  YK_REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && head_dim > 0 && head_dim % 4 == 0, "gemm from attention: bad head sizes");
  YK_REQUIRE(n_splits > 1 && n_tiles > 0 && attn_workspace && token_col, "gemm from attention: no splits to merge");
  const int K = n_heads * head_dim;
  YK_REQUIRE(M >= 0 && N > 0 && ldw % 8 == 0 && ldw >= K && ldy >= N && reinterpret_cast<uintptr_t>(w) % 16 == 0,
             "gemm from attention: bad sizes or alignment");
  YK_REQUIRE(y_dtype == YK_F32 || y_dtype == YK_BF16, "gemm from attention: unsupported output dtype");
  YK_REQUIRE(yk_gemm_skinny_from_attention_ok(M, N, K) || M == 0, "gemm from attention: takes up to 16 rows and short K slices (ask yk_gemm_skinny_from_attention_ok)");
  if (M == 0) return 0;
  AttnSplits xa;
  xa.hpt = attn_heads_per_tile(n_heads, n_kv);
  xa.chunks = (n_heads / n_kv + xa.hpt - 1) / xa.hpt;
  const size_t cols = static_cast<size_t>(n_tiles) * n_kv * xa.chunks * n_splits * 16;
  YK_REQUIRE(attn_workspace_floats >= cols * (head_dim + 2), "gemm from attention: the attention workspace is too small for these tiles");
  xa.o = attn_workspace;
  xa.ml = attn_workspace + cols * head_dim;
  xa.token_col = token_col;
  xa.n_splits = n_splits;
  xa.n_heads = n_heads;
  xa.n_kv = n_kv;
  xa.head_dim = head_dim;
  return skinny_product(nullptr, &xa, static_cast<const bf16_t*>(w), y, y_dtype, workspace, workspace_floats, M, N, K, 0,
                        ldw, ldy, keep_splits, 0, stream);
}
