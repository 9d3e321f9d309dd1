// Causal attention with grouped key/value heads over the paged cache, for any span:
// the queries of a step's tokens (prompt portions and single decoded tokens alike)
// against the keys and values that the block tables name.
//
// Arithmetic (reference: yalis/attention/backend_impl/sdpa_and_flex.py:59-90, 300-312):
// score[h, p, j] = q[h, p] . k[h / (H/G), j] * scale; key j is visible to the query at
// position p iff j <= p (and p - j < window when a window is set); softmax over the
// visible keys in float32; output = P . V.
//
// Page layout: keys [page][kv_head][page_size][head_dim], values transposed
// [page][kv_head][head_dim][page_size].  Pages are never cleared, so nothing beyond a
// request's token count is ever read as a number: invisible scores are replaced, and
// values of tokens that do not exist yet, or that lie below a window, are zeroed before they meet a probability.
//
// Two kernels:
//  * attn_generic: one wave per (token, head), float32 arithmetic throughout, any
//    head_dim that is a multiple of 16 up to 256, float32 or bfloat16 storage.  This is
//    the true-32-bit path and the fallback for head sizes the matrix-core kernel lacks.
//  * attn_mfma: bfloat16 on the gfx950 matrix cores.  One wave owns 16 "columns": a few
//    consecutive tokens of one request times the query heads that share one key/value
//    head.  It computes S^T = K . Q^T and O^T = V^T . P^T, so that keys and transposed
//    values stream from memory straight into the matrix-core A operand and each lane
//    keeps one column's softmax state.  The visible keys can be split over several
//    waves; a second kernel merges the partial results in float32.
#include <algorithm>

#include "common.h"

// ---------------------------------------------------------------------------- generic
template <typename T>
__global__ __launch_bounds__(64) void attn_generic_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ token_seq, const int32_t* __restrict__ block_table, int table_width,
    int page_size, int head_dim, int n_heads, int n_kv, float scale, int window) {
  const bool tiled = cache_is_tiled(sizeof(T) == 2 ? YK_BF16 : YK_F32, head_dim, page_size);
  const size_t slab = static_cast<size_t>(page_size) * head_dim;
  __shared__ float qs[256];
  __shared__ float ps[64];
  __shared__ int pbase[64];  // (page * n_kv + kv_head) per key of the tile
  __shared__ int poff[64];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int qpk = n_heads / n_kv, g = h / qpk;
  const int pos = positions[n], seq = token_seq[n];
  const int hi = pos + 1;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const T* qrow = q + static_cast<size_t>(n) * q_stride + static_cast<size_t>(h) * head_dim;
  for (int d = lane; d < head_dim; d += 64) qs[d] = to_f32<T>(qrow[d]);
  __syncthreads();
  const int32_t* bt = block_table + static_cast<size_t>(seq) * table_width;
  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = lo; t0 < hi; t0 += 64) {
    const int key = t0 + lane;
    const bool valid = key < hi;
    float s = -INFINITY;
    int base = 0, off = 0;
    if (valid) {
      const int page = bt[key / page_size];
      off = key % page_size;
      base = page * n_kv + g;
      const T* kp = k_cache + static_cast<size_t>(base) * slab;
      float dot = 0.f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], to_f32<T>(kp[cache_k_offset(tiled, page_size, head_dim, off, d)]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: the tile holds at least one key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // 0 on the first tile
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();  // the previous tile's ps/pbase are no longer read
    ps[lane] = p;
    pbase[lane] = base;
    poff[lane] = off;
    __syncthreads();
    const int count = min(64, hi - t0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < head_dim) {
        float a = acc[i] * alpha;
        for (int j = 0; j < count; ++j) {
          const T* vp = v_cache + static_cast<size_t>(pbase[j]) * slab + cache_v_offset(tiled, page_size, head_dim, poff[j], d);
          a = fmaf(ps[j], to_f32<T>(*vp), a);
        }
        acc[i] = a;
      }
    }
  }
  T* orow = out + (static_cast<size_t>(n) * n_heads + h) * head_dim;
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < head_dim) orow[d] = from_f32<T>(acc[i] * inv);
  }
}

extern "C" int yk_attn_generic(const void* q, int q_stride, void* out, const void* k_cache,
                               const void* v_cache, int dtype, const int32_t* positions,
                               const int32_t* token_seq, const int32_t* block_table,
                               int table_width, int n_tokens, int page_size, int head_dim,
                               int n_heads, int n_kv, float scale, int window,
                               hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv > 0, "attention: bad sizes");
  YK_REQUIRE(n_heads % n_kv == 0, "attention: the head count must be a multiple of the kv head count");
  YK_REQUIRE(head_dim > 0 && head_dim % 16 == 0 && head_dim <= 256,
             "attention: head_dim must be a multiple of 16 and at most 256");
  YK_REQUIRE(page_size > 0 && table_width > 0, "attention: bad page table");
  YK_REQUIRE(n_heads <= 65535, "attention: too many heads for one launch");
  YK_REQUIRE(window >= 0, "attention: window must not be negative");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, n_heads), block(64);
  if (dtype == YK_F32)
    attn_generic_kernel<float><<<grid, block, 0, stream>>>(
        static_cast<const float*>(q), q_stride, static_cast<float*>(out),
        static_cast<const float*>(k_cache), static_cast<const float*>(v_cache), positions,
        token_seq, block_table, table_width, page_size, head_dim, n_heads, n_kv, scale, window);
  else if (dtype == YK_BF16)
    attn_generic_kernel<bf16_t><<<grid, block, 0, stream>>>(
        static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out),
        static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), positions,
        token_seq, block_table, table_width, page_size, head_dim, n_heads, n_kv, scale, window);
  else
    return yk_fail("attention: unsupported dtype");
  return yk_check_launch("attn_generic");
}

// ------------------------------------------------------------------------ matrix cores
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

union AFrag8 {
  u32x4_t u;
  bf16x8_t v;
  bf16_t h[8];
};


// 2^x for scores: -inf gives 0, no denormal handling needed
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Layout of a tile row handed over by the host: (request, first token index in the
// batch, token count, position of the first token).
//
// Columns of a wave: column c in 0..15 is token c / hpt of the tile and query head
// h_base + c % hpt, hpt = min(H/G, 16) heads per tile; a kv head with more than 16
// query heads takes several "chunks" of 16.
//
// Keys are walked in blocks of 64 = two groups of 32.  Within a group the 16 rows of the
// two score products are assigned to keys so that afterwards lane group g holds the
// probabilities of keys 8g .. 8g+7 of the group in order: row i of the first product is key
// 8*(i/4) + i%4, row i of the second is key 8*(i/4) + 4 + i%4.  Then the transposed values
// feed the second product as one 16-byte load per lane (8 consecutive keys of one value
// row).  Every load is unconditional (addresses are clamped into allocated pages, what they
// bring for keys that do not count is masked or zeroed), so that the values of a block and
// the keys of the next are in flight while the block's scores are worked on.
//
// A workgroup has W waves that share the columns and divide the workgroup's key blocks
// among themselves; at the end waves 1.. hand their running maximum, sum and output to
// wave 0 through LDS (every lane to the same lane), and wave 0 merges and stores.  Across
// workgroups (blockIdx.z) the keys are split further when the launch needs more waves;
// those partial results go through the workspace to the combine kernel.
//
// TILED: the pages are stored in the order these loads take them (cache_is_tiled): a block of
// 64 keys lies in one page, its page is looked up once, and every load instruction reads
// 1 KiB of consecutive memory instead of 16 rows x 64 bytes (measured at 64 requests of 1,024
// tokens: 46 us a layer against 58).
//
// ROPE: the launch also does what rotary + append would have done before it, for steps whose
// tiles hold one token each (single decoded tokens).  The queries are then not read from `q`
// but made from the projection's raw output rows [query heads | key heads | value heads]
// (bfloat16, or the unreduced float32 K slices of the product): every workgroup sums the
// slices of its heads, rotates them by the token's angle and parks them in LDS in bfloat16,
// with the arithmetic and roundings of rope_append_kernel, so the bits are those of the
// two-kernel path.  The token's own key and value are not in the pages yet: the one workgroup
// (per kv head and split) whose share of the keys holds the token's position makes them too,
// puts them into its operand registers in place of what the pages gave, and (chunk 0 only)
// stores them in the pages for later steps.  Nobody reads that slot of the pages as a number
// in this launch.
struct RopeSrc {
  const void* src;      // [tokens][src_stride] rows, n_splits slices split_stride elements apart:
                        // float32 (slices are summed, the sum rounded when round_sum) or bfloat16
  int n_splits;
  size_t split_stride;
  int round_sum;
  int src_stride;
  const float* cos_t;   // [max_positions][rotary_dim / 2] (null when rotary_dim == 0)
  const float* sin_t;
  int rotary_dim, interleaved, max_positions;
  int append;           // 1: src holds the token's key and value heads too; they go to the pages
};

// Up to eight slices of one element, all asked for before any is used (a slice index beyond
// the last is clamped and its value dropped, so that the loads carry no condition).
// SRC 1: bfloat16 rows (one slice); SRC 2: float32 slices.
template <int SRC>
__device__ __forceinline__ void rope_src_load8(const void* src, size_t row, int idx, const size_t (&slice)[8], float (&d)[8]) {
  if (SRC == 1) {
    d[0] = bf16_to_f32(static_cast<const bf16_t*>(src)[row + idx]);
#pragma unroll
    for (int j = 1; j < 8; ++j) d[j] = 0.f;
  } else {
    const float* p = static_cast<const float*>(src) + row + idx;
#pragma unroll
    for (int j = 0; j < 8; ++j) d[j] = p[slice[j]];
  }
}
// where the slices s0 .. s0 + 7 start (clamped to the last)
__device__ __forceinline__ void rope_src_slices(int s0, int n_splits, size_t split_stride, size_t (&slice)[8]) {
#pragma unroll
  for (int j = 0; j < 8; ++j) slice[j] = static_cast<size_t>(min(s0 + j, n_splits - 1)) * split_stride;
}
// added in the order of the slices, as every other consumer of a product's slices adds them
__device__ __forceinline__ float rope_src_add8(float acc, const float (&d)[8], int s0, int n_splits) {
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (s0 + j < n_splits) acc += d[j];
  return acc;
}

template <int D, int W, bool TILED, int SRC>
__global__ __launch_bounds__(64 * W, 2) void attn_mfma_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* k_cache, const bf16_t* v_cache,  // (written too, with ROPE: the token's own slot)
    const int32_t* __restrict__ tiles, const int32_t* __restrict__ block_table, int table_width,
    int page_size, int n_heads, int n_kv, int hpt, int chunks, float scale_log2, int window,
    int n_splits, float* __restrict__ ws_o, float* __restrict__ ws_ml, RopeSrc rs) {
  constexpr int KS = D / 32;  // matrix-core steps over the head dimension
  constexpr int DT = D / 16;  // output tiles over the head dimension
  constexpr bool ROPE = SRC != 0;  // SRC 0: queries from `q`; 1, 2: rotary + append in here (rope_src_load8)
  const int lane = threadIdx.x % 64, r = lane % 16, gq = lane / 16;
  // (the same in every lane, and said so: what hangs on it then branches instead of masking lanes)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int t = blockIdx.x;
  const int seq = tiles[4 * t], tok0 = tiles[4 * t + 1], pos0 = tiles[4 * t + 3];
  const int ntok = ROPE ? 1 : tiles[4 * t + 2];
  const int g = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
  const int qpk = n_heads / n_kv;
  const int h_base = g * qpk + chunk * hpt;
  const int heads_here = min(hpt, qpk - chunk * hpt);
  const int tt = r / hpt, hh = r % hpt;
  const bool col_ok = tt < ntok && hh < heads_here;
  const int pos_c = pos0 + tt;
  const int lo_c = window > 0 ? max(0, pos_c - window + 1) : 0;
  const int hi = pos0 + ntok;
  const int lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int kb_lo = lo / 64, kb_hi = (hi + 63) / 64;
  const int per_split = (kb_hi - kb_lo + n_splits - 1) / n_splits;
  const int wg_lo = kb_lo + blockIdx.z * per_split;
  const int wg_hi = min(kb_hi, wg_lo + per_split);
  // the waves divide the workgroup's keys in halves of a block (32 keys: one group of the two
  // score products), so that the longest share is at most half a block above the mean; a half
  // beyond the last key is nobody's.  A half that is not the wave's own is not loaded: its keys
  // and values stand as zeros in the products and its scores are masked.
  const int h_lo = wg_lo * 2, h_hi = min(wg_hi * 2, (hi + 31) / 32);
  const int per_wave = (max(0, h_hi - h_lo) + W - 1) / W;
  const int my_hlo = h_lo + wave * per_wave;
  const int my_hhi = min(h_hi, my_hlo + per_wave);
  const int my_lo = my_hlo / 2;
  const int my_hi = my_hlo < my_hhi ? (my_hhi + 1) / 2 : my_lo;
  auto mine = [&](int kb, int u) { return 2 * kb + u >= my_hlo && 2 * kb + u < my_hhi; };
  const int32_t* bt = block_table + static_cast<size_t>(seq) * table_width;
  const int last_page_col = min(table_width - 1, (hi - 1) / page_size);

  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  float m = -INFINITY, l = 0.f;
  f32x4_t acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // the key this lane's score rows stand for, relative to the block: [group][product]
  const int krow = 8 * (r / 4) + r % 4;
  // a page that exists for any key: keys beyond the request read the last allocated page
  auto page_of = [&](int key) { return max(0, bt[min(key / page_size, last_page_col)]); };

  AFrag8 kf[2][2][KS];
#define ATT_LOAD_K(KB) ATT_LOAD_K_AT(KB, page_of((KB) * 64))
  // PAGE0: the page of the block's first key, for tiled pages (looked up by the caller)
#define ATT_LOAD_K_AT(KB, PAGE0)                                                                  \
  {                                                                                                \
  if (TILED) {                                                                                     \
    const int key0 = (KB) * 64;                                                                    \
    const bf16_t* kp = k_cache + (static_cast<size_t>(PAGE0) * n_kv + g) * page_size * D +         \
                       static_cast<size_t>(key0 % page_size) * D + 8 * lane;                       \
    _Pragma("unroll") for (int u = 0; u < 2; ++u) {                                                \
      if (mine((KB), u)) {                                                                         \
        _Pragma("unroll") for (int sb = 0; sb < 2; ++sb)                                           \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                          \
            kf[u][sb][ks].u = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(kp + ((u * 2 + sb) * KS + ks) * 512)); \
      } else {                                                                                     \
        _Pragma("unroll") for (int sb = 0; sb < 2; ++sb)                                           \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) kf[u][sb][ks].u = zero4;                 \
      }                                                                                            \
    }                                                                                              \
  } else {                                                                                         \
    _Pragma("unroll") for (int u = 0; u < 2; ++u) {                                                \
      if (mine((KB), u)) {                                                                         \
        _Pragma("unroll") for (int sb = 0; sb < 2; ++sb) {                                         \
          const int key = (KB) * 64 + 32 * u + krow + 4 * sb;                                     \
          const bf16_t* kp = k_cache + ((static_cast<size_t>(page_of(key)) * n_kv + g) * page_size + key % page_size) * D + 8 * gq; \
          _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                       \
              kf[u][sb][ks].u = *reinterpret_cast<const u32x4_t*>(kp + 32 * ks);                  \
        }                                                                                          \
      } else {                                                                                     \
        _Pragma("unroll") for (int sb = 0; sb < 2; ++sb)                                           \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) kf[u][sb][ks].u = zero4;                 \
      }                                                                                            \
    }                                                                                              \
  }                                                                                                \
  }

  // values of a block: lane (r, gq) holds 8 consecutive keys of value row 16*dt + r
  AFrag8 vf[2][DT];
#define ATT_LOAD_V_AT(KB, PAGE0)                                                                   \
  {                                                                                                \
  if (TILED) {                                                                                     \
    const int key0 = (KB) * 64;                                                                    \
    const bf16_t* vp = v_cache + (static_cast<size_t>(PAGE0) * n_kv + g) * D * page_size +         \
                       static_cast<size_t>(key0 % page_size) * D + 8 * lane;                       \
    _Pragma("unroll") for (int u = 0; u < 2; ++u) {                                                \
      if (mine((KB), u)) {                                                                         \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt)                                          \
            vf[u][dt].u = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(vp + (u * DT + dt) * 512)); \
      } else {                                                                                     \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) vf[u][dt].u = zero4;                     \
      }                                                                                            \
    }                                                                                              \
  } else {                                                                                         \
    _Pragma("unroll") for (int u = 0; u < 2; ++u) {                                                \
      if (mine((KB), u)) {                                                                         \
        const int key = (KB) * 64 + 32 * u + 8 * gq;                                               \
        const bf16_t* vp = v_cache + (static_cast<size_t>(page_of(key)) * n_kv + g) * D * page_size + key % page_size; \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt)                                          \
            vf[u][dt].u = *reinterpret_cast<const u32x4_t*>(vp + static_cast<size_t>(16 * dt + r) * page_size); \
      } else {                                                                                     \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) vf[u][dt].u = zero4;                     \
      }                                                                                            \
    }                                                                                              \
  }                                                                                                \
  }

  // ROPE: the token's own key replaces what the pages gave for its slot
#define ATT_PUT_NEW_K(KB)                                                                          \
  if (ROPE && makes_kv && (KB) == kb_new && r == new_r) {                                          \
    _Pragma("unroll") for (int u = 0; u < 2; ++u)                                                  \
    _Pragma("unroll") for (int sb = 0; sb < 2; ++sb)                                               \
      if (u == new_u && sb == new_sb && mine((KB), u)) {                                           \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                          \
            kf[u][sb][ks].u = *reinterpret_cast<const u32x4_t*>(&kv_s[0][32 * ks + 8 * gq]);       \
      }                                                                                            \
  }
  AFrag8 qf[KS];
  // ROPE: the block of 64 keys that holds the token's own position, and whether this workgroup
  // is the one that makes the token's key and value (its share of the keys holds that block)
  const int kb_new = pos0 / 64;
  const bool makes_kv = ROPE && rs.append && kb_new >= wg_lo && kb_new < wg_hi;
  __shared__ __attribute__((aligned(16))) bf16_t q_s[ROPE ? 16 : 1][ROPE ? D : 8];
  __shared__ __attribute__((aligned(16))) bf16_t kv_s[2][ROPE ? D : 8];  // the token's key, its value
  // ROPE: items of two elements: D / 2 a head (a rotated pair, or two neighbours beyond the
  // rotated part) for the query heads, then, where this workgroup makes them, for the key head
  // and (never rotated) the value head.  A thread takes two items a round, T apart (the second
  // only where the workgroup has more items than threads), and asks for everything both need
  // before it uses any of it: in most launches there is one round, and one wait for memory.
  constexpr int T = 64 * W;
  if (ROPE) {
    const int items = (heads_here + (makes_kv ? 2 : 0)) * (D / 2);
    const int half = rs.rotary_dim / 2;
    const size_t row = static_cast<size_t>(tok0) * rs.src_stride;
    const size_t at = static_cast<size_t>(min(max(pos0, 0), rs.max_positions - 1)) * half;
    // (without a table the loads below read a valid word that is never used)
    const float* cs = half > 0 ? rs.cos_t + at : reinterpret_cast<const float*>(tiles);
    const float* sn = half > 0 ? rs.sin_t + at : reinterpret_cast<const float*>(tiles);
    const int half_m1 = max(half - 1, 0);
    const int src_splits = SRC == 2 ? rs.n_splits : 1;
    const size_t src_split_stride = rs.split_stride;
    // the page of the first block is asked for first: the keys' addresses wait for it, and a
    // wait for an older load leaves the younger ones in flight
    const int first_page = my_lo < my_hi ? page_of(my_lo * 64) : 0;
    // one round; LOAD_K: the first block's keys are asked for while the round's rows are on
    // their way (the first round is straight-line code: its loads are all issued before the
    // first of them is waited for; rows of more than eight slices finish in a loop)
    auto round = [&](int first, auto load_k) {
      const bool two = first + T < items;  // the same for every thread
      int ia[2], ib[2], base[2];
      bf16_t* dst[2];
      bool rot[2], ok[2];
      float c[2], sv[2], acc_a[2], acc_b[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int item = first + j * T + static_cast<int>(threadIdx.x);
        ok[j] = item < items;
        const int it = ok[j] ? item : 0;
        const int hq = it / (D / 2), i = it % (D / 2);
        const bool is_k = hq == heads_here, is_v = hq == heads_here + 1;
        base[j] = (is_v ? n_heads + n_kv + g : (is_k ? n_heads + g : h_base + hq)) * D;
        dst[j] = is_v ? kv_s[1] : (is_k ? kv_s[0] : q_s[hq]);
        rot[j] = !is_v && i < half;
        ia[j] = rot[j] ? (rs.interleaved ? 2 * i : i) : (is_v ? 2 * i : rs.rotary_dim + 2 * (i - half));
        ib[j] = rot[j] ? (rs.interleaved ? 2 * i + 1 : i + half) : ia[j] + 1;
        c[j] = cs[min(i, half_m1)];  // (clamped: asked for whether the pair rotates or not)
        sv[j] = sn[min(i, half_m1)];
      }
      float da0[8], db0[8], da1[8], db1[8];
      size_t slice[8];
      rope_src_slices(0, src_splits, src_split_stride, slice);
      rope_src_load8<SRC>(rs.src, row, base[0] + ia[0], slice, da0);
      rope_src_load8<SRC>(rs.src, row, base[0] + ib[0], slice, db0);
      if (two) {
        rope_src_load8<SRC>(rs.src, row, base[1] + ia[1], slice, da1);
        rope_src_load8<SRC>(rs.src, row, base[1] + ib[1], slice, db1);
      }
      load_k();
      acc_a[0] = rope_src_add8(0.f, da0, 0, src_splits);
      acc_b[0] = rope_src_add8(0.f, db0, 0, src_splits);
      acc_a[1] = acc_b[1] = 0.f;
      if (two) {
        acc_a[1] = rope_src_add8(0.f, da1, 0, src_splits);
        acc_b[1] = rope_src_add8(0.f, db1, 0, src_splits);
      }
      for (int s0 = 8; s0 < src_splits; s0 += 8) {
        rope_src_slices(s0, src_splits, src_split_stride, slice);
        rope_src_load8<SRC>(rs.src, row, base[0] + ia[0], slice, da0);
        rope_src_load8<SRC>(rs.src, row, base[0] + ib[0], slice, db0);
        rope_src_load8<SRC>(rs.src, row, base[1] + ia[1], slice, da1);
        rope_src_load8<SRC>(rs.src, row, base[1] + ib[1], slice, db1);
        acc_a[0] = rope_src_add8(acc_a[0], da0, s0, src_splits);
        acc_b[0] = rope_src_add8(acc_b[0], db0, s0, src_splits);
        acc_a[1] = rope_src_add8(acc_a[1], da1, s0, src_splits);
        acc_b[1] = rope_src_add8(acc_b[1], db1, s0, src_splits);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (ok[j] && (j == 0 || two)) {
          const float a = as_output(acc_a[j], rs.round_sum), b = as_output(acc_b[j], rs.round_sum);
          dst[j][ia[j]] = f32_to_bf16(rot[j] ? rot_first(a, b, c[j], sv[j]) : a);
          dst[j][ib[j]] = f32_to_bf16(rot[j] ? rot_second(a, b, c[j], sv[j]) : b);
        }
    };
    round(0, [&]() {
      if (my_lo < my_hi) {
        ATT_LOAD_K_AT(my_lo, first_page)
        ATT_LOAD_V_AT(my_lo, first_page)
      }
    });
    for (int first = 2 * T; first < items; first += 2 * T) round(first, []() {});
    __syncthreads();
    if (makes_kv && chunk == 0) {
      // into the pages, for the steps that follow
      const int slot = pos0 % page_size;
      const size_t slab = (static_cast<size_t>(max(0, bt[min(pos0 / page_size, table_width - 1)])) * n_kv + g) * page_size * D;
      for (int d = threadIdx.x; d < D; d += 64 * W) {
        const_cast<bf16_t*>(k_cache)[slab + cache_k_offset(TILED, page_size, D, slot, d)] = kv_s[0][d];
        const_cast<bf16_t*>(v_cache)[slab + cache_v_offset(TILED, page_size, D, slot, d)] = kv_s[1][d];
      }
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[ks].u = col_ok ? *reinterpret_cast<const u32x4_t*>(&q_s[hh][32 * ks + 8 * gq]) : zero4;
  } else {
    const bf16_t* qp = q + static_cast<size_t>(tok0 + (col_ok ? tt : 0)) * q_stride +
                       static_cast<size_t>(h_base + (col_ok ? hh : 0)) * D + 8 * gq;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks].u = *reinterpret_cast<const u32x4_t*>(qp + 32 * ks);
      if (!col_ok) qf[ks].u = zero4;
    }
  }
  // where the token's own key sits among a block's score rows and value pieces
  const int new_j = pos0 % 64, new_u = new_j / 32;
  const int new_sb = (new_j % 8) / 4, new_r = 4 * ((new_j % 32) / 8) + new_j % 4;  // key row of the score products
  const int new_gq = (new_j % 32) / 8, new_e = new_j % 8;                          // value piece and place in it
  if (my_lo < my_hi) {
    if (!ROPE) ATT_LOAD_K(my_lo)
    ATT_PUT_NEW_K(my_lo)
  }
  for (int kb = my_lo; kb < my_hi; ++kb) {
    const bool mine0 = mine(kb, 0), mine1 = mine(kb, 1);
    if (!(ROPE && kb == my_lo)) ATT_LOAD_V_AT(kb, page_of(kb * 64))  // (ROPE: the first block's are on their way)
    // scores
    f32x4_t s[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
        s[u][sb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          s[u][sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][sb][ks].v, qf[ks].v, s[u][sb], 0, 0, 0);
      }
    if (kb + 1 < my_hi) {
      ATT_LOAD_K(kb + 1)
      ATT_PUT_NEW_K(kb + 1)
    }
    float tmax = -INFINITY;
    // a block that every column sees whole needs no mask (columns that stand for nothing
    // compute on zeros and are never stored)
    const bool whole = mine0 && mine1 && kb * 64 + 63 <= pos0 && (window == 0 || kb * 64 >= max(0, pos0 + ntok - window));
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (!whole) {
            const int key = kb * 64 + 32 * u + 8 * gq + 4 * sb + i;
            const bool ok = col_ok && key <= pos_c && key >= lo_c && (u == 0 ? mine0 : mine1);
            if (!ok) s[u][sb][i] = -INFINITY;
          }
          tmax = fmaxf(tmax, s[u][sb][i]);
        }
    tmax = column_lanes_max(tmax);
    // the maximum was taken over the raw scores (the scale is positive); the scale joins the
    // subtraction of the maximum in one fused multiply-add
    const float m_new = fmaxf(m, tmax * scale_log2);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const bool grew = __any(m_new > m);  // only then the running sums need rescaling
    const float alpha = fast_exp2(m - m_safe);
    float psum = 0.f;
    AFrag8 pf[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[u][sb][i] = fast_exp2(fmaf(s[u][sb][i], scale_log2, -m_safe));
          psum += s[u][sb][i];
        }
        pf[u].u[2 * sb] = pack_bf16x2(s[u][sb][0], s[u][sb][1]);
        pf[u].u[2 * sb + 1] = pack_bf16x2(s[u][sb][2], s[u][sb][3]);
      }
    }
    l = l * alpha + psum;
    m = m_new;
    if (grew) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[dt] *= alpha;
    }
    // values of keys that do not exist yet, or that lie below the window (their pages may have
    // been given back), may be anything: zero them (the last and the first block only)
    if (kb * 64 + 64 > hi || kb * 64 < lo) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int key = kb * 64 + 32 * u + 8 * gq;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (key + e >= hi || key + e < lo) vf[u][dt].h[e] = 0;
      }
    }
    if (ROPE && makes_kv && kb == kb_new && gq == new_gq) {
      // the token's own value: element new_e of this lane's piece of every value row, put in
      // with word masks (an index into the registers would not stay in registers)
      const uint32_t keep = new_e % 2 ? 0x0000ffffu : 0xffff0000u;
#pragma unroll
      for (int u = 0; u < 2; ++u)
        if (u == new_u && (u == 0 ? mine0 : mine1)) {
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const uint32_t v = static_cast<uint32_t>(kv_s[1][16 * dt + r]) << (new_e % 2 ? 16 : 0);
#pragma unroll
            for (int wd = 0; wd < 4; ++wd)
              if (wd == new_e / 2) vf[u][dt].u[wd] = (vf[u][dt].u[wd] & keep) | v;
          }
        }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[u][dt].v, pf[u].v, acc[dt], 0, 0, 0);
  }
#undef ATT_LOAD_K
#undef ATT_LOAD_K_AT
#undef ATT_LOAD_V_AT
#undef ATT_PUT_NEW_K
  l = column_lanes_sum(l);

  if (W > 1) {
    constexpr int WP = W > 1 ? W - 1 : 1;
    __shared__ f32x4_t part_o[WP][DT][64];
    __shared__ float part_m[WP][64], part_l[WP][64];
    if (wave > 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) part_o[wave - 1][dt][lane] = acc[dt];
      part_m[wave - 1][lane] = m;
      part_l[wave - 1][lane] = l;
    }
    __syncthreads();
    if (wave > 0) return;
    float m_all = m;
#pragma unroll
    for (int w = 0; w < W - 1; ++w) m_all = fmaxf(m_all, part_m[w][lane]);
    const float m_safe = m_all == -INFINITY ? 0.f : m_all;
    const float a0 = fast_exp2(m - m_safe);
    l *= a0;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] *= a0;
#pragma unroll
    for (int w = 0; w < W - 1; ++w) {
      const float aw = fast_exp2(part_m[w][lane] - m_safe);
      l += aw * part_l[w][lane];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[dt] += aw * part_o[w][dt][lane];
    }
    m = m_all;
  }

  if (n_splits == 1) {
    if (col_ok) {
      const float inv = 1.f / l;
      bf16_t* op = out + (static_cast<size_t>(tok0 + tt) * n_heads + h_base + hh) * D + 4 * gq;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        u32x2_t w;
        w[0] = pack_bf16x2(acc[dt][0] * inv, acc[dt][1] * inv);
        w[1] = pack_bf16x2(acc[dt][2] * inv, acc[dt][3] * inv);
        *reinterpret_cast<u32x2_t*>(op + 16 * dt) = w;
      }
    }
  } else {
    // partial result of this split: unnormalised output, running maximum and sum
    const size_t widx = (static_cast<size_t>(t) * gridDim.y + blockIdx.y) * n_splits + blockIdx.z;
    float* wo = ws_o + (widx * 16 + r) * D + 4 * gq;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4_t*>(wo + 16 * dt) = acc[dt];
    if (gq == 0) {
      ws_ml[(widx * 16 + r) * 2] = m;
      ws_ml[(widx * 16 + r) * 2 + 1] = l;
    }
  }
}

// The same arithmetic for long spans (prompt portions): a workgroup of four waves owns one
// long tile of a request; every wave has CT column tiles of 16 (consecutive tokens), so the
// workgroup walks the keys once for 64 * CT columns and every key or value operand read from
// LDS feeds CT products.  Each block of 64 keys and values is fetched from the pages with
// coalesced loads, parked in LDS (keys in the row order the score products read them, so
// that the reads are free of bank conflicts) and read from there by the four waves; the next
// block's loads are in flight meanwhile.  The keys are split across workgroups only where
// few tiles meet a long context.
// CT is the caller's choice, with the tiles it built: one column tile per wave (three
// workgroups a CU) balances the triangle of a prompt that starts from nothing; two (224
// registers, two workgroups a CU) stage every block through LDS for twice the columns and
// win where many tiles each meet thousands of keys (measured on the 8B shape: 2,048 tokens
// against 8,192 cached 383 us against 499, a whole 2,048-token prompt 99 us against 80).
template <int D, bool TILED, int CT>
__global__ __launch_bounds__(256, CT == 1 ? 3 : 2) void attn_mfma_prefill_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ tiles, const int32_t* __restrict__ block_table, int table_width,
    int page_size, int n_heads, int n_kv, int hpt, int chunks, float scale_log2, int window,
    int n_splits, float* __restrict__ ws_o, float* __restrict__ ws_ml, int pages_lds_limit) {
  constexpr int KS = D / 32, DT = D / 16;
  constexpr int KROW = D + 8;   // bf16 elements per parked key row
  constexpr int VROW = 64 + 8;  // bf16 elements per parked value row
  constexpr int PP = D / 32;    // 16-byte pieces of keys (and of values) per thread and block
  __shared__ __attribute__((aligned(16))) bf16_t ks[64][KROW];
  __shared__ __attribute__((aligned(16))) bf16_t vs[D][VROW];
  const int lane = threadIdx.x % 64, r = lane % 16, gq = lane / 16;
  // (the same in every lane, and said so: what hangs on it then branches instead of masking lanes)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  // Workgroups start in the order of blockIdx.x: heads vary fastest, so that the tiles the
  // host put first (those with the most keys) start first on every head and the short ones
  // fill the gaps at the end; consecutive workgroups, which land on different dies, hold
  // different kv heads.
  const int n_y = n_kv * chunks;
  const int t = blockIdx.x / n_y, by = blockIdx.x % n_y;
  const int seq = tiles[4 * t], tile_tok0 = tiles[4 * t + 1], tile_ntok = tiles[4 * t + 2], tile_pos0 = tiles[4 * t + 3];
  const int g = by / chunks, chunk = by % chunks;
  const int qpk = n_heads / n_kv;
  const int h_base = g * qpk + chunk * hpt;
  const int heads_here = min(hpt, qpk - chunk * hpt);
  const int tpt = 16 / hpt;  // tokens per column tile
  const int tt = r / hpt, hh = r % hpt;
  const int wave_tok0 = wave * CT * tpt;  // first token of this wave within the tile
  int tok_c[CT], pos_c[CT], lo_c[CT];
  bool col_ok[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    tok_c[c] = wave_tok0 + c * tpt + tt;
    col_ok[c] = tt < tpt && tok_c[c] < tile_ntok && hh < heads_here;
    pos_c[c] = tile_pos0 + tok_c[c];
    lo_c[c] = window > 0 ? max(0, pos_c[c] - window + 1) : 0;
  }
  const int hi = tile_pos0 + tile_ntok;  // keys the workgroup may need
  const int lo = window > 0 ? max(0, tile_pos0 - window + 1) : 0;
  const int wave_hi = min(hi, tile_pos0 + wave_tok0 + CT * tpt);  // keys this wave may need
  // the workgroup's share of the key blocks when a launch splits them (blockIdx.y): few long
  // tiles against a long context would otherwise leave most of the GPU idle
  const int all_lo = lo / 64, all_hi = (hi + 63) / 64;
  const int per_split = (all_hi - all_lo + n_splits - 1) / n_splits;
  const int kb_lo = all_lo + blockIdx.y * per_split, kb_hi = min(all_hi, kb_lo + per_split);
  const int32_t* bt = block_table + static_cast<size_t>(seq) * table_width;
  const int last_page_col = min(table_width - 1, (hi - 1) / page_size);
  // page ids of the keys this workgroup walks, once, into LDS (a lookup per fetched piece
  // would put a dependent memory round trip before every load)
  constexpr int PAGES_LDS = 2048;
  __shared__ int32_t pages_s[PAGES_LDS];
  const int first_col = min(last_page_col, max(0, kb_lo) * 64 / page_size);
  // (pages_lds_limit: at most PAGES_LDS; tests lower it to walk the other way with short tables)
  const bool pages_in_lds = last_page_col - first_col < min(PAGES_LDS, pages_lds_limit);
  if (pages_in_lds)
    for (int c = first_col + threadIdx.x; c <= last_page_col; c += 256) pages_s[c - first_col] = max(0, bt[c]);
  const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
  auto page_col = [&](int key) { return min(page_shift >= 0 ? key >> page_shift : key / page_size, last_page_col); };
  auto page_off = [&](int key) { return page_shift >= 0 ? key & (page_size - 1) : key % page_size; };
  auto page_of = [&](int key) {
    const int c = page_col(key);
    return pages_in_lds ? pages_s[c - first_col] : max(0, bt[c]);
  };
  __syncthreads();

  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  AFrag8 qf[CT][KS];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const bf16_t* qp = q + static_cast<size_t>(tile_tok0 + (col_ok[c] ? tok_c[c] : 0)) * q_stride +
                       static_cast<size_t>(h_base + (col_ok[c] ? hh : 0)) * D + 8 * gq;
#pragma unroll
    for (int ks_ = 0; ks_ < KS; ++ks_) {
      qf[c][ks_].u = *reinterpret_cast<const u32x4_t*>(qp + 32 * ks_);
      if (!col_ok[c]) qf[c][ks_].u = zero4;
    }
  }
  float m[CT], l[CT];
  f32x4_t acc[CT][DT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    m[c] = -INFINITY;
    l[c] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[c][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // what this thread fetches of every block: PP pieces of keys and PP pieces of values.
  // Tiled pages (a multiple of 64 tokens): a block lies in one page as 2 x 16 KiB of consecutive
  // pieces; the page id is looked up once per block, thread e takes pieces e, e + 256, ... and
  // works out once which key and dims (or dim and keys) each of them holds.
  u32x4_t kreg[PP], vreg[PP];
  int k_key[PP], k_piece[PP], v_dim[PP], v_key[PP];  // of piece p: key (0..63) and 8-dim piece; dim and first key
#pragma unroll
  for (int p = 0; p < PP; ++p) {
    const int e = threadIdx.x + 256 * p;
    if (TILED) {
      const int rr = e % 16, gg = (e / 16) % 4;
      const int kk = (e / 64) % KS, usb = e / (64 * KS);  // u * 2 + sb
      k_key[p] = 32 * (usb / 2) + 8 * (rr / 4) + 4 * (usb % 2) + rr % 4;
      k_piece[p] = 4 * kk + gg;
      const int dd = (e / 64) % DT, uu = e / (64 * DT);
      v_dim[p] = 16 * dd + rr;
      v_key[p] = 32 * uu + 8 * gg;
    } else {
      k_key[p] = e / (D / 8);
      k_piece[p] = e % (D / 8);
      v_dim[p] = e / 8;
      v_key[p] = 8 * (e % 8);
    }
  }
  const size_t page_elems = static_cast<size_t>(n_kv) * page_size * D;
  // (tiled pages: the blocks are fetched in their order, so the column of the block table and
  // the place within the page are stepped along instead of divided out for every block)
  int pf_col = page_col(kb_lo * 64), pf_off = page_off(kb_lo * 64);
#define PF_LOAD(KB)                                                                                \
  if (TILED) {                                                                                      \
    const int page = pages_in_lds ? pages_s[pf_col - first_col] : max(0, bt[pf_col]);               \
    const size_t base = static_cast<size_t>(page) * page_elems + static_cast<size_t>(g) * page_size * D + \
                        static_cast<size_t>(pf_off) * D;                                            \
    _Pragma("unroll") for (int p = 0; p < PP; ++p) {                                                \
      kreg[p] = *reinterpret_cast<const u32x4_t*>(k_cache + base + 8 * (threadIdx.x + 256 * p));    \
      vreg[p] = *reinterpret_cast<const u32x4_t*>(v_cache + base + 8 * (threadIdx.x + 256 * p));    \
    }                                                                                               \
    pf_off += 64;                                                                                   \
    if (pf_off >= page_size) {                                                                      \
      pf_off = 0;                                                                                   \
      pf_col = min(pf_col + 1, last_page_col);                                                      \
    }                                                                                               \
  } else {                                                                                          \
    _Pragma("unroll") for (int p = 0; p < PP; ++p) {                                                \
      {                                                                                             \
        const int key = (KB) * 64 + k_key[p];                                                       \
        kreg[p] = *reinterpret_cast<const u32x4_t*>(                                                \
            k_cache + ((static_cast<size_t>(page_of(key)) * n_kv + g) * page_size + page_off(key)) * D + 8 * k_piece[p]); \
      }                                                                                             \
      {                                                                                             \
        const int key = (KB) * 64 + v_key[p];                                                       \
        vreg[p] = *reinterpret_cast<const u32x4_t*>(                                                \
            v_cache + ((static_cast<size_t>(page_of(key)) * n_kv + g) * D + v_dim[p]) * page_size + page_off(key)); \
      }                                                                                             \
    }                                                                                               \
  }

  if (kb_lo < kb_hi) { PF_LOAD(kb_lo) }
  for (int kb = kb_lo; kb < kb_hi; ++kb) {
    __syncthreads();  // every wave is done with the previous block
#pragma unroll
    for (int p = 0; p < PP; ++p) {
      {
        // key kappa = 32u + 8a + 4sb + c of the block is parked at row 32u + 16sb + 4a + c
        const int kappa = k_key[p];
        const int row = (kappa & 32) | ((kappa & 4) << 2) | ((kappa & 24) >> 1) | (kappa & 3);
        *reinterpret_cast<u32x4_t*>(&ks[row][8 * k_piece[p]]) = kreg[p];
      }
      {
        u32x4_t v = vreg[p];
        const int key = kb * 64 + v_key[p];
        if (key + 8 > hi || key < lo) {  // values of keys that do not exist yet, or below the window, may be anything
          AFrag8 f;
          f.u = v;
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (key + i >= hi || key + i < lo) f.h[i] = 0;
          v = f.u;
        }
        *reinterpret_cast<u32x4_t*>(&vs[v_dim[p]][v_key[p]]) = v;
      }
    }
    __syncthreads();
    if (kb + 1 < kb_hi) { PF_LOAD(kb + 1) }  // in flight while this block is worked on
    const int key0 = kb * 64;
    if (key0 >= wave_hi) continue;  // nothing of this block is visible to this wave

    f32x4_t s[CT][2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
        for (int c = 0; c < CT; ++c) s[c][u][sb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks_ = 0; ks_ < KS; ++ks_) {
          AFrag8 a;
          a.u = *reinterpret_cast<const u32x4_t*>(&ks[32 * u + 16 * sb + r][32 * ks_ + 8 * gq]);
#pragma unroll
          for (int c = 0; c < CT; ++c)
            s[c][u][sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[c][ks_].v, s[c][u][sb], 0, 0, 0);
        }
      }
    // keys that every column sees whole need no mask (columns that stand for nothing
    // compute on zeros and are never stored)
    const bool whole = key0 + 63 <= (tile_pos0 + wave_tok0) && (window == 0 || key0 >= max(0, wave_hi - window));
    AFrag8 pf[CT][2];
    float alpha[CT];
    bool grew = false;  // some column's maximum rose: only then the running sums need rescaling
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      // the maximum is taken over the raw scores (the scale is positive), and the scale
      // joins the subtraction of the maximum in one fused multiply-add
      if (!whole) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int sb = 0; sb < 2; ++sb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int key = key0 + 32 * u + 8 * gq + 4 * sb + i;
              const bool ok = col_ok[c] && key <= pos_c[c] && key >= lo_c[c];
              s[c][u][sb][i] = ok ? s[c][u][sb][i] : -INFINITY;
            }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
#pragma unroll
          for (int i = 0; i < 4; ++i) tmax = fmaxf(tmax, s[c][u][sb][i]);
      tmax = column_lanes_max(tmax);
      const float m_new = fmaxf(m[c], tmax * scale_log2);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      grew = grew || m_new > m[c];
      alpha[c] = fast_exp2(m[c] - m_safe);
      float psum = 0.f;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            s[c][u][sb][i] = fast_exp2(fmaf(s[c][u][sb][i], scale_log2, -m_safe));
            psum += s[c][u][sb][i];
          }
          pf[c][u].u[2 * sb] = pack_bf16x2(s[c][u][sb][0], s[c][u][sb][1]);
          pf[c][u].u[2 * sb + 1] = pack_bf16x2(s[c][u][sb][2], s[c][u][sb][3]);
        }
      l[c] = l[c] * alpha[c] + psum;
      m[c] = m_new;
    }
    if (__any(grew)) {
      asm volatile("" ::: "memory");  // (a branch, not a multiplication and a select per element)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int c = 0; c < CT; ++c) acc[c][dt] *= alpha[c];
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        AFrag8 a;
        a.u = *reinterpret_cast<const u32x4_t*>(&vs[16 * dt + r][32 * u + 8 * gq]);
#pragma unroll
        for (int c = 0; c < CT; ++c)
          acc[c][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pf[c][u].v, acc[c][dt], 0, 0, 0);
      }
    }
  }
#undef PF_LOAD
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    float lc = l[c];
    lc = column_lanes_sum(lc);
    if (n_splits > 1) {
      // partial result of this split, a group of 16 columns per wave (and column tile)
      const size_t group = (static_cast<size_t>(t) * 4 * CT + wave * CT + c) * n_y + by;
      const size_t widx = group * n_splits + blockIdx.y;
      float* wo = ws_o + (widx * 16 + r) * D + 4 * gq;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4_t*>(wo + 16 * dt) = acc[c][dt];
      if (gq == 0) {
        ws_ml[(widx * 16 + r) * 2] = m[c];
        ws_ml[(widx * 16 + r) * 2 + 1] = lc;
      }
      continue;
    }
    if (col_ok[c]) {
      const float inv = 1.f / lc;
      bf16_t* op = out + (static_cast<size_t>(tile_tok0 + tok_c[c]) * n_heads + h_base + hh) * D + 4 * gq;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        u32x2_t w;
        w[0] = pack_bf16x2(acc[c][dt][0] * inv, acc[c][dt][1] * inv);
        w[1] = pack_bf16x2(acc[c][dt][2] * inv, acc[c][dt][3] * inv);
        *reinterpret_cast<u32x2_t*>(op + 16 * dt) = w;
      }
    }
  }
}

// Merge the splits of every column: weights exp2(m_s - max m), in the order of s.
// A thread owns four consecutive output elements of one column.
// blockIdx.x names a group of 16 columns: a tile of the short-span kernel (parts == 1), or one
// wave's share of a long tile (parts == 4: group x is wave x % 4 of tile x / 4).
template <int D>
__global__ __launch_bounds__(256) void attn_combine_kernel(
    bf16_t* __restrict__ out, const int32_t* __restrict__ tiles, int n_heads, int n_kv, int hpt,
    int chunks, int n_splits, const float* __restrict__ ws_o, const float* __restrict__ ws_ml, int parts) {
  const int t = blockIdx.x / parts, part = blockIdx.x % parts;
  const int tpt_ = 16 / hpt;
  const int tok0 = tiles[4 * t + 1] + part * tpt_, ntok = tiles[4 * t + 2] - part * tpt_;
  const int g = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
  const int qpk = n_heads / n_kv;
  const int h_base = g * qpk + chunk * hpt;
  const int heads_here = min(hpt, qpk - chunk * hpt);
  const size_t w0 = (static_cast<size_t>(blockIdx.x) * gridDim.y + blockIdx.y) * n_splits;
  for (int e = threadIdx.x; e < 16 * (D / 4); e += blockDim.x) {
    const int c = e / (D / 4), d = (e % (D / 4)) * 4;
    const int tt = c / hpt, hh = c % hpt;
    // (a group of 16 columns holds tpt_ tokens; with a head count that does not divide 16 the
    // columns left over stand for nothing, not for the next part's first token)
    if (tt >= min(ntok, tpt_) || hh >= heads_here) continue;
    float merged[4];
    attn_merge_splits(ws_o, ws_ml, w0 * 16 + c, n_splits, D, d, merged);
    u32x2_t o;
    o[0] = pack_bf16x2(merged[0], merged[1]);
    o[1] = pack_bf16x2(merged[2], merged[3]);
    *reinterpret_cast<u32x2_t*>(out + (static_cast<size_t>(tok0 + tt) * n_heads + h_base + hh) * D + d) = o;
  }
}

extern "C" int yk_attn_mfma_supported(int head_dim) { return head_dim == 64 || head_dim == 128; }

// Heads of one kv head that share a wave, and tokens per tile, for a head layout.
extern "C" int yk_attn_heads_per_tile(int n_heads, int n_kv) { return attn_heads_per_tile(n_heads, n_kv); }
extern "C" int yk_attn_tokens_per_tile(int n_heads, int n_kv) {
  return 16 / yk_attn_heads_per_tile(n_heads, n_kv);
}
// Tokens of one long tile (a workgroup of the long-span kernel): four waves of col_tiles (1 or 2)
// column tiles.
extern "C" int yk_attn_long_tile_tokens(int n_heads, int n_kv, int col_tiles) {
  return 4 * col_tiles * yk_attn_tokens_per_tile(n_heads, n_kv);
}

// Floats of workspace for a launch with n_splits > 1: outputs, then (max, sum) pairs.
extern "C" size_t yk_attn_mfma_workspace(int n_tiles, int n_heads, int n_kv, int head_dim,
                                         int n_splits) {
  if (n_splits <= 1) return 0;
  const int hpt = yk_attn_heads_per_tile(n_heads, n_kv);
  const int chunks = (n_heads / n_kv + hpt - 1) / hpt;
  const size_t w = static_cast<size_t>(n_tiles) * n_kv * chunks * n_splits * 16;
  return w * head_dim + w * 2;
}

// Long spans: ``tiles`` hold up to yk_attn_long_tile_tokens tokens each (one workgroup a tile).
// pages_lds_limit: a workgroup keeps the page ids of the keys it walks in LDS when they are fewer
// than this (and than the kernel's own 2,048), else it looks each up in the block table.
extern "C" int yk_attn_mfma_prefill(const void* q, int q_stride, void* out, const void* k_cache,
                                    const void* v_cache, const int32_t* tiles, int n_tiles,
                                    const int32_t* block_table, int table_width, int page_size,
                                    int head_dim, int n_heads, int n_kv, float scale, int window,
                                    int n_splits, int col_tiles, float* workspace, size_t workspace_floats,
                                    int pages_lds_limit, hipStream_t stream) {
  YK_REQUIRE(n_tiles >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attn_mfma_prefill: bad head counts");
  YK_REQUIRE(col_tiles == 1 || col_tiles == 2, "attn_mfma_prefill: a wave has 1 or 2 column tiles");
  YK_REQUIRE(yk_attn_mfma_supported(head_dim), "attn_mfma_prefill: head_dim must be 64 or 128");
  YK_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_mfma_prefill: page_size must be a multiple of 16");
  YK_REQUIRE(q_stride % 8 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0,
             "attn_mfma_prefill: query rows must be 16-byte aligned");
  YK_REQUIRE(reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0,
             "attn_mfma_prefill: cache must be 16-byte aligned");
  YK_REQUIRE(window >= 0 && table_width > 0, "attn_mfma_prefill: bad window or table");
  YK_REQUIRE(scale > 0.f, "attn_mfma_prefill: the score scale must be positive");
  if (n_tiles == 0) return 0;
  const int hpt = yk_attn_heads_per_tile(n_heads, n_kv);
  const int chunks = (n_heads / n_kv + hpt - 1) / hpt;
  YK_REQUIRE(static_cast<long long>(n_tiles) * n_kv * chunks <= 0x7fffffffLL, "attn_mfma_prefill: too many tiles for one launch");
  YK_REQUIRE(n_splits >= 1 && n_splits <= 65535, "attn_mfma_prefill: bad split count");
  const size_t need = yk_attn_mfma_workspace(4 * col_tiles * n_tiles, n_heads, n_kv, head_dim, n_splits);
  YK_REQUIRE(workspace_floats >= need, "attn_mfma_prefill: workspace too small");
  float* ws_o = workspace;
  float* ws_ml = workspace ? workspace + (need / (head_dim + 2)) * head_dim : nullptr;
  const float scale_log2 = scale * 1.4426950408889634f;
  dim3 grid(n_tiles * n_kv * chunks, n_splits), block(256);
#define YK_PF_ARGS                                                                                           \
  static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_cache),     \
      static_cast<const bf16_t*>(v_cache), tiles, block_table, table_width, page_size, n_heads, n_kv, hpt,     \
      chunks, scale_log2, window, n_splits, ws_o, ws_ml, pages_lds_limit
#define YK_PF(DD, BIP)                                                                                       \
  if (col_tiles == 2)                                                                                        \
    attn_mfma_prefill_kernel<DD, BIP, 2><<<grid, block, 0, stream>>>(YK_PF_ARGS);                            \
  else                                                                                                       \
    attn_mfma_prefill_kernel<DD, BIP, 1><<<grid, block, 0, stream>>>(YK_PF_ARGS)
  const bool bip = cache_is_tiled(YK_BF16, head_dim, page_size);
  if (head_dim == 64) {
    if (bip) { YK_PF(64, true); } else { YK_PF(64, false); }
  } else {
    if (bip) { YK_PF(128, true); } else { YK_PF(128, false); }
  }
#undef YK_PF
#undef YK_PF_ARGS
  if (yk_check_launch("attn_mfma_prefill")) return -1;
  if (n_splits > 1) {
    dim3 cgrid(4 * col_tiles * n_tiles, n_kv * chunks);
    if (head_dim == 64)
      attn_combine_kernel<64><<<cgrid, 256, 0, stream>>>(static_cast<bf16_t*>(out), tiles, n_heads, n_kv, hpt, chunks, n_splits, ws_o, ws_ml, 4 * col_tiles);
    else
      attn_combine_kernel<128><<<cgrid, 256, 0, stream>>>(static_cast<bf16_t*>(out), tiles, n_heads, n_kv, hpt, chunks, n_splits, ws_o, ws_ml, 4 * col_tiles);
    return yk_check_launch("attn_combine");
  }
  return 0;
}

// Short spans (single tokens, short portions): tiles of up to yk_attn_tokens_per_tile tokens.
// leave_splits != 0 with n_splits > 1: the splits stay unmerged in the workspace (`out` is not
// written) for a consumer that merges them itself or for yk_attn_combine.
// rope: null, or where the launch makes its queries (and the tokens' keys and values) from.
static int launch_attn_mfma(const void* q, int q_stride, void* out, const void* k_cache, const void* v_cache,
                            const int32_t* tiles, int n_tiles, const int32_t* block_table, int table_width,
                            int page_size, int head_dim, int n_heads, int n_kv, float scale, int window,
                            int n_waves, int n_splits, float* workspace, size_t workspace_floats,
                            int leave_splits, const RopeSrc* rope, bool rope_f32, hipStream_t stream) {
  YK_REQUIRE(n_tiles >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attn_mfma: bad head counts");
  YK_REQUIRE(n_waves == 1 || n_waves == 4, "attn_mfma: a workgroup has 1 or 4 waves");
  YK_REQUIRE(yk_attn_mfma_supported(head_dim), "attn_mfma: head_dim must be 64 or 128");
  YK_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_mfma: page_size must be a multiple of 16");
  YK_REQUIRE(rope || (q_stride % 8 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0),
             "attn_mfma: query rows must be 16-byte aligned");
  YK_REQUIRE(reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0,
             "attn_mfma: cache must be 16-byte aligned");
  YK_REQUIRE(n_splits >= 1 && n_splits <= 65535, "attn_mfma: bad split count");
  YK_REQUIRE(window >= 0 && table_width > 0, "attn_mfma: bad window or table");
  YK_REQUIRE(scale > 0.f, "attn_mfma: the score scale must be positive");
  if (n_tiles == 0) return 0;
  const int hpt = yk_attn_heads_per_tile(n_heads, n_kv);
  const int chunks = (n_heads / n_kv + hpt - 1) / hpt;
  YK_REQUIRE(n_kv * chunks <= 65535, "attn_mfma: too many heads for one launch");
  const size_t need = yk_attn_mfma_workspace(n_tiles, n_heads, n_kv, head_dim, n_splits);
  YK_REQUIRE(workspace_floats >= need, "attn_mfma: workspace too small");
  float* ws_o = workspace;
  float* ws_ml = workspace ? workspace + (need / (head_dim + 2)) * head_dim : nullptr;
  const float scale_log2 = scale * 1.4426950408889634f;
  dim3 grid(n_tiles, n_kv * chunks, n_splits), block(64 * n_waves);
  const bool tiled = cache_is_tiled(YK_BF16, head_dim, page_size);
  const RopeSrc rs = rope ? *rope : RopeSrc{};
#define YK_ARGS                                                                                    \
      static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out),                          \
      static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), tiles, block_table, \
      table_width, page_size, n_heads, n_kv, hpt, chunks, scale_log2, window, n_splits, ws_o, ws_ml, rs
#define YK_LAUNCH_R(DD, RR)                                                                        \
  if (tiled) {                                                                                     \
    if (n_waves == 1) attn_mfma_kernel<DD, 1, true, RR><<<grid, block, 0, stream>>>(YK_ARGS);      \
    else attn_mfma_kernel<DD, 4, true, RR><<<grid, block, 0, stream>>>(YK_ARGS);                   \
  } else {                                                                                         \
    if (n_waves == 1) attn_mfma_kernel<DD, 1, false, RR><<<grid, block, 0, stream>>>(YK_ARGS);     \
    else attn_mfma_kernel<DD, 4, false, RR><<<grid, block, 0, stream>>>(YK_ARGS);                  \
  }
#define YK_LAUNCH(DD)                                                                              \
  if (!rope) { YK_LAUNCH_R(DD, 0) } else if (rope_f32) { YK_LAUNCH_R(DD, 2) } else { YK_LAUNCH_R(DD, 1) } \
  if (yk_check_launch("attn_mfma")) return -1;                                                     \
  if (n_splits > 1 && !leave_splits) {                                                             \
    attn_combine_kernel<DD><<<dim3(n_tiles, n_kv * chunks), 256, 0, stream>>>(                     \
        static_cast<bf16_t*>(out), tiles, n_heads, n_kv, hpt, chunks, n_splits, ws_o, ws_ml, 1);   \
    if (yk_check_launch("attn_combine")) return -1;                                                \
  }
  if (head_dim == 64) {
    YK_LAUNCH(64)
  } else {
    YK_LAUNCH(128)
  }
#undef YK_LAUNCH
#undef YK_LAUNCH_R
#undef YK_ARGS
  return 0;
}

extern "C" int yk_attn_mfma(const void* q, int q_stride, void* out, const void* k_cache,
                            const void* v_cache, const int32_t* tiles, int n_tiles,
                            const int32_t* block_table, int table_width, int page_size,
                            int head_dim, int n_heads, int n_kv, float scale, int window,
                            int n_waves, int n_splits, float* workspace, size_t workspace_floats,
                            int leave_splits, hipStream_t stream) {
  return launch_attn_mfma(q, q_stride, out, k_cache, v_cache, tiles, n_tiles, block_table, table_width, page_size,
                          head_dim, n_heads, n_kv, scale, window, n_waves, n_splits, workspace, workspace_floats,
                          leave_splits, nullptr, false, stream);
}

// yk_attn_mfma for a step of single tokens (every tile holds ONE token), with rotary + append
// inside the launch: `src` holds the projection's output rows [n_heads query heads | n_kv key
// heads | n_kv value heads] (src_dtype bfloat16 with n_src_splits == 1, or float32 with the
// product's unreduced K slices [n_src_splits][tokens][src_stride], whose sum is rounded to
// bfloat16 when round_sum).  The queries are rotated as yk_rope_append rotates them; with
// append != 0 the tokens' rotated keys and their values are used by the launch and stored in
// the pages (k_cache, v_cache are written), with append == 0 the rows hold queries only and
// the pages already have the tokens' keys and values.
extern "C" int yk_attn_mfma_rope(const void* src, int src_dtype, int n_src_splits, int round_sum, int src_stride,
                                 int n_tokens, const float* cos_t, const float* sin_t, int rotary_dim,
                                 int interleaved, int max_positions, int append, void* out, void* k_cache,
                                 void* v_cache, const int32_t* tiles, int n_tiles, const int32_t* block_table,
                                 int table_width, int page_size, int head_dim, int n_heads, int n_kv, float scale,
                                 int window, int n_waves, int n_splits, float* workspace, size_t workspace_floats,
                                 int leave_splits, hipStream_t stream) {
  YK_REQUIRE(src && (src_dtype == YK_F32 || src_dtype == YK_BF16), "attn_mfma_rope: the rows must be float32 or bfloat16");
  YK_REQUIRE(n_src_splits >= 1 && (n_src_splits == 1 || src_dtype == YK_F32), "attn_mfma_rope: unreduced slices must be float32");
  YK_REQUIRE(n_tokens >= n_tiles && n_tiles >= 0, "attn_mfma_rope: one tile a token");
  YK_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
             "attn_mfma_rope: rotary_dim must be even and at most head_dim");
  YK_REQUIRE(rotary_dim == 0 || (cos_t && sin_t && max_positions > 0), "attn_mfma_rope: missing table");
  YK_REQUIRE(n_heads > 0 && n_kv > 0 && src_stride >= (n_heads + (append ? 2 * n_kv : 0)) * head_dim,
             "attn_mfma_rope: row stride too small");
  RopeSrc rs;
  rs.src = src;
  rs.n_splits = n_src_splits;
  rs.split_stride = static_cast<size_t>(n_tokens) * src_stride;
  rs.round_sum = round_sum;
  rs.src_stride = src_stride;
  rs.cos_t = rotary_dim ? cos_t : nullptr;
  rs.sin_t = rotary_dim ? sin_t : nullptr;
  rs.rotary_dim = rotary_dim;
  rs.interleaved = interleaved;
  rs.max_positions = rotary_dim ? max_positions : 1;
  rs.append = append != 0;
  return launch_attn_mfma(nullptr, 0, out, k_cache, v_cache, tiles, n_tiles, block_table, table_width, page_size,
                          head_dim, n_heads, n_kv, scale, window, n_waves, n_splits, workspace, workspace_floats,
                          leave_splits, &rs, src_dtype == YK_F32, stream);
}

// The second half of yk_attn_mfma for a launch that was told to leave its splits in the
// workspace (leave_splits): merges them into `out`.  Same arguments as that launch had.
extern "C" int yk_attn_combine(void* out, const int32_t* tiles, int n_tiles, int head_dim, int n_heads,
                               int n_kv, int n_splits, const float* workspace, size_t workspace_floats,
                               hipStream_t stream) {
  YK_REQUIRE(n_tiles >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attn_combine: bad head counts");
  YK_REQUIRE(yk_attn_mfma_supported(head_dim), "attn_combine: head_dim must be 64 or 128");
  YK_REQUIRE(n_splits > 1 && n_splits <= 65535, "attn_combine: nothing to merge");
  if (n_tiles == 0) return 0;
  const int hpt = attn_heads_per_tile(n_heads, n_kv);
  const int chunks = (n_heads / n_kv + hpt - 1) / hpt;
  const size_t need = yk_attn_mfma_workspace(n_tiles, n_heads, n_kv, head_dim, n_splits);
  YK_REQUIRE(workspace && workspace_floats >= need, "attn_combine: workspace too small");
  const float* ws_o = workspace;
  const float* ws_ml = workspace + (need / (head_dim + 2)) * head_dim;
  const dim3 grid(n_tiles, n_kv * chunks);
  if (head_dim == 64)
    attn_combine_kernel<64><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), tiles, n_heads, n_kv, hpt, chunks, n_splits, ws_o, ws_ml, 1);
  else
    attn_combine_kernel<128><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), tiles, n_heads, n_kv, hpt, chunks, n_splits, ws_o, ws_ml, 1);
  return yk_check_launch("attn_combine");
}
