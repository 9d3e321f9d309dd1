// Memory-bound kernels of a step: embedding gather, fused residual add + RMS norm,
// rotary position encoding fused with the append of keys and values to the paged
// cache, and the gated activation of the feed-forward.
//
// Reference arithmetic: RMS norm yalis/external/model.py:979-986; rotary
// yalis/external/model.py:894-909 with the table of :786-820; cache append
// yalis/attention/utils/flash_utils.py:34-43,64-89; silu(gate) * up
// yalis/external/model.py:741-743.  Everything is computed in float32 and rounded once.
#include <algorithm>

#include "common.h"

// Whether the pages of such a cache are stored tiled (cache_is_tiled).
extern "C" int yk_cache_tiled(int dtype, int head_dim, int page_size) { return cache_is_tiled(dtype, head_dim, page_size) ? 1 : 0; }

// ------------------------------------------------------------------------- embedding
// out[n, :] = float(table[ids[n], :])
template <typename T>
__global__ void embed_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ out, int width, int vocab) {
  const int n = blockIdx.x;
  int id = ids[n];
  // ids are checked on the host; clamp so that a bad id cannot read out of bounds
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + static_cast<size_t>(id) * width;
  float* dst = out + static_cast<size_t>(n) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = to_f32<T>(src[c]);
}

// eight elements per thread, no loop (bfloat16 tables whose width is a multiple of 8)
__global__ void embed_bf16x8_kernel(const int32_t* __restrict__ ids, const bf16_t* __restrict__ table,
                                    float* __restrict__ out, int width, int vocab, size_t total_vec) {
  const size_t v = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
  if (v >= total_vec) return;
  const int per_row = width / 8;
  const size_t n = v / per_row;
  const int c = static_cast<int>(v % per_row) * 8;
  int id = ids[n];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const uint4 raw = *reinterpret_cast<const uint4*>(table + static_cast<size_t>(id) * width + c);
  const uint32_t wds[4] = {raw.x, raw.y, raw.z, raw.w};
  float4 lo, hi;
  lo.x = __uint_as_float(wds[0] << 16);
  lo.y = __uint_as_float(wds[0] & 0xffff0000u);
  lo.z = __uint_as_float(wds[1] << 16);
  lo.w = __uint_as_float(wds[1] & 0xffff0000u);
  hi.x = __uint_as_float(wds[2] << 16);
  hi.y = __uint_as_float(wds[2] & 0xffff0000u);
  hi.z = __uint_as_float(wds[3] << 16);
  hi.w = __uint_as_float(wds[3] & 0xffff0000u);
  float* dst = out + n * width + c;
  *reinterpret_cast<float4*>(dst) = lo;
  *reinterpret_cast<float4*>(dst + 4) = hi;
}

extern "C" int yk_embed(const int32_t* ids, const void* table, int table_dtype, float* out,
                        int n_tokens, int width, int vocab, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && width > 0 && vocab > 0, "embed: bad sizes");
  if (n_tokens == 0) return 0;
  if (table_dtype == YK_BF16 && width % 8 == 0 && reinterpret_cast<uintptr_t>(table) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const size_t total_vec = static_cast<size_t>(n_tokens) * (width / 8);
    embed_bf16x8_kernel<<<static_cast<unsigned>((total_vec + 255) / 256), 256, 0, stream>>>(
        ids, static_cast<const bf16_t*>(table), out, width, vocab, total_vec);
    return yk_check_launch("embed");
  }
  dim3 grid(n_tokens), block(256);
  if (table_dtype == YK_F32)
    embed_kernel<float><<<grid, block, 0, stream>>>(ids, static_cast<const float*>(table), out, width, vocab);
  else if (table_dtype == YK_BF16)
    embed_kernel<bf16_t><<<grid, block, 0, stream>>>(ids, static_cast<const bf16_t*>(table), out, width, vocab);
  else
    return yk_fail("embed: unsupported table dtype");
  return yk_check_launch("embed");
}

// ---------------------------------------------------------------- four-wide accessors
template <typename T>
__device__ __forceinline__ float4 load4(const T* p);
template <>
__device__ __forceinline__ float4 load4<float>(const float* p) {
  return *reinterpret_cast<const float4*>(p);
}
template <>
__device__ __forceinline__ float4 load4<bf16_t>(const bf16_t* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  float4 v;
  v.x = __uint_as_float(raw.x << 16);
  v.y = __uint_as_float(raw.x & 0xffff0000u);
  v.z = __uint_as_float(raw.y << 16);
  v.w = __uint_as_float(raw.y & 0xffff0000u);
  return v;
}
template <typename T>
__device__ __forceinline__ void store4(T* p, float4 v);
template <>
__device__ __forceinline__ void store4<float>(float* p, float4 v) {
  *reinterpret_cast<float4*>(p) = v;
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float4 v) {
  uint2 raw;
  raw.x = pack_bf16x2(v.x, v.y);
  raw.y = pack_bf16x2(v.z, v.w);
  *reinterpret_cast<uint2*>(p) = raw;
}

// (as_output, in common.h: the sum of a product's K slices is rounded as the product's
// output would have been)

// the row of an embedding table that token `src` of the step names (ids are checked on the
// host; clamped here so that a bad id cannot read out of bounds)
__device__ __forceinline__ size_t table_row(const int32_t* __restrict__ ids, size_t src, int table_rows) {
  const int id = ids[src];
  return static_cast<size_t>(id < 0 ? 0 : (id >= table_rows ? table_rows - 1 : id));
}

// ------------------------------------------------------------- residual add + RMS norm
// For row r (source row rows[r] when rows is given):
//   v = residual[src] + sum over s of delta[s][src]   (float32; delta may be absent;
//       n_splits > 1: delta holds the unreduced K slices of a product, float32)
//   residual[src] = v                                  (only when rows is null)
//   out[r] = v * rsqrt(mean(v^2) + eps) * (weight [+ 1])
// Without a residual (null) v is the delta alone and nothing is written back: the plain norm
// of rows that are no residual stream (a branch's output, queries, keys).
// With table_ids the residual stream starts here: `delta` is an embedding table, v =
// table[table_ids[src]] (the residual is not read, and written as in the plain form).
// General form: any width, two passes over the row.
template <typename TD, typename TW, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                   int n_splits, size_t split_stride, int round_sum,
                                   const int32_t* __restrict__ rows, const TW* __restrict__ weight,
                                   TO* __restrict__ out, int width, float eps, int unit_offset,
                                   const int32_t* __restrict__ table_ids, int table_rows) {
  __shared__ float scratch[17];
  const int r = blockIdx.x;
  const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* res = residual ? residual + src * width : nullptr;
  const bool fresh = table_ids != nullptr || res == nullptr;  // nothing is read from a residual
  const TD* del = delta ? delta + (table_ids ? table_row(table_ids, src, table_rows) : src) * width : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = fresh ? 0.f : res[c];
    if (del) {
      float d = 0.f;
      for (int s = 0; s < n_splits; ++s) d += to_f32<TD>(del[s * split_stride + c]);
      v += as_output(d, round_sum);
      if (!rows && res) res[c] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(width) + eps);
  TO* o = out + static_cast<size_t>(r) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = res ? res[c] : 0.f;
    if (del && (rows || !res)) {  // not written back in the gathered form, nor without a residual
      float d = 0.f;
      for (int s = 0; s < n_splits; ++s) d += to_f32<TD>(del[s * split_stride + c]);
      v += as_output(d, round_sum);
    }
    float w = to_f32<TW>(weight[c]);
    if (unit_offset) w += 1.f;
    o[c] = from_f32<TO>(v * inv * w);
  }
}

// Fast form: width a multiple of 4 and at most 4 * NORM_IT * blockDim; the row stays in
// registers, every load of a thread is issued before the first use.  NORM_IT (four-wide
// pieces per thread) is chosen by the launcher as small as the width allows.
constexpr int NORM_IT_MAX = 8;
template <typename TD, typename TW, typename TO, int NORM_IT>
__global__ __launch_bounds__(1024) void add_rmsnorm_vec_kernel(
    float* __restrict__ residual, const TD* __restrict__ delta, int n_splits, size_t split_stride,
    int round_sum, const int32_t* __restrict__ rows, const TW* __restrict__ weight, TO* __restrict__ out,
    int width, float eps, int unit_offset, const int32_t* __restrict__ table_ids, int table_rows) {
  __shared__ float scratch[17];
  const int r = blockIdx.x;
  const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* res = residual ? residual + src * width : nullptr;
  const bool fresh = table_ids != nullptr || res == nullptr;  // nothing is read from a residual
  const TD* del = delta ? delta + (table_ids ? table_row(table_ids, src, table_rows) : src) * width : nullptr;
  float4 v[NORM_IT], w[NORM_IT], ds[NORM_IT];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NORM_IT; ++it) {
    const int c = (threadIdx.x + it * blockDim.x) * 4;
    if (c < width) {
      v[it] = fresh ? make_float4(0.f, 0.f, 0.f, 0.f) : load4<float>(res + c);
      w[it] = load4<TW>(weight + c);
    }
  }
  if (del) {
    // SL slices at a time (eight where a thread has one piece of the row: a product's eight
    // slices then cost one wait for memory, not two), all loads issued before the first
    // sum; a slice index beyond the last is clamped and its value dropped, so that the
    // loads carry no condition
    constexpr int SL = NORM_IT == 1 ? 8 : 4;
#pragma unroll
    for (int it = 0; it < NORM_IT; ++it) ds[it] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < n_splits; s0 += SL) {
#pragma unroll
      for (int it = 0; it < NORM_IT; ++it) {
        const int c = (threadIdx.x + it * blockDim.x) * 4;
        if (c < width) {
          float4 d[SL];
#pragma unroll
          for (int j = 0; j < SL; ++j) d[j] = load4<TD>(del + static_cast<size_t>(min(s0 + j, n_splits - 1)) * split_stride + c);
#pragma unroll
          for (int j = 0; j < SL; ++j) {
            if (s0 + j < n_splits) {
              ds[it].x += d[j].x;
              ds[it].y += d[j].y;
              ds[it].z += d[j].z;
              ds[it].w += d[j].w;
            }
          }
        }
      }
    }
#pragma unroll
    for (int it = 0; it < NORM_IT; ++it) {
      v[it].x += as_output(ds[it].x, round_sum);
      v[it].y += as_output(ds[it].y, round_sum);
      v[it].z += as_output(ds[it].z, round_sum);
      v[it].w += as_output(ds[it].w, round_sum);
    }
  }
#pragma unroll
  for (int it = 0; it < NORM_IT; ++it) {
    const int c = (threadIdx.x + it * blockDim.x) * 4;
    if (c < width) {
      if (del && !rows && res) store4<float>(res + c, v[it]);
      ss += v[it].x * v[it].x + v[it].y * v[it].y + v[it].z * v[it].z + v[it].w * v[it].w;
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(width) + eps);
  const float off = unit_offset ? 1.f : 0.f;
  TO* o = out + static_cast<size_t>(r) * width;
#pragma unroll
  for (int it = 0; it < NORM_IT; ++it) {
    const int c = (threadIdx.x + it * blockDim.x) * 4;
    if (c < width) {
      float4 y;
      y.x = v[it].x * inv * (w[it].x + off);
      y.y = v[it].y * inv * (w[it].y + off);
      y.z = v[it].z * inv * (w[it].z + off);
      y.w = v[it].w * inv * (w[it].w + off);
      store4<TO>(o + c, y);
    }
  }
}

template <typename TD, typename TW, typename TO>
static int launch_add_rmsnorm(float* residual, const void* delta, int n_splits, size_t split_stride,
                              int round_sum, const int32_t* rows, const void* weight, void* out, int n_rows,
                              int width, float eps, int unit_offset, const int32_t* table_ids, int table_rows,
                              hipStream_t stream) {
  const bool aligned = width % 4 == 0 && reinterpret_cast<uintptr_t>(residual) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(delta) % 16 == 0 && reinterpret_cast<uintptr_t>(weight) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(out) % 16 == 0 && split_stride % 4 == 0;
  if (aligned && width <= 4 * NORM_IT_MAX * 512) {
    // one four-wide chunk per thread where the row allows (faster than two at 8 rows), at most
    // 1,024 threads; with rows enough to fill the GPU several times over, two chunks per thread:
    // twice the rows are in flight on a compute unit and a row's sum meets half the waves
    // (2,048 rows of 4,096: 21.6 -> 18.4 us; of 3,072: 18.2 -> 14.2; 8,192 of 4,096: 68.9 -> 62.6)
    int threads = ((n_rows >= 1024 ? width / 8 : width / 4) + 63) / 64 * 64;
    threads = std::max(64, std::min(threads, 1024));
    const int pieces = (width / 4 + threads - 1) / threads;
#define YK_NORM(IT)                                                                           \
    add_rmsnorm_vec_kernel<TD, TW, TO, IT><<<n_rows, threads, 0, stream>>>(                   \
        residual, static_cast<const TD*>(delta), n_splits, split_stride, round_sum, rows,     \
        static_cast<const TW*>(weight), static_cast<TO*>(out), width, eps, unit_offset, table_ids, table_rows)
    if (pieces <= 1) YK_NORM(1);
    else if (pieces <= 2) YK_NORM(2);
    else if (pieces <= 4) YK_NORM(4);
    else YK_NORM(8);
#undef YK_NORM
  } else {
    add_rmsnorm_kernel<TD, TW, TO><<<n_rows, width >= 2048 ? 512 : 256, 0, stream>>>(
        residual, static_cast<const TD*>(delta), n_splits, split_stride, round_sum, rows,
        static_cast<const TW*>(weight), static_cast<TO*>(out), width, eps, unit_offset, table_ids, table_rows);
  }
  return yk_check_launch("add_rmsnorm");
}

// delta may be null (then delta_dtype is ignored); rows may be null.  n_splits > 1 needs
// float32 delta laid out [n_splits][rows of the residual][width]; round_sum: the slices' sum
// is rounded to bfloat16 before it is added.  table_ids (null, or one id per residual row):
// delta is an embedding table of table_rows rows and the residual starts as its rows
// table_ids[.] (n_splits 1, no rows).
extern "C" int yk_add_rmsnorm(float* residual, const void* delta, int delta_dtype, int n_splits,
                              int round_sum, const int32_t* rows, const void* weight, int weight_dtype, void* out,
                              int out_dtype, int n_rows, int n_residual_rows, int width, float eps,
                              int unit_offset, const int32_t* table_ids, int table_rows, hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && width > 0 && n_residual_rows >= 0, "add_rmsnorm: bad sizes");
  YK_REQUIRE(residual || (delta && !table_ids), "add_rmsnorm: without a residual there must be rows to normalise");
  YK_REQUIRE(!table_ids || (delta && n_splits == 1 && !rows && table_rows > 0 && !round_sum),
             "add_rmsnorm: an embedding table comes whole, with one id per row of the residual");
  YK_REQUIRE(eps >= 0.f, "add_rmsnorm: eps must not be negative");
  YK_REQUIRE(n_splits >= 1, "add_rmsnorm: bad split count");
  YK_REQUIRE(n_splits == 1 || delta_dtype == YK_F32, "add_rmsnorm: unreduced slices must be float32");
  if (n_rows == 0) return 0;
  if (!delta) {
    delta_dtype = YK_F32;
    n_splits = 1;
  }
  const size_t stride = static_cast<size_t>(n_residual_rows) * width;
#define YK_CASE(DD, TD, WD, TW, OD, TO)                                  \
  if (delta_dtype == DD && weight_dtype == WD && out_dtype == OD)        \
    return launch_add_rmsnorm<TD, TW, TO>(residual, delta, n_splits, stride, round_sum, rows, weight, out, n_rows, width, eps, unit_offset, table_ids, table_rows, stream);
  YK_CASE(YK_F32, float, YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("add_rmsnorm: unsupported dtype combination");
}

// -------------------------------------------------- rotary + append to the paged cache
// One workgroup per (token, head).  The token's row of `src` holds n_heads query heads,
// then n_kv key heads, then n_kv value heads, each of head_dim elements; with n_splits > 1
// `src` holds the unreduced float32 K slices of the projection and they are summed here.
// Query heads are rotated into `q_out` (which may be `src` itself); key heads are rotated
// and stored at the token's slot of the key pages [page][kv_head][page_size x head_dim];
// value heads are stored in the value pages [page][kv_head][head_dim x page_size] (within a
// slab plain or tiled: cache_k_offset, cache_v_offset).
// n_kv may be 0 (rotate queries only).  Rotation of a pair (a, b) by the angle of
// (position, pair index i): a' = a cos - b sin, b' = b cos + a sin; pairs are
// (i, i + rotary_dim/2) ("half") or (2i, 2i + 1) ("interleaved"); elements beyond
// rotary_dim pass unchanged.
// (rot_first, rot_second: common.h)

template <typename TS, typename T>
__global__ void rope_append_kernel(const TS* src, int n_splits, size_t split_stride, int round_sum,
                                   int src_stride, T* q_out, int q_stride, int n_heads,
                                   int n_kv, int head_dim, const int32_t* __restrict__ positions,
                                   const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                   int rotary_dim, int interleaved, int max_positions,
                                   T* __restrict__ k_cache, T* __restrict__ v_cache,
                                   const int32_t* __restrict__ slots, int page_size) {
  const int n = blockIdx.x, h = blockIdx.y;
  int pos = positions[n];
  pos = pos < 0 ? 0 : (pos >= max_positions ? max_positions - 1 : pos);
  const int half = rotary_dim / 2;
  const float* cs = cos_t ? cos_t + static_cast<size_t>(pos) * half : nullptr;
  const float* sn = sin_t ? sin_t + static_cast<size_t>(pos) * half : nullptr;
  const TS* row = src + static_cast<size_t>(n) * src_stride;
  // Two elements at once (a rotary pair, or two value elements): up to eight slices of both
  // are in flight before the first is added; a slice index beyond the last is clamped and
  // its value dropped, so that the loads carry no condition.  Slices are added in order.
  auto value2 = [&](int idx_a, int idx_b, float& out_a, float& out_b) {
    float a = 0.f, b = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
      float da[8], db[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const size_t off = static_cast<size_t>(min(s0 + j, n_splits - 1)) * split_stride;
        da[j] = to_f32<TS>(row[off + idx_a]);
        db[j] = to_f32<TS>(row[off + idx_b]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (s0 + j < n_splits) {
          a += da[j];
          b += db[j];
        }
    }
    out_a = as_output(a, round_sum);
    out_b = as_output(b, round_sum);
  };
  auto value = [&](int idx) {
    float a, b;
    value2(idx, idx, a, b);
    return a;
  };
  const bool is_q = h < n_heads;
  const bool tiled = cache_is_tiled(sizeof(T) == 2 ? YK_BF16 : YK_F32, head_dim, page_size);
  const size_t slab = static_cast<size_t>(page_size) * head_dim;
  T* dst;   // the query row, or the key slab of the token's page
  int off = 0;  // the token's slot within its page
  if (is_q) {
    dst = q_out + static_cast<size_t>(n) * q_stride + static_cast<size_t>(h) * head_dim;
  } else {
    const int slot = slots[n];
    const size_t page = static_cast<size_t>(slot / page_size);
    off = slot % page_size;
    const int g = h - n_heads;
    dst = k_cache + (page * n_kv + g) * slab;
    // the value head of the same group
    T* vdst = v_cache + (page * n_kv + g) * slab;
    const int vbase = (n_heads + n_kv + g) * head_dim;
    for (int d = threadIdx.x; d < head_dim; d += 2 * blockDim.x) {
      const int d2 = d + blockDim.x;  // this thread's second element, when there is one
      float va, vb;
      value2(vbase + d, vbase + min(d2, head_dim - 1), va, vb);
      vdst[cache_v_offset(tiled, page_size, head_dim, off, d)] = from_f32<T>(va);
      if (d2 < head_dim) vdst[cache_v_offset(tiled, page_size, head_dim, off, d2)] = from_f32<T>(vb);
    }
  }
  auto put = [&](int d, float v) {
    dst[is_q ? static_cast<size_t>(d) : cache_k_offset(tiled, page_size, head_dim, off, d)] = from_f32<T>(v);
  };
  const int base = h * head_dim;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const int ia = interleaved ? 2 * i : i;
    const int ib = interleaved ? 2 * i + 1 : i + half;
    float a, b;
    value2(base + ia, base + ib, a, b);
    const float c = cs[i], s = sn[i];
    put(ia, rot_first(a, b, c, s));
    put(ib, rot_second(a, b, c, s));
  }
  for (int d = rotary_dim + threadIdx.x; d < head_dim; d += blockDim.x) put(d, value(base + d));
}

// The same for many tokens of plain bfloat16 rows with "half" pairs: a workgroup takes
// ROPE_TOK consecutive tokens of one head and moves 16 bytes per access.  Value heads
// (blockIdx.y beyond the query and key heads) gather the tokens' elements of one value row
// and, where the tokens' slots are consecutive and start at a multiple of ROPE_TOK (a
// prompt portion that starts on such a boundary), store them as one 16-byte piece of the
// transposed page instead of ROPE_TOK separate elements.
constexpr int ROPE_TOK = 8;

__device__ __forceinline__ void rope_rotate8(const uint4& a, const uint4& b, const float* __restrict__ c,
                                             const float* __restrict__ s, uint4& oa, uint4& ob) {
  const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
  uint32_t ra[4], rb[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float a0 = __uint_as_float(aw[j] << 16), a1 = __uint_as_float(aw[j] & 0xffff0000u);
    const float b0 = __uint_as_float(bw[j] << 16), b1 = __uint_as_float(bw[j] & 0xffff0000u);
    const float c0 = c[2 * j], c1 = c[2 * j + 1], s0 = s[2 * j], s1 = s[2 * j + 1];
    ra[j] = pack_bf16x2(rot_first(a0, b0, c0, s0), rot_first(a1, b1, c1, s1));
    rb[j] = pack_bf16x2(rot_second(a0, b0, c0, s0), rot_second(a1, b1, c1, s1));
  }
  oa = make_uint4(ra[0], ra[1], ra[2], ra[3]);
  ob = make_uint4(rb[0], rb[1], rb[2], rb[3]);
}

__global__ __launch_bounds__(64) void rope_append_vec_kernel(
    const bf16_t* src, int src_stride, bf16_t* q_out, int q_stride, int n_tokens, int n_heads,
    int n_kv, int head_dim, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int rotary_dim, int max_positions, bf16_t* __restrict__ k_cache,
    bf16_t* __restrict__ v_cache, const int32_t* __restrict__ slots, int page_size) {
  const int n0 = blockIdx.x * ROPE_TOK, h = blockIdx.y;
  const int n_here = min(ROPE_TOK, n_tokens - n0);
  const int half = rotary_dim / 2;
  const bool tiled = cache_is_tiled(YK_BF16, head_dim, page_size);
  const size_t slab = static_cast<size_t>(page_size) * head_dim;
  if (h >= n_heads + n_kv) {
    // value head g of these tokens, transposed into the pages
    const int g = h - n_heads - n_kv;
    const int vbase = (n_heads + n_kv + g) * head_dim;
    const int slot0 = slots[n0];
    bool together = n_here == ROPE_TOK && slot0 % ROPE_TOK == 0;
    for (int t = 1; t < n_here; ++t) together = together && slots[n0 + t] == slot0 + t;
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
      bf16_t v[ROPE_TOK];
#pragma unroll
      for (int t = 0; t < ROPE_TOK; ++t)
        v[t] = src[static_cast<size_t>(n0 + min(t, n_here - 1)) * src_stride + vbase + d];
      if (together) {
        const size_t page = static_cast<size_t>(slot0 / page_size);
        bf16_t* vdst = v_cache + (page * n_kv + g) * slab + cache_v_offset(tiled, page_size, head_dim, slot0 % page_size, d);
        uint4 w;
        w.x = v[0] | (static_cast<uint32_t>(v[1]) << 16);
        w.y = v[2] | (static_cast<uint32_t>(v[3]) << 16);
        w.z = v[4] | (static_cast<uint32_t>(v[5]) << 16);
        w.w = v[6] | (static_cast<uint32_t>(v[7]) << 16);
        *reinterpret_cast<uint4*>(vdst) = w;
      } else {
        for (int t = 0; t < n_here; ++t) {
          const int slot = slots[n0 + t];
          const size_t page = static_cast<size_t>(slot / page_size);
          v_cache[(page * n_kv + g) * slab + cache_v_offset(tiled, page_size, head_dim, slot % page_size, d)] = v[t];
        }
      }
    }
    return;
  }
  const bool is_q = h < n_heads;
  const int pieces = half / 8;                      // rotated pairs of 16-byte pieces per head
  const int tail = (head_dim - rotary_dim) / 8;     // pieces beyond the rotated part
  const int per_tok = pieces + tail;
  for (int item = threadIdx.x; item < n_here * per_tok; item += blockDim.x) {
    const int t = item / per_tok, pc = item % per_tok;
    const int n = n0 + t;
    const bf16_t* row = src + static_cast<size_t>(n) * src_stride + static_cast<size_t>(h) * head_dim;
    bf16_t* dst;  // the query row, or the key slab of the token's page
    int off = 0;
    if (is_q) {
      dst = q_out + static_cast<size_t>(n) * q_stride + static_cast<size_t>(h) * head_dim;
    } else {
      const int slot = slots[n];
      const size_t page = static_cast<size_t>(slot / page_size);
      off = slot % page_size;
      dst = k_cache + (page * n_kv + (h - n_heads)) * slab;
    }
    // where the 8 elements from d on go (they stay together in either layout)
    auto at = [&](int d) { return dst + (is_q ? static_cast<size_t>(d) : cache_k_offset(tiled, page_size, head_dim, off, d)); };
    if (pc < pieces) {
      int pos = positions[n];
      pos = pos < 0 ? 0 : (pos >= max_positions ? max_positions - 1 : pos);
      const float* cs = cos_t + static_cast<size_t>(pos) * half + 8 * pc;
      const float* sn = sin_t + static_cast<size_t>(pos) * half + 8 * pc;
      const uint4 a = *reinterpret_cast<const uint4*>(row + 8 * pc);
      const uint4 b = *reinterpret_cast<const uint4*>(row + half + 8 * pc);
      float c[8], s_[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        c[j] = cs[j];
        s_[j] = sn[j];
      }
      uint4 oa, ob;
      rope_rotate8(a, b, c, s_, oa, ob);
      *reinterpret_cast<uint4*>(at(8 * pc)) = oa;
      *reinterpret_cast<uint4*>(at(half + 8 * pc)) = ob;
    } else {
      const int d = rotary_dim + 8 * (pc - pieces);
      *reinterpret_cast<uint4*>(at(d)) = *reinterpret_cast<const uint4*>(row + d);
    }
  }
}

// src_dtype/n_splits describe `src`; act_dtype is the dtype of q_out and of the cache.
extern "C" int yk_rope_append(const void* src, int src_dtype, int n_splits, int round_sum, int src_stride,
                              void* q_out, int act_dtype, int q_stride, int n_tokens, int n_heads,
                              int n_kv, int head_dim, const int32_t* positions, const float* cos_t,
                              const float* sin_t, int rotary_dim, int interleaved,
                              int max_positions, void* k_cache, void* v_cache,
                              const int32_t* slots, int page_size, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads >= 0 && n_kv >= 0 && head_dim > 0, "rope_append: bad sizes");
  YK_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
             "rope_append: rotary_dim must be even and at most head_dim");
  YK_REQUIRE(src_stride >= (n_heads + 2 * n_kv) * head_dim, "rope_append: row stride too small");
  YK_REQUIRE(q_stride >= n_heads * head_dim, "rope_append: query row stride too small");
  YK_REQUIRE(rotary_dim == 0 || (cos_t && sin_t && max_positions > 0), "rope_append: missing table");
  YK_REQUIRE(n_kv == 0 || (k_cache && v_cache && slots && page_size > 0), "rope_append: missing cache");
  YK_REQUIRE(n_splits >= 1 && (n_splits == 1 || src_dtype == YK_F32), "rope_append: unreduced slices must be float32");
  YK_REQUIRE(n_heads + n_kv <= 65535, "rope_append: too many heads for one launch");
  if (n_tokens == 0 || n_heads + n_kv == 0) return 0;
  const auto aligned16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (src_dtype == YK_BF16 && act_dtype == YK_BF16 && n_splits == 1 && !interleaved && n_tokens >= 4 * ROPE_TOK &&
      rotary_dim % 16 == 0 && head_dim % 8 == 0 && src_stride % 8 == 0 && q_stride % 8 == 0 && page_size % ROPE_TOK == 0 &&
      aligned16(src) && aligned16(q_out) && (n_kv == 0 || (aligned16(k_cache) && aligned16(v_cache))) &&
      (rotary_dim == 0 || (aligned16(cos_t) && aligned16(sin_t))) && n_heads + 2 * n_kv <= 65535) {
    dim3 vgrid((n_tokens + ROPE_TOK - 1) / ROPE_TOK, n_heads + 2 * n_kv);
    rope_append_vec_kernel<<<vgrid, 64, 0, stream>>>(
        static_cast<const bf16_t*>(src), src_stride, static_cast<bf16_t*>(q_out), q_stride, n_tokens, n_heads, n_kv,
        head_dim, positions, cos_t, sin_t, rotary_dim, max_positions, static_cast<bf16_t*>(k_cache),
        static_cast<bf16_t*>(v_cache), slots, page_size);
    return yk_check_launch("rope_append_vec");
  }
  dim3 grid(n_tokens, n_heads + n_kv), block(head_dim <= 128 ? 64 : 128);
  const size_t stride = static_cast<size_t>(n_tokens) * src_stride;
#define YK_CASE(SD, TS, AD, T)                                                                          \
  if (src_dtype == SD && act_dtype == AD) {                                                             \
    rope_append_kernel<TS, T><<<grid, block, 0, stream>>>(                                              \
        static_cast<const TS*>(src), n_splits, stride, round_sum, src_stride, static_cast<T*>(q_out), q_stride, \
        n_heads, n_kv, head_dim, positions, cos_t, sin_t, rotary_dim, interleaved, max_positions,       \
        static_cast<T*>(k_cache), static_cast<T*>(v_cache), slots, page_size);                          \
    return yk_check_launch("rope_append");                                                              \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("rope_append: unsupported dtype combination");
}

// ------------------------------------------------------------------ gated activation
// out[n, j] = act(gate[n, j]) * up[n, j]; act 0 = silu, 1 = gelu (tanh form).  The columns
// of gu are [gate | up] (group 0) or alternate in groups: `group` gate columns, then the
// `group` up columns that belong to them, and so on (the layout the fused product uses).
// With n_splits > 1, gu holds unreduced float32 K slices [n_splits][rows][2 * inter].
__device__ __forceinline__ size_t gate_col(size_t j, int inter, int group) {
  return group ? (j / group) * 2 * group + j % group : j;
}
__device__ __forceinline__ size_t up_offset(int inter, int group) { return group ? group : inter; }


template <typename TS, typename TO>
__global__ void gated_act_kernel(const TS* __restrict__ gu, int n_splits, size_t split_stride, int round_sum,
                                 TO* __restrict__ out, int inter, size_t total, int act, int group) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t n = i / inter, j = i % inter;
    float g = 0.f, u = 0.f;
    const size_t gc = n * 2 * inter + gate_col(j, inter, group);
    for (int s = 0; s < n_splits; ++s) {
      g += to_f32<TS>(gu[s * split_stride + gc]);
      u += to_f32<TS>(gu[s * split_stride + gc + up_offset(inter, group)]);
    }
    g = as_output(g, round_sum);
    u = as_output(u, round_sum);
    out[i] = from_f32<TO>(act_apply(g, act) * u);
  }
}

// four outputs per thread, no loop (inter a multiple of 4)
template <typename TS, typename TO>
__global__ void gated_act_vec_kernel(const TS* __restrict__ gu, int n_splits, size_t split_stride, int round_sum,
                                     TO* __restrict__ out, int inter, size_t total_vec, int act, int group) {
  const size_t v = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
  if (v >= total_vec) return;
  const int per_row = inter / 4;
  const size_t n = v / per_row;
  const int j = static_cast<int>(v % per_row) * 4;
  const TS* p = gu + n * 2 * inter + gate_col(j, inter, group);  // four columns of one group (group % 4 == 0)
  const size_t up = up_offset(inter, group);
  float4 g = load4<TS>(p), u = load4<TS>(p + up);
  for (int s0 = 1; s0 < n_splits; s0 += 2) {  // two slices in flight
    const int s1 = min(s0 + 1, n_splits - 1);
    const float4 g2 = load4<TS>(p + s0 * split_stride), u2 = load4<TS>(p + s0 * split_stride + up);
    const float4 g3 = load4<TS>(p + s1 * split_stride), u3 = load4<TS>(p + s1 * split_stride + up);
    g.x += g2.x; g.y += g2.y; g.z += g2.z; g.w += g2.w;
    u.x += u2.x; u.y += u2.y; u.z += u2.z; u.w += u2.w;
    if (s0 + 1 < n_splits) {
      g.x += g3.x; g.y += g3.y; g.z += g3.z; g.w += g3.w;
      u.x += u3.x; u.y += u3.y; u.z += u3.z; u.w += u3.w;
    }
  }
  float4 y;
  y.x = act_apply(as_output(g.x, round_sum), act) * as_output(u.x, round_sum);
  y.y = act_apply(as_output(g.y, round_sum), act) * as_output(u.y, round_sum);
  y.z = act_apply(as_output(g.z, round_sum), act) * as_output(u.z, round_sum);
  y.w = act_apply(as_output(g.w, round_sum), act) * as_output(u.w, round_sum);
  store4<TO>(out + n * inter + j, y);
}

// bfloat16 in and out, one slice, eight outputs per thread with 16-byte accesses (in the
// grouped layout a thread's gate and up values are 32 contiguous bytes)
__global__ void gated_act_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int inter,
                                        size_t total_vec, int act, int group) {
  const size_t v = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
  if (v >= total_vec) return;
  const int per_row = inter / 8;
  const size_t n = v / per_row;
  const int j = static_cast<int>(v % per_row) * 8;
  const bf16_t* p = gu + n * 2 * inter + gate_col(j, inter, group);
  const uint4 g = *reinterpret_cast<const uint4*>(p);
  const uint4 u = *reinterpret_cast<const uint4*>(p + up_offset(inter, group));
  const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
  uint32_t o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
    o[k] = pack_bf16x2(act_apply(g0, act) * u0, act_apply(g1, act) * u1);
  }
  *reinterpret_cast<uint4*>(out + n * inter + j) = make_uint4(o[0], o[1], o[2], o[3]);
}

template <typename TS, typename TO>
static int launch_gated_act(const void* gu, int n_splits, int round_sum, void* out, int n_rows, int inter, int act,
                            int group, hipStream_t stream) {
  const size_t stride = static_cast<size_t>(n_rows) * 2 * inter;
  const bool aligned = inter % 4 == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (aligned && sizeof(TS) == 2 && sizeof(TO) == 2 && n_splits == 1 && inter % 8 == 0 && group % 8 == 0) {
    const size_t total_vec = static_cast<size_t>(n_rows) * (inter / 8);
    YK_REQUIRE((total_vec + 255) / 256 < (1ull << 31), "gated_act: too large for one launch");
    gated_act_bf16x8_kernel<<<static_cast<unsigned>((total_vec + 255) / 256), 256, 0, stream>>>(
        static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), inter, total_vec, act, group);
  } else if (aligned) {
    const size_t total_vec = static_cast<size_t>(n_rows) * (inter / 4);
    YK_REQUIRE((total_vec + 255) / 256 < (1ull << 31), "gated_act: too large for one launch");
    gated_act_vec_kernel<TS, TO><<<static_cast<unsigned>((total_vec + 255) / 256), 256, 0, stream>>>(
        static_cast<const TS*>(gu), n_splits, stride, round_sum, static_cast<TO*>(out), inter, total_vec, act, group);
  } else {
    const size_t total = static_cast<size_t>(n_rows) * inter;
    const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 65535));
    gated_act_kernel<TS, TO><<<grid, 256, 0, stream>>>(static_cast<const TS*>(gu), n_splits, stride, round_sum,
                                                        static_cast<TO*>(out), inter, total, act, group);
  }
  return yk_check_launch("gated_act");
}

extern "C" int yk_gated_act(const void* gu, int src_dtype, int n_splits, int round_sum, void* out, int out_dtype,
                            int n_rows, int inter, int act, int group, hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && inter > 0, "gated_act: bad sizes");
  YK_REQUIRE(group == 0 || (group % 4 == 0 && inter % group == 0), "gated_act: groups are multiples of 4 that divide the width");
  YK_REQUIRE(act == 0 || act == 1, "gated_act: unknown activation");
  YK_REQUIRE(n_splits >= 1 && (n_splits == 1 || src_dtype == YK_F32), "gated_act: unreduced slices must be float32");
  if (n_rows == 0) return 0;
  if (src_dtype == YK_F32 && out_dtype == YK_F32) return launch_gated_act<float, float>(gu, n_splits, round_sum, out, n_rows, inter, act, group, stream);
  if (src_dtype == YK_F32 && out_dtype == YK_BF16) return launch_gated_act<float, bf16_t>(gu, n_splits, round_sum, out, n_rows, inter, act, group, stream);
  if (src_dtype == YK_BF16 && out_dtype == YK_BF16) return launch_gated_act<bf16_t, bf16_t>(gu, n_splits, round_sum, out, n_rows, inter, act, group, stream);
  return yk_fail("gated_act: unsupported dtype combination");
}

// ------------------------------------------------------------------------------- bias
// y[m, :] = src[m, :] + bias, the sum in float32 and rounded once to y's dtype (src may be y
// itself).  A projection with a bias takes its product in float32 and comes here, so that the
// result is rounded once, as a product that adds the bias to its accumulators would round it
// (the reference's biased Linear does: yalis/external/model.py:449, torch's addmm).  Llama has no
// biases; parts offer them as an option, and this is all that option costs the kernel library.
template <typename TS, typename TY, typename TB>
__global__ void add_bias_kernel(const TS* __restrict__ src, int lds, TY* __restrict__ y, const TB* __restrict__ bias,
                                size_t total, int cols, int ldy) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t m = i / cols;
    const int n = static_cast<int>(i % cols);
    y[m * ldy + n] = from_f32<TY>(to_f32<TS>(src[m * lds + n]) + to_f32<TB>(bias[n]));
  }
}

extern "C" int yk_add_bias(const void* src, int src_dtype, int lds, void* y, int y_dtype, int ldy, const void* bias,
                           int bias_dtype, int rows, int cols, hipStream_t stream) {
  YK_REQUIRE(rows >= 0 && cols > 0 && ldy >= cols && lds >= cols, "add_bias: bad sizes");
  YK_REQUIRE(src != y || (src_dtype == y_dtype && lds == ldy), "add_bias: in place needs one dtype and one stride");
  if (rows == 0) return 0;
  const size_t total = static_cast<size_t>(rows) * cols;
  const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 65535));
#define YK_CASE(SD, TS, YD, TY, BD, TB)                                                      \
  if (src_dtype == SD && y_dtype == YD && bias_dtype == BD) {                               \
    add_bias_kernel<TS, TY, TB><<<grid, 256, 0, stream>>>(static_cast<const TS*>(src), lds, static_cast<TY*>(y), \
                                                          static_cast<const TB*>(bias), total, cols, ldy);       \
    return yk_check_launch("add_bias");                                                     \
  }
  YK_CASE(YK_F32, float, YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("add_bias: unsupported dtype combination");
}
