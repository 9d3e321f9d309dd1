// Memory-bound kernels of a step: embedding gather, fused residual add + RMS norm,
// rotary position encoding fused with the append of keys and values to the paged
// cache, and the gated activation of the feed-forward.
//
// Reference arithmetic: RMS norm yalis/external/model.py:979-986; rotary
// yalis/external/model.py:894-909 with the table of :786-820; cache append
// yalis/attention/utils/flash_utils.py:34-43,64-89; silu(gate) * up
// yalis/external/model.py:741-743.  Everything is computed in float32 and rounded once.
#include "common.h"

// ------------------------------------------------------------------ error reporting
std::string& yk_error_slot() {
  static thread_local std::string s;
  return s;
}
int yk_fail(const std::string& msg) {
  yk_error_slot() = msg;
  return -1;
}
int yk_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return yk_fail(std::string(what) + ": " + hipGetErrorString(e));
  return 0;
}
extern "C" const char* yk_last_error() { return yk_error_slot().c_str(); }
extern "C" int yk_abi_version() { return 1; }

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

extern "C" int yk_embed(const int32_t* ids, const void* table, int table_dtype, float* out,
                        int n_tokens, int width, int vocab, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && width > 0 && vocab > 0, "embed: bad sizes");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens), block(256);
  if (table_dtype == YK_F32)
    embed_kernel<float><<<grid, block, 0, stream>>>(ids, static_cast<const float*>(table), out, width, vocab);
  else if (table_dtype == YK_BF16)
    embed_kernel<bf16_t><<<grid, block, 0, stream>>>(ids, static_cast<const bf16_t*>(table), out, width, vocab);
  else
    return yk_fail("embed: unsupported table dtype");
  return yk_check_launch("embed");
}

// ------------------------------------------------------------- residual add + RMS norm
// For row r (source row rows[r] when rows is given):
//   v = residual[src] + delta[src]           (float32; delta may be absent)
//   residual[src] = v                        (only when rows is null)
//   out[r] = v * rsqrt(mean(v^2) + eps) * (weight [+ 1])
template <typename TD, typename TW, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                   const int32_t* __restrict__ rows, const TW* __restrict__ weight,
                                   TO* __restrict__ out, int width, float eps, int unit_offset) {
  __shared__ float scratch[17];
  const int r = blockIdx.x;
  const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* res = residual + src * width;
  const TD* del = delta ? delta + src * width : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = res[c];
    if (del) {
      v += to_f32<TD>(del[c]);
      if (!rows) res[c] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(width) + eps);
  TO* o = out + static_cast<size_t>(r) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = res[c];
    if (del && rows) v += to_f32<TD>(del[c]);  // not written back in the gathered form
    float w = to_f32<TW>(weight[c]);
    if (unit_offset) w += 1.f;
    o[c] = from_f32<TO>(v * inv * w);
  }
}

template <typename TD, typename TW>
static int launch_add_rmsnorm_o(float* residual, const void* delta, const int32_t* rows,
                                const void* weight, void* out, int out_dtype, int n_rows, int width,
                                float eps, int unit_offset, hipStream_t stream) {
  dim3 grid(n_rows), block(width >= 2048 ? 512 : 256);
  if (out_dtype == YK_F32)
    add_rmsnorm_kernel<TD, TW, float><<<grid, block, 0, stream>>>(
        residual, static_cast<const TD*>(delta), rows, static_cast<const TW*>(weight),
        static_cast<float*>(out), width, eps, unit_offset);
  else if (out_dtype == YK_BF16)
    add_rmsnorm_kernel<TD, TW, bf16_t><<<grid, block, 0, stream>>>(
        residual, static_cast<const TD*>(delta), rows, static_cast<const TW*>(weight),
        static_cast<bf16_t*>(out), width, eps, unit_offset);
  else
    return yk_fail("add_rmsnorm: unsupported output dtype");
  return yk_check_launch("add_rmsnorm");
}

// delta may be null (then delta_dtype is ignored); rows may be null.
extern "C" int yk_add_rmsnorm(float* residual, const void* delta, int delta_dtype,
                              const int32_t* rows, const void* weight, int weight_dtype, void* out,
                              int out_dtype, int n_rows, int width, float eps, int unit_offset,
                              hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && width > 0, "add_rmsnorm: bad sizes");
  YK_REQUIRE(eps >= 0.f, "add_rmsnorm: eps must not be negative");
  if (n_rows == 0) return 0;
  if (!delta) delta_dtype = YK_F32;
#define YK_CASE(DD, TD, WD, TW)                        \
  if (delta_dtype == DD && weight_dtype == WD)         \
    return launch_add_rmsnorm_o<TD, TW>(residual, delta, rows, weight, out, out_dtype, n_rows, width, eps, unit_offset, stream);
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("add_rmsnorm: unsupported dtype combination");
}

// -------------------------------------------------- rotary + append to the paged cache
// One block per token.  The token's row of `qkv` holds n_heads query heads, then
// n_kv key heads, then n_kv value heads, each of head_dim elements.  Query heads are
// rotated in place; key heads are rotated and stored at the token's slot of the key
// pages [page][kv_head][page_size][head_dim]; value heads are stored transposed in the
// value pages [page][kv_head][head_dim][page_size].  n_kv may be 0 (rotate queries only).
// Rotation of a pair (a, b) by the angle of (position, pair index i):
//   a' = a cos - b sin, b' = b cos + a sin; pairs are (i, i + rotary_dim/2) ("half")
//   or (2i, 2i + 1) ("interleaved"); elements beyond rotary_dim pass unchanged.
template <typename T>
__global__ void rope_append_kernel(T* __restrict__ qkv, int row_stride, int n_heads, int n_kv,
                                   int head_dim, const int32_t* __restrict__ positions,
                                   const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                   int rotary_dim, int interleaved, int max_positions,
                                   T* __restrict__ k_cache, T* __restrict__ v_cache,
                                   const int32_t* __restrict__ slots, int page_size) {
  const int n = blockIdx.x;
  T* row = qkv + static_cast<size_t>(n) * row_stride;
  int pos = positions[n];
  pos = pos < 0 ? 0 : (pos >= max_positions ? max_positions - 1 : pos);
  const int half = rotary_dim / 2;
  const float* cs = cos_t ? cos_t + static_cast<size_t>(pos) * half : nullptr;
  const float* sn = sin_t ? sin_t + static_cast<size_t>(pos) * half : nullptr;
  size_t page = 0;
  int off = 0;
  if (n_kv > 0) {
    const int slot = slots[n];
    page = static_cast<size_t>(slot / page_size);
    off = slot % page_size;
  }
  const size_t page_elems = static_cast<size_t>(n_kv) * page_size * head_dim;

  // rotated pairs of the query and key heads
  const int rot_heads = n_heads + n_kv;
  for (int w = threadIdx.x; w < rot_heads * half; w += blockDim.x) {
    const int h = w / half, i = w % half;
    const int ia = interleaved ? 2 * i : i;
    const int ib = interleaved ? 2 * i + 1 : i + half;
    T* head = row + static_cast<size_t>(h) * head_dim;
    const float a = to_f32<T>(head[ia]), b = to_f32<T>(head[ib]);
    const float c = cs[i], s = sn[i];
    const T ra = from_f32<T>(a * c - b * s);
    const T rb = from_f32<T>(b * c + a * s);
    if (h < n_heads) {
      head[ia] = ra;
      head[ib] = rb;
    } else {
      const int g = h - n_heads;
      T* dst = k_cache + page * page_elems + (static_cast<size_t>(g) * page_size + off) * head_dim;
      dst[ia] = ra;
      dst[ib] = rb;
    }
  }
  // key elements that do not rotate
  const int rest = head_dim - rotary_dim;
  for (int w = threadIdx.x; w < n_kv * rest; w += blockDim.x) {
    const int g = w / rest, d = rotary_dim + w % rest;
    const T* head = row + static_cast<size_t>(n_heads + g) * head_dim;
    k_cache[page * page_elems + (static_cast<size_t>(g) * page_size + off) * head_dim + d] = head[d];
  }
  // values, transposed
  for (int w = threadIdx.x; w < n_kv * head_dim; w += blockDim.x) {
    const int g = w / head_dim, d = w % head_dim;
    const T* head = row + static_cast<size_t>(n_heads + n_kv + g) * head_dim;
    v_cache[page * page_elems + (static_cast<size_t>(g) * head_dim + d) * page_size + off] = head[d];
  }
}

extern "C" int yk_rope_append(void* qkv, int dtype, int n_tokens, int row_stride, int n_heads,
                              int n_kv, int head_dim, const int32_t* positions, const float* cos_t,
                              const float* sin_t, int rotary_dim, int interleaved,
                              int max_positions, void* k_cache, void* v_cache,
                              const int32_t* slots, int page_size, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads >= 0 && n_kv >= 0 && head_dim > 0, "rope_append: bad sizes");
  YK_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
             "rope_append: rotary_dim must be even and at most head_dim");
  YK_REQUIRE(row_stride >= (n_heads + 2 * n_kv) * head_dim, "rope_append: row stride too small");
  YK_REQUIRE(rotary_dim == 0 || (cos_t && sin_t && max_positions > 0), "rope_append: missing table");
  YK_REQUIRE(n_kv == 0 || (k_cache && v_cache && slots && page_size > 0), "rope_append: missing cache");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens), block(256);
  if (dtype == YK_F32)
    rope_append_kernel<float><<<grid, block, 0, stream>>>(
        static_cast<float*>(qkv), row_stride, n_heads, n_kv, head_dim, positions, cos_t, sin_t,
        rotary_dim, interleaved, max_positions, static_cast<float*>(k_cache),
        static_cast<float*>(v_cache), slots, page_size);
  else if (dtype == YK_BF16)
    rope_append_kernel<bf16_t><<<grid, block, 0, stream>>>(
        static_cast<bf16_t*>(qkv), row_stride, n_heads, n_kv, head_dim, positions, cos_t, sin_t,
        rotary_dim, interleaved, max_positions, static_cast<bf16_t*>(k_cache),
        static_cast<bf16_t*>(v_cache), slots, page_size);
  else
    return yk_fail("rope_append: unsupported dtype");
  return yk_check_launch("rope_append");
}

// ------------------------------------------------------------------ gated activation
// out[n, j] = act(gu[n, j]) * gu[n, inter + j]; act 0 = silu, 1 = gelu (tanh form)
__device__ __forceinline__ float act_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float act_gelu_tanh(float z) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  return 0.5f * z * (1.f + tanhf(k * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter,
                                 size_t total, int act) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t n = i / inter, j = i % inter;
    const float g = to_f32<T>(gu[n * 2 * inter + j]);
    const float u = to_f32<T>(gu[n * 2 * inter + inter + j]);
    const float a = act == 0 ? act_silu(g) : act_gelu_tanh(g);
    out[i] = from_f32<T>(a * u);
  }
}

extern "C" int yk_gated_act(const void* gu, void* out, int dtype, int n_rows, int inter, int act,
                            hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && inter > 0, "gated_act: bad sizes");
  YK_REQUIRE(act == 0 || act == 1, "gated_act: unknown activation");
  if (n_rows == 0) return 0;
  const size_t total = static_cast<size_t>(n_rows) * inter;
  const int block = 256;
  const int grid = static_cast<int>(std::min<size_t>((total + block - 1) / block, 65535));
  if (dtype == YK_F32)
    gated_act_kernel<float><<<grid, block, 0, stream>>>(static_cast<const float*>(gu),
                                                         static_cast<float*>(out), inter, total, act);
  else if (dtype == YK_BF16)
    gated_act_kernel<bf16_t><<<grid, block, 0, stream>>>(static_cast<const bf16_t*>(gu),
                                                          static_cast<bf16_t*>(out), inter, total, act);
  else
    return yk_fail("gated_act: unsupported dtype");
  return yk_check_launch("gated_act");
}
