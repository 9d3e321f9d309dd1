// Shared helpers of the HIP kernels: bfloat16 storage, wave and block reductions,
// error reporting of the C interface.
//
// Conventions of the library: every entry point is extern "C", takes raw device
// pointers and sizes plus the stream to launch on, checks its arguments on the host
// (a size a kernel cannot take is refused with a message, never computed wrongly),
// returns 0 on success and a negative number on failure; yk_last_error() returns the
// message.  dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#define YK_F32 0
#define YK_BF16 1

typedef uint16_t bf16_t;  // bfloat16 storage

std::string& yk_error_slot();
int yk_fail(const std::string& msg);
int yk_check_launch(const char* what);

#define YK_REQUIRE(cond, msg)        \
  do {                               \
    if (!(cond)) return yk_fail(msg); \
  } while (0)

__device__ __forceinline__ float bf16_to_f32(bf16_t x) {
  return __uint_as_float(static_cast<uint32_t>(x) << 16);
}

// Over the four lanes r, r + 16, r + 32 and r + 48 (the lanes that share a column of a 16 x 16
// matrix-core tile): the maximum, or the sum, in all four of them.  The swaps of half-waves and
// of rows of 16 lanes move registers directly; a shuffle would go through the LDS pipe and
// wait on its counter together with the operand reads.
__device__ __forceinline__ float column_lanes_max(float v) {
  const auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float column_lanes_sum(float v) {
  const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// two floats to two bfloat16 (round to nearest even; NaN stays NaN) in one word: gfx950
// converts in hardware (v_cvt_pk_bf16_f32), one instruction where the shifts and adds of a
// conversion by hand take six (measured: 2 us of a 41 us product that converted its staged rows)
typedef __bf16 yk_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float yk_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  union {
    yk_bf16x2_t v;
    uint32_t u;
  } c;
  c.v = __builtin_convertvector(yk_f32x2_t{lo, hi}, yk_bf16x2_t);
  return c.u;
}

__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return static_cast<bf16_t>(pack_bf16x2(f, 0.f) & 0xffffu); }

template <typename T>
__device__ __forceinline__ float to_f32(T x);
template <>
__device__ __forceinline__ float to_f32<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ float to_f32<bf16_t>(bf16_t x) {
  return bf16_to_f32(x);
}

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) {
  return f32_to_bf16(x);
}

constexpr int kWave = 64;

// ------------------------------------------------------------------ layout of a cache page
// A page holds, for every kv head, a slab of page_size x head_dim keys and one of values.
// Plain slabs: keys [slot][dim], values transposed [dim][slot].
// Tiled slabs (bfloat16, a head size the matrix-core attention takes, pages of a multiple of
// 64 tokens): the slab is cut into blocks of 64 slots, and a block is stored as the 16-byte
// pieces that the matrix-core attention loads, in the order of the lanes that load them, so
// that one wave-wide load reads 1 KiB of consecutive memory:
//   keys:   piece (((u*2 + sb) * head_dim/32 + ks) * 4 + g) * 16 + r holds dims 32ks + 8g .. 8g+7
//           of slot 32u + 8(r/4) + 4sb + r%4 (the row order of the two score products of a
//           group of 32 keys),
//   values: piece ((u * head_dim/16 + dt) * 4 + g) * 16 + r holds slots 32u + 8g .. 8g+7 of dim
//           16dt + r.
// Writers (rotary + append) and readers (the attention kernels) go through these functions.
__host__ __device__ inline bool cache_is_tiled(int dtype, int head_dim, int page_size) {
  return dtype == YK_BF16 && (head_dim == 64 || head_dim == 128) && page_size % 64 == 0;
}
// element offsets within a slab
__host__ __device__ inline size_t cache_k_offset(bool tiled, int page_size, int head_dim, int slot, int d) {
  if (!tiled) return static_cast<size_t>(slot) * head_dim + d;
  const int j = slot % 64, u = j / 32, r = 4 * ((j % 32) / 8) + j % 4, sb = (j % 8) / 4;
  const int piece = (((u * 2 + sb) * (head_dim / 32) + d / 32) * 4 + (d % 32) / 8) * 16 + r;
  return static_cast<size_t>(slot / 64) * 64 * head_dim + piece * 8 + d % 8;
}
__host__ __device__ inline size_t cache_v_offset(bool tiled, int page_size, int head_dim, int slot, int d) {
  if (!tiled) return static_cast<size_t>(d) * page_size + slot;
  const int j = slot % 64, u = j / 32, g = (j % 32) / 8;
  const int piece = ((u * (head_dim / 16) + d / 16) * 4 + g) * 16 + d % 16;
  return static_cast<size_t>(slot / 64) * 64 * head_dim + piece * 8 + j % 8;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` is shared memory for 17 floats.
// Gated activations: 0 = silu, 1 = gelu (tanh form); float32.
__device__ __forceinline__ float act_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float act_gelu_tanh(float z) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  return 0.5f * z * (1.f + tanhf(k * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float act_apply(float z, int act) { return act == 0 ? act_silu(z) : act_gelu_tanh(z); }

// The sum of a product's K slices (or an accumulator) stands for the product's output: with
// `round_sum` it is rounded to bfloat16 as that output would have been, so that what follows
// does not depend on whether the product came reduced (bfloat16), as slices, or fused.
__device__ __forceinline__ float as_output(float v, int round_sum) {
  return round_sum ? to_f32<bf16_t>(from_f32<bf16_t>(v)) : v;
}

// Rotation of a pair (a, b) by the angle with cosine c and sine s: a' = a c - b s, b' = b c + a s.
// One rounding of b*s (or a*s), then a fused multiply-add: written out so that every kernel
// that rotates (rotary + append on its own, or inside the attention launch) gives the same bits.
__device__ __forceinline__ float rot_first(float a, float b, float c, float s) { return fmaf(a, c, -__fmul_rn(b, s)); }
__device__ __forceinline__ float rot_second(float a, float b, float c, float s) { return fmaf(b, c, __fmul_rn(a, s)); }

// ------------------------------------------------ attention whose keys were split across workgroups
// Heads of one kv head that share a wave of the matrix-core attention (its 16 columns hold
// 16 / heads_per_tile tokens of those heads); a kv group with more heads takes several
// chunks of them.
__host__ __device__ inline int attn_heads_per_tile(int n_heads, int n_kv) {
  const int qpk = n_heads / n_kv;
  return qpk < 16 ? qpk : 16;
}

// What the splits of a launch leave behind: for every group of 16 columns and split, the
// unnormalised outputs [16][head_dim] in `o` and (running maximum, sum) pairs [16][2] in `ml`,
// groups numbered (tile * groups_y + kv head * chunks + chunk) * n_splits + split.
// Four consecutive output elements of one column, merged over its splits: weights
// exp2(m_s - max m), in the order of s.  `col0` is the column's index in split 0
// (group * 16 + column); split s lies 16 columns further each.
__device__ __forceinline__ void attn_merge_splits(const float* __restrict__ o, const float* __restrict__ ml,
                                                  size_t col0, int n_splits, int head_dim, int d,
                                                  float out[4]) {
  const float* mlc = ml + col0 * 2;
  float m_max = -INFINITY;
#pragma unroll 4
  for (int s = 0; s < n_splits; ++s) m_max = fmaxf(m_max, mlc[static_cast<size_t>(s) * 32]);
  float num[4] = {0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
#pragma unroll 4
  for (int s = 0; s < n_splits; ++s) {
    const float w = exp2f(mlc[static_cast<size_t>(s) * 32] - m_max);
    const float4 v = *reinterpret_cast<const float4*>(o + (col0 + static_cast<size_t>(s) * 16) * head_dim + d);
    num[0] += w * v.x;
    num[1] += w * v.y;
    num[2] += w * v.z;
    num[3] += w * v.w;
    den += w * mlc[static_cast<size_t>(s) * 32 + 1];
  }
  const float inv = 1.f / den;
#pragma unroll
  for (int e = 0; e < 4; ++e) out[e] = num[e] * inv;
}

__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nwaves ? scratch[lane] : 0.f;
    t = wave_sum(t);
    if (lane == 0) scratch[16] = t;
  }
  __syncthreads();
  return scratch[16];
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nwaves ? scratch[lane] : -INFINITY;
    t = wave_max(t);
    if (lane == 0) scratch[16] = t;
  }
  __syncthreads();
  return scratch[16];
}
