// Choosing the next token from float32 logits, one workgroup per row.
//
// Order of operations (reference: yalis/external/sampling.py:41-74): keep the top_k
// largest logits; divide by the temperature; keep the smallest set of most likely tokens
// whose cumulative probability does not exceed top_p (the most likely token is always
// kept; the token that crosses the threshold is dropped, :16-38); softmax in float32;
// draw by the exponential race argmax(p_i / e_i) with e_i = -log(u_i) (:5-13, the form
// the reference uses under compilation).  temperature == 0 selects the largest logit
// (lowest index on ties).
//
// The uniforms are a documented function of (seed, draw, token index) so that a plain
// implementation can reproduce a draw:
//   z = mix64(mix64(seed * 2^32 + draw) + i);  u = ((z >> 41) + 0.5) / 2^23
// with mix64 the splitmix64 finaliser (add 0x9E3779B97F4A7C15, two xor-shift-multiply
// rounds, a last xor-shift).
//
// Thresholds (the k-th largest logit, the probability mass limit) are found by
// bisection over the order-preserving integer image of the floats, 32 counting passes
// over the row, without sorting.
#include <algorithm>

#include "common.h"

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// monotone map float -> uint32 (larger float, larger key)
__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct ArgMax {
  float v;
  int i;
};

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  // larger value wins; on equal values the lower index; NaN never wins
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ ArgMax block_argmax(ArgMax x, ArgMax* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax y;
    y.v = __shfl_xor(x.v, o, 64);
    y.i = __shfl_xor(x.i, o, 64);
    x = better(x, y);
  }
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int nwaves = (blockDim.x + 63) / 64;
  __syncthreads();
  if (lane == 0) scratch[wave] = x;
  __syncthreads();
  if (wave == 0) {
    ArgMax y = lane < nwaves ? scratch[lane] : ArgMax{-INFINITY, 0x7fffffff};
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      ArgMax z;
      z.v = __shfl_xor(y.v, o, 64);
      z.i = __shfl_xor(y.i, o, 64);
      y = better(y, z);
    }
    if (lane == 0) scratch[16] = y;
  }
  __syncthreads();
  return scratch[16];
}

__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits,
                                                      int32_t* __restrict__ out, int vocab) {
  __shared__ ArgMax scratch[17];
  const float* row = logits + static_cast<size_t>(blockIdx.x) * vocab;
  ArgMax best{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) best = better(best, ArgMax{row[i], i});
  best = block_argmax(best, scratch);
  if (threadIdx.x == 0) out[blockIdx.x] = best.i == 0x7fffffff ? 0 : best.i;
}

// Large vocabularies, few rows: first the best of each of ARGMAX_CHUNKS slices of the
// row, then the best of those (the lowest index still wins ties: slices are in order).
constexpr int ARGMAX_CHUNKS = 32;

__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ logits,
                                                          float* __restrict__ part_v,
                                                          int32_t* __restrict__ part_i, int vocab) {
  __shared__ ArgMax scratch[17];
  const float* row = logits + static_cast<size_t>(blockIdx.x) * vocab;
  const int per = (vocab + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
  const int lo = blockIdx.y * per, hi = min(vocab, lo + per);
  ArgMax best{-INFINITY, 0x7fffffff};
  for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) best = better(best, ArgMax{row[i], i});
  best = block_argmax(best, scratch);
  if (threadIdx.x == 0) {
    part_v[blockIdx.x * ARGMAX_CHUNKS + blockIdx.y] = best.v;
    part_i[blockIdx.x * ARGMAX_CHUNKS + blockIdx.y] = best.i;
  }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ part_v,
                                                          const int32_t* __restrict__ part_i,
                                                          int32_t* __restrict__ out) {
  const int lane = threadIdx.x;
  ArgMax x = lane < ARGMAX_CHUNKS ? ArgMax{part_v[blockIdx.x * ARGMAX_CHUNKS + lane], part_i[blockIdx.x * ARGMAX_CHUNKS + lane]}
                                  : ArgMax{-INFINITY, 0x7fffffff};
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax y;
    y.v = __shfl_xor(x.v, o, 64);
    y.i = __shfl_xor(x.i, o, 64);
    x = better(x, y);
  }
  if (lane == 0) out[blockIdx.x] = x.i == 0x7fffffff ? 0 : x.i;
}

// workspace: n_rows * 32 floats and as many ints (may be null for small vocabularies)
extern "C" int yk_argmax(const float* logits, int32_t* out, int n_rows, int vocab,
                         float* workspace, size_t workspace_floats, hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && vocab > 0, "argmax: bad sizes");
  if (n_rows == 0) return 0;
  const size_t need = static_cast<size_t>(n_rows) * ARGMAX_CHUNKS * 2;
  if (vocab >= 8192 && workspace && workspace_floats >= need && n_rows <= 65535) {
    float* pv = workspace;
    int32_t* pi = reinterpret_cast<int32_t*>(workspace + static_cast<size_t>(n_rows) * ARGMAX_CHUNKS);
    argmax_part_kernel<<<dim3(n_rows, ARGMAX_CHUNKS), 256, 0, stream>>>(logits, pv, pi, vocab);
    if (yk_check_launch("argmax_part")) return -1;
    argmax_final_kernel<<<n_rows, 64, 0, stream>>>(pv, pi, out);
    return yk_check_launch("argmax_final");
  }
  argmax_kernel<<<n_rows, 1024, 0, stream>>>(logits, out, vocab);
  return yk_check_launch("argmax");
}

// Per row: temperature, top_k (0: off), top_p, seed, draw.
__global__ __launch_bounds__(1024) void sample_kernel(
    const float* __restrict__ logits, int32_t* __restrict__ out, int vocab,
    const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const int32_t* __restrict__ seeds,
    const int32_t* __restrict__ draws) {
  __shared__ ArgMax ascratch[17];
  __shared__ float fscratch[17];
  const int rowi = blockIdx.x;
  const float* row = logits + static_cast<size_t>(rowi) * vocab;
  const float temp = temperature[rowi];
  const int k = top_k[rowi];
  const float p_lim = top_p[rowi];

  // the largest logit and its index
  ArgMax best{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) best = better(best, ArgMax{row[i], i});
  best = block_argmax(best, ascratch);
  if (temp <= 0.f) {
    if (threadIdx.x == 0) out[rowi] = best.i == 0x7fffffff ? 0 : best.i;
    return;
  }

  // top-k: the largest key t with count(key >= t) >= k; logits below it are dropped
  uint32_t k_key = 0u;
  if (k > 0 && k < vocab) {
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = k_key | (1u << bit);
      float cnt = 0.f;
      for (int i = threadIdx.x; i < vocab; i += blockDim.x) cnt += order_key(row[i]) >= cand ? 1.f : 0.f;
      cnt = block_sum(cnt, fscratch);
      if (cnt >= static_cast<float>(k)) k_key = cand;
    }
  }

  // softmax denominator over the kept logits at this temperature
  const float inv_t = 1.f / temp;
  const float top = best.v * inv_t;
  float z = 0.f;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float x = row[i];
    if (order_key(x) >= k_key) z += expf(x * inv_t - top);
  }
  z = block_sum(z, fscratch);

  // top-p: keep token i iff the mass of all tokens at least as likely as i is <= top_p.
  // Find the largest key t whose mass(key >= t) still exceeds top_p; tokens above it stay.
  uint32_t p_key = k_key;  // tokens with key > p_key are kept (plus the best one)
  bool p_active = false;
  if (p_lim < 1.f) {
    p_active = true;
    uint32_t t = 0u;
    bool any = false;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = t | (1u << bit);
      float mass = 0.f;
      for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        const float x = row[i];
        const uint32_t key = order_key(x);
        if (key >= cand && key >= k_key) mass += expf(x * inv_t - top);
      }
      mass = block_sum(mass, fscratch);
      if (mass > p_lim * z) {
        t = cand;
        any = true;
      }
    }
    // mass(key >= 0) = z > top_p * z always, so `any` only says whether t moved off 0
    (void)any;
    p_key = t;
  }

  // the race over the kept tokens
  const uint64_t base = mix64((static_cast<uint64_t>(static_cast<uint32_t>(seeds[rowi])) << 32) |
                              static_cast<uint32_t>(draws[rowi]));
  ArgMax win{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float x = row[i];
    const uint32_t key = order_key(x);
    bool keep = key >= k_key;
    if (p_active) keep = keep && (key > p_key || i == best.i);
    if (!keep) continue;
    const uint64_t zz = mix64(base + static_cast<uint64_t>(i));
    const float u = (static_cast<float>(zz >> 41) + 0.5f) * (1.f / 8388608.f);
    const float e = -logf(u);
    const float p = expf(x * inv_t - top) / z;
    win = better(win, ArgMax{p / e, i});
  }
  win = block_argmax(win, ascratch);
  if (threadIdx.x == 0) out[rowi] = win.i == 0x7fffffff ? best.i : win.i;
}

extern "C" int yk_sample(const float* logits, int32_t* out, int n_rows, int vocab,
                         const float* temperature, const int32_t* top_k, const float* top_p,
                         const int32_t* seeds, const int32_t* draws, hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes");
  if (n_rows == 0) return 0;
  sample_kernel<<<n_rows, 1024, 0, stream>>>(logits, out, vocab, temperature, top_k, top_p, seeds, draws);
  return yk_check_launch("sample");
}
