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
// bisection over the order-preserving integer image of the floats, without sorting.
// Equal logits are therefore treated alike: all tokens tied with the k-th largest stay (as
// in the reference, which compares with the k-th value), and tokens tied with the one that
// crosses top_p are dropped together (the reference's sort leaves their order undefined).
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

// ------------------------------------------------------------------------- sampling
// Every element of a row, four at a time where the row is 16-byte aligned.  f(x, index).
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ row, int vocab, F f) {
  if (reinterpret_cast<uintptr_t>(row) % 16 == 0) {
    const int n4 = vocab / 4;
    // four loads in flight per thread: a pass over a row is one workgroup's work and would
    // otherwise wait for memory once per load (elements still reach f in ascending order)
    int j = threadIdx.x;
    for (; j + 3 * static_cast<int>(blockDim.x) < n4; j += 4 * blockDim.x) {
      float4 v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = reinterpret_cast<const float4*>(row)[j + q * blockDim.x];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i = 4 * (j + q * blockDim.x);
        f(v[q].x, i);
        f(v[q].y, i + 1);
        f(v[q].z, i + 2);
        f(v[q].w, i + 3);
      }
    }
    for (; j < n4; j += blockDim.x) {
      const float4 v = reinterpret_cast<const float4*>(row)[j];
      f(v.x, 4 * j);
      f(v.y, 4 * j + 1);
      f(v.z, 4 * j + 2);
      f(v.w, 4 * j + 3);
    }
    for (int i = 4 * n4 + threadIdx.x; i < vocab; i += blockDim.x) f(row[i], i);
  } else {
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) f(row[i], i);
  }
}

// Tokens that can still matter once the largest ones are known are kept in LDS; a row whose
// candidates do not fit (a flat distribution under top_p alone, thousands of equal logits)
// takes the slow path, which passes over the whole row for every bit of a threshold.
constexpr int CAND_MAX = 4096;

struct SampleShared {
  ArgMax ascratch[17];
  float fscratch[17];
  int counts[16];
  int wave_count[17];
  uint32_t key[CAND_MAX];
  float e[CAND_MAX];
  int32_t idx[CAND_MAX];
};

// The whole-row path: thresholds by bisection over the row itself (32 passes each).
__device__ int sample_whole_row(const float* __restrict__ row, int vocab, ArgMax best, float inv_t,
                                int k, float p_lim, uint64_t base, SampleShared& sh) {
  const float top = best.v * inv_t;
  // top-k: the largest key t with count(key >= t) >= k; logits below it are dropped
  uint32_t k_key = 0u;
  if (k > 0 && k < vocab) {
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = k_key | (1u << bit);
      float cnt = 0.f;
      for_each_logit(row, vocab, [&](float x, int) { cnt += order_key(x) >= cand ? 1.f : 0.f; });
      cnt = block_sum(cnt, sh.fscratch);
      if (cnt >= static_cast<float>(k)) k_key = cand;
    }
  }
  float z = 0.f;
  for_each_logit(row, vocab, [&](float x, int) {
    if (order_key(x) >= k_key) z += expf(x * inv_t - top);
  });
  z = block_sum(z, sh.fscratch);
  // top-p: keep token i iff the mass of all tokens at least as likely as i is <= top_p.
  // Find the largest key t whose mass(key >= t) still exceeds top_p; tokens above it stay.
  uint32_t p_key = k_key;
  const bool p_active = p_lim < 1.f;
  if (p_active) {
    uint32_t t = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = t | (1u << bit);
      float mass = 0.f;
      for_each_logit(row, vocab, [&](float x, int) {
        const uint32_t key = order_key(x);
        if (key >= cand && key >= k_key) mass += expf(x * inv_t - top);
      });
      mass = block_sum(mass, sh.fscratch);
      if (mass > p_lim * z) t = cand;  // mass(key >= 0) = z > top_p * z: t = 0 always qualifies
    }
    p_key = t;
  }
  ArgMax win{-INFINITY, 0x7fffffff};
  for_each_logit(row, vocab, [&](float x, int i) {
    const uint32_t key = order_key(x);
    bool keep = key >= k_key;
    if (p_active) keep = keep && (key > p_key || i == best.i);
    if (keep) {
      const uint64_t zz = mix64(base + static_cast<uint64_t>(i));
      const float u = (static_cast<float>(zz >> 41) + 0.5f) * (1.f / 8388608.f);
      win = better(win, ArgMax{expf(x * inv_t - top) / z / -logf(u), i});
    }
  });
  win = block_argmax(win, sh.ascratch);
  return win.i == 0x7fffffff ? best.i : win.i;
}

// Per row: temperature, top_k (0: off), top_p, seed, draw.
//
// With top_k or top_p the tokens that can be kept are first narrowed down: passes over the
// row count the keys at or above 15 thresholds at once (four bits of the threshold a pass)
// until at most CAND_MAX tokens lie at or above the bound that still holds the wanted
// number (k, or CAND_MAX itself for top_p alone); those are copied to LDS in index order
// (each wave owns a stretch of the row, so the order does not depend on timing) and the
// exact thresholds, the sums and the race are done there.
__global__ __launch_bounds__(1024) void sample_kernel(
    const float* __restrict__ logits, int32_t* __restrict__ out, int vocab,
    const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const int32_t* __restrict__ seeds,
    const int32_t* __restrict__ draws, int force_whole_row) {
  __shared__ SampleShared sh;
  const int rowi = blockIdx.x;
  const float* row = logits + static_cast<size_t>(rowi) * vocab;
  const float temp = temperature[rowi];
  const int k = top_k[rowi];
  const float p_lim = top_p[rowi];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, n_waves = blockDim.x / 64;

  // the largest logit and its index
  ArgMax best{-INFINITY, 0x7fffffff};
  for_each_logit(row, vocab, [&](float x, int i) { best = better(best, ArgMax{x, i}); });
  best = block_argmax(best, sh.ascratch);
  if (temp <= 0.f) {
    if (threadIdx.x == 0) out[rowi] = best.i == 0x7fffffff ? 0 : best.i;
    return;
  }
  const float inv_t = 1.f / temp;
  const float top = best.v * inv_t;
  const uint64_t base = mix64((static_cast<uint64_t>(static_cast<uint32_t>(seeds[rowi])) << 32) |
                              static_cast<uint32_t>(draws[rowi]));
  const bool k_active = k > 0 && k < vocab;
  const bool p_active = p_lim < 1.f;

  if (!k_active && !p_active) {
    // plain temperature sampling: the denominator, then the race, over the whole row
    float z = 0.f;
    for_each_logit(row, vocab, [&](float x, int) { z += expf(x * inv_t - top); });
    z = block_sum(z, sh.fscratch);
    ArgMax win{-INFINITY, 0x7fffffff};
    for_each_logit(row, vocab, [&](float x, int i) {
      const uint64_t zz = mix64(base + static_cast<uint64_t>(i));
      const float u = (static_cast<float>(zz >> 41) + 0.5f) * (1.f / 8388608.f);
      win = better(win, ArgMax{expf(x * inv_t - top) / z / -logf(u), i});
    });
    win = block_argmax(win, sh.ascratch);
    if (threadIdx.x == 0) out[rowi] = win.i == 0x7fffffff ? best.i : win.i;
    return;
  }

  // ---- narrow down: the largest bound with count(key >= bound) >= want, four bits a pass
  // (top_p alone: any bound with between CAND_MAX / 2 and CAND_MAX tokens above it will do)
  const int want = k_active ? k : min(CAND_MAX / 2, vocab);
  uint32_t bound = 0u;
  int n_ge = vocab;  // count(key >= bound)
  int bits_done = 0;
  bool fits = !force_whole_row && want <= CAND_MAX;
  while (fits && n_ge > CAND_MAX && bits_done < 32) {
    const int shift = 28 - bits_done;
    int c[15];
#pragma unroll
    for (int j = 0; j < 15; ++j) c[j] = 0;
    for_each_logit(row, vocab, [&](float x, int) {
      const uint32_t key = order_key(x);
      if (key >= bound) {
        const uint32_t digit = (key - bound) >> shift;  // 0..15 within the current bucket, more above it
#pragma unroll
        for (int j = 0; j < 15; ++j) c[j] += digit >= static_cast<uint32_t>(j + 1) ? 1 : 0;
      }
    });
    __syncthreads();
    if (threadIdx.x < 16) sh.counts[threadIdx.x] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 15; ++j) {
      int v = c[j];
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
      if (lane == 0 && v) atomicAdd(&sh.counts[j], v);
    }
    __syncthreads();
    int pick = 0;
#pragma unroll
    for (int j = 0; j < 15; ++j)
      if (sh.counts[j] >= want) pick = j + 1;  // counts fall with j: the last that holds is the largest
    if (pick > 0) {
      n_ge = sh.counts[pick - 1];
      bound += static_cast<uint32_t>(pick) << shift;
    }
    bits_done += 4;
  }
  fits = fits && n_ge <= CAND_MAX;
  if (!fits) {
    const int tok = sample_whole_row(row, vocab, best, inv_t, k, p_lim, base, sh);
    if (threadIdx.x == 0) out[rowi] = tok;
    return;
  }

  // ---- copy the candidates (key >= bound) to LDS in index order: wave w owns the w-th stretch
  const int per_wave = (vocab + n_waves - 1) / n_waves;
  const int w_lo = min(vocab, wave * per_wave), w_hi = min(vocab, w_lo + per_wave);
  int mine = 0;
  for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
    const int i = i0 + lane;
    const bool hit = i < w_hi && order_key(row[i]) >= bound;
    mine += __popcll(__ballot(hit));
  }
  __syncthreads();
  if (lane == 0) sh.wave_count[wave] = mine;
  __syncthreads();
  int at = 0;
  for (int w = 0; w < wave; ++w) at += sh.wave_count[w];
  for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
    const int i = i0 + lane;
    const float x = i < w_hi ? row[i] : 0.f;
    const uint32_t key = order_key(x);
    const bool hit = i < w_hi && key >= bound;
    const unsigned long long mask = __ballot(hit);
    if (hit) {
      const int slot = at + __popcll(mask & ((1ull << lane) - 1ull));
      sh.key[slot] = key;
      sh.e[slot] = expf(x * inv_t - top);
      sh.idx[slot] = i;
    }
    at += __popcll(mask);
  }
  __syncthreads();
  const int n_cand = n_ge;

  // ---- top-k: the exact k-th largest key, by bisection over the candidates
  uint32_t k_key = 0u;
  if (k_active) {
    k_key = bound;  // count(key >= bound) >= k holds; raise it bit by bit where it still does
    for (int bit = 31 - bits_done; bit >= 0; --bit) {
      const uint32_t cand = k_key | (1u << bit);
      float cnt = 0.f;
      for (int j = threadIdx.x; j < n_cand; j += blockDim.x) cnt += sh.key[j] >= cand ? 1.f : 0.f;
      cnt = block_sum(cnt, sh.fscratch);
      if (cnt >= static_cast<float>(k)) k_key = cand;
    }
  }

  // ---- softmax denominator over the kept logits
  float z = 0.f;
  if (k_active) {
    for (int j = threadIdx.x; j < n_cand; j += blockDim.x)
      if (sh.key[j] >= k_key) z += sh.e[j];
  } else {
    for_each_logit(row, vocab, [&](float x, int) { z += expf(x * inv_t - top); });
  }
  z = block_sum(z, sh.fscratch);

  // ---- top-p over the candidates
  uint32_t p_key = k_key;
  if (p_active) {
    if (!k_active) {
      // the candidates must hold the threshold: their mass has to exceed top_p of the whole
      float mass = 0.f;
      for (int j = threadIdx.x; j < n_cand; j += blockDim.x) mass += sh.e[j];
      mass = block_sum(mass, sh.fscratch);
      if (!(mass > p_lim * z) && n_cand < vocab) {
        const int tok = sample_whole_row(row, vocab, best, inv_t, k, p_lim, base, sh);
        if (threadIdx.x == 0) out[rowi] = tok;
        return;
      }
    }
    uint32_t t = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = t | (1u << bit);
      float mass = 0.f;
      for (int j = threadIdx.x; j < n_cand; j += blockDim.x) {
        const uint32_t key = sh.key[j];
        if (key >= cand && key >= k_key) mass += sh.e[j];
      }
      mass = block_sum(mass, sh.fscratch);
      if (mass > p_lim * z) t = cand;
    }
    // (below the candidates' bound the sum misses tokens, but there it exceeds the limit
    // anyway, as the true mass does: the bisection decides as it would on the whole row)
    p_key = t;
  }

  // ---- the race over the kept candidates
  ArgMax win{-INFINITY, 0x7fffffff};
  for (int j = threadIdx.x; j < n_cand; j += blockDim.x) {
    const uint32_t key = sh.key[j];
    const int i = sh.idx[j];
    bool keep = key >= k_key;
    if (p_active) keep = keep && (key > p_key || i == best.i);
    if (keep) {
      const uint64_t zz = mix64(base + static_cast<uint64_t>(i));
      const float u = (static_cast<float>(zz >> 41) + 0.5f) * (1.f / 8388608.f);
      win = better(win, ArgMax{sh.e[j] / z / -logf(u), i});
    }
  }
  win = block_argmax(win, sh.ascratch);
  if (threadIdx.x == 0) out[rowi] = win.i == 0x7fffffff ? best.i : win.i;
}

extern "C" int yk_sample(const float* logits, int32_t* out, int n_rows, int vocab,
                         const float* temperature, const int32_t* top_k, const float* top_p,
                         const int32_t* seeds, const int32_t* draws, int force_whole_row,
                         hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes");
  if (n_rows == 0) return 0;
  sample_kernel<<<n_rows, 1024, 0, stream>>>(logits, out, vocab, temperature, top_k, top_p, seeds, draws,
                                             force_whole_row);
  return yk_check_launch("sample");
}
