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
#include <mutex>
#include <string>

#include "common.h"
#include "no_alloc.h"

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

// ------------------------------------------------- argmax without any allocation (no_alloc.h)
// The partial results of argmax_part_kernel for up to YK_ARGMAX_STATIC_MAX_ROWS rows: the
// values, then the indices.  In host code this name is only a handle for
// hipGetSymbolAddress: the device address it yields (one per GPU) is what kernels get.
static __device__ __align__(256) unsigned char yk_static_scratch[YK_ARGMAX_STATIC_MAX_ROWS * ARGMAX_CHUNKS * (sizeof(float) + sizeof(int32_t))];

constexpr int YK_MAX_DEVICES = 64;
static void* yk_static_scratch_ptr[YK_MAX_DEVICES];  // per device, null until looked up
static std::mutex yk_static_scratch_lock;

// The current device's copy of the array, looked up at the first call on that device.
static void* static_scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= YK_MAX_DEVICES) {
    yk_fail("argmax_static: cannot tell the current device");
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(yk_static_scratch_lock);
  if (!yk_static_scratch_ptr[dev]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(yk_static_scratch));
    if (e != hipSuccess || !p) {
      yk_fail(std::string("argmax_static: hipGetSymbolAddress failed: ") + hipGetErrorString(e));
      return nullptr;
    }
    yk_static_scratch_ptr[dev] = p;
  }
  return yk_static_scratch_ptr[dev];
}

extern "C" int yk_argmax_static_setup(void) { return static_scratch_of_current_device() ? 0 : -1; }

extern "C" int yk_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && vocab > 0, "argmax_static: bad sizes");
  YK_REQUIRE(n_rows <= YK_ARGMAX_STATIC_MAX_ROWS,
             "argmax_static: more rows than the static scratch holds (" + std::to_string(YK_ARGMAX_STATIC_MAX_ROWS) + ")");
  if (n_rows == 0) return 0;
  YK_REQUIRE(logits && out, "argmax_static: null argument");
  void* scratch = static_scratch_of_current_device();
  if (!scratch) return -1;
  // every row goes through the two kernels (slices of a short row may be empty: they hold the
  // "nothing" entry, which never wins), so that the scratch is what carries the result
  float* pv = static_cast<float*>(scratch);
  int32_t* pi = reinterpret_cast<int32_t*>(pv + static_cast<size_t>(n_rows) * ARGMAX_CHUNKS);
  argmax_part_kernel<<<dim3(n_rows, ARGMAX_CHUNKS), 256, 0, stream>>>(logits, pv, pi, vocab);
  if (yk_check_launch("argmax_part (static scratch)")) return -1;
  argmax_final_kernel<<<n_rows, 64, 0, stream>>>(pv, pi, out);
  return yk_check_launch("argmax_final (static scratch)");
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

// ------------------------------------------------- a row divided among workgroups
// One workgroup passes over a row of 128K logits in about ten microseconds, and the
// thresholds need several passes: for large vocabularies a row is divided among SP_CHUNKS
// workgroups instead.  Tokens are put into SP_BINS bins by their distance from the largest
// logit (after the temperature), each bin with its count and its probability mass; the bin
// that holds a threshold follows from the running sums, and only that bin's tokens (top_p)
// or the tokens down to that bin (top_k) are candidates for the exact threshold, which one
// wave finds among them.  Masses are summed as integers (units of 2^-40 of the largest
// token's), so that sums do not depend on their order and a sum over bins equals the sum
// over their tokens.  A row whose candidates do not fit is left to the one-workgroup kernel.
constexpr int SP_CHUNKS = 8;
constexpr int SP_BINS = 1024;
constexpr int SP_THREADS = 1024;
constexpr double SP_ONE = 1099511627776.0;  // 2^40
constexpr float SP_FAR = 32.f;              // tokens e^-32 of the largest or less share the last bin
constexpr int SP_MIN_VOCAB = 8192;

enum SamplePath : int { SP_GREEDY = 0, SP_RACE = 1, SP_CANDS = 2, SP_DONE = 3, SP_WHOLE_ROW = 4 };

struct __attribute__((aligned(16))) SamplePlan {
  int path;
  int k_active, p_active;
  int bin_lo, bin_hi;  // candidates: the tokens of these bins
  int n_cand;
  int best_i;
  float best_v;
  float inv_t, bin_scale;
  uint32_t p_key;  // with p_active on path SP_RACE: tokens above it stay (and the largest)
  float z;         // the race's denominator
  unsigned long long mass_before;  // of the bins before bin_lo
  unsigned long long mass_total;
  int chunk_at[SP_CHUNKS];  // where each chunk's candidates start among the row's
};

typedef unsigned long long sp_mass_t;

// x * inv_t - top, rounded once: not above a rounding error of zero, and monotone in x
__device__ __forceinline__ float sp_exponent(float x, float inv_t, float top) { return __fmaf_rn(x, inv_t, -top); }
__device__ __forceinline__ int sp_bin(float exponent, float bin_scale) {
  return static_cast<int>(fminf(fmaxf(-exponent * bin_scale, 0.f), static_cast<float>(SP_BINS - 1)));
}
__device__ __forceinline__ sp_mass_t sp_mass(float e) { return static_cast<sp_mass_t>(static_cast<double>(e) * SP_ONE); }

__device__ __forceinline__ void sp_chunk(int vocab, int chunk, int& lo, int& hi) {
  const int per = ((vocab + SP_CHUNKS - 1) / SP_CHUNKS + 3) & ~3;  // starts stay 16-byte aligned
  lo = min(vocab, chunk * per);
  hi = min(vocab, lo + per);
}

// The largest logit of a row and the scale of its bins, from the chunks' parts.
struct SampleExtent {
  ArgMax best;
  float top, bin_scale;
};
__device__ __forceinline__ SampleExtent sp_extent(const ArgMax* __restrict__ part_best,
                                                  const float* __restrict__ part_low, float inv_t) {
  SampleExtent x;
  x.best = ArgMax{-INFINITY, 0x7fffffff};
  float low = INFINITY;
  for (int c = 0; c < SP_CHUNKS; ++c) {
    x.best = better(x.best, part_best[c]);
    low = fminf(low, part_low[c]);
  }
  x.top = x.best.v * inv_t;
  const float far = -sp_exponent(low, inv_t, x.top);  // the smallest finite logit's distance
  x.bin_scale = static_cast<float>(SP_BINS - 1) / fminf(fmaxf(far, 1e-6f), SP_FAR);
  return x;
}

template <typename T>
__device__ __forceinline__ T sp_wave_sum(T v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
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
    const int32_t* __restrict__ draws, int force_whole_row, const SamplePlan* __restrict__ plans,
    const ArgMax* __restrict__ race_part, int32_t* __restrict__ paths_out) {
  __shared__ SampleShared sh;
  const int rowi = blockIdx.x;
  if (plans) {
    // the row was divided among workgroups: finish what they left, or do the whole row here
    const SamplePlan& plan = plans[rowi];
    if (paths_out && threadIdx.x == 0) paths_out[rowi] = plan.path;
    if (plan.path == SP_DONE) return;
    if (plan.path == SP_GREEDY) {
      if (threadIdx.x == 0) out[rowi] = plan.best_i == 0x7fffffff ? 0 : plan.best_i;
      return;
    }
    if (plan.path == SP_RACE) {
      if (threadIdx.x == 0) {
        ArgMax win{-INFINITY, 0x7fffffff};
        for (int c = 0; c < SP_CHUNKS; ++c) win = better(win, race_part[rowi * SP_CHUNKS + c]);
        out[rowi] = win.i == 0x7fffffff ? plan.best_i : win.i;
      }
      return;
    }
  }
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

// ---- 1: the largest and the smallest finite logit of each chunk
__global__ __launch_bounds__(SP_THREADS) void sp_extent_kernel(const float* __restrict__ logits, int vocab,
                                                               ArgMax* __restrict__ part_best,
                                                               float* __restrict__ part_low) {
  __shared__ ArgMax ascratch[17];
  __shared__ float fscratch[17];
  const int rowi = blockIdx.x, chunk = blockIdx.y;
  const float* row = logits + static_cast<size_t>(rowi) * vocab;
  int lo, hi;
  sp_chunk(vocab, chunk, lo, hi);
  ArgMax best{-INFINITY, 0x7fffffff};
  float neg_low = -INFINITY;
  for_each_logit(row + lo, hi - lo, [&](float x, int i) {
    best = better(best, ArgMax{x, lo + i});
    if (x > -INFINITY) neg_low = fmaxf(neg_low, -x);
  });
  best = block_argmax(best, ascratch);
  neg_low = block_max(neg_low, fscratch);
  if (threadIdx.x == 0) {
    part_best[rowi * SP_CHUNKS + chunk] = best;
    part_low[rowi * SP_CHUNKS + chunk] = -neg_low;
  }
}

// ---- 2: count and mass of every bin, chunk by chunk
__global__ __launch_bounds__(SP_THREADS) void sp_histogram_kernel(
    const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
    const ArgMax* __restrict__ part_best, const float* __restrict__ part_low,
    uint32_t* __restrict__ hist_count, sp_mass_t* __restrict__ hist_mass) {
  __shared__ uint32_t count[SP_BINS];
  __shared__ sp_mass_t mass[SP_BINS];
  const int rowi = blockIdx.x, chunk = blockIdx.y;
  const float temp = temperature[rowi];
  if (temp <= 0.f) return;
  const float inv_t = 1.f / temp;
  const SampleExtent ext = sp_extent(part_best + rowi * SP_CHUNKS, part_low + rowi * SP_CHUNKS, inv_t);
  for (int b = threadIdx.x; b < SP_BINS; b += blockDim.x) {
    count[b] = 0u;
    mass[b] = 0ull;
  }
  __syncthreads();
  const float* row = logits + static_cast<size_t>(rowi) * vocab;
  int lo, hi;
  sp_chunk(vocab, chunk, lo, hi);
  for_each_logit(row + lo, hi - lo, [&](float x, int) {
    const float a = sp_exponent(x, inv_t, ext.top);
    const int b = sp_bin(a, ext.bin_scale);
    atomicAdd(&count[b], 1u);
    const sp_mass_t m = sp_mass(expf(a));
    if (m) atomicAdd(&mass[b], m);
  });
  __syncthreads();
  const size_t at = (static_cast<size_t>(rowi) * SP_CHUNKS + chunk) * SP_BINS;
  for (int b = threadIdx.x; b < SP_BINS; b += blockDim.x) {
    hist_count[at + b] = count[b];
    hist_mass[at + b] = mass[b];
  }
}

// Running sum over the block's threads in thread order; every thread gets its own.
__device__ sp_mass_t sp_block_scan(sp_mass_t v, sp_mass_t* scratch) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const sp_mass_t y = __shfl_up(v, o, 64);
    if (lane >= o) v += y;
  }
  __syncthreads();
  if (lane == 63) scratch[wave] = v;
  __syncthreads();
  sp_mass_t before = 0ull;
  for (int w = 0; w < wave; ++w) before += scratch[w];
  return v + before;
}

// ---- 3: which bins hold the thresholds; one workgroup a row, one thread a bin
__global__ __launch_bounds__(SP_BINS) void sp_plan_kernel(
    int vocab, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const ArgMax* __restrict__ part_best,
    const float* __restrict__ part_low, const uint32_t* __restrict__ hist_count,
    const sp_mass_t* __restrict__ hist_mass, SamplePlan* __restrict__ plans) {
  __shared__ sp_mass_t scan_scratch[17];
  __shared__ float fscratch[17];
  __shared__ sp_mass_t picked[3];
  const int rowi = blockIdx.x, b = threadIdx.x;
  const float temp = temperature[rowi];
  SamplePlan plan;
  plan.path = SP_GREEDY;
  plan.k_active = plan.p_active = 0;
  plan.bin_lo = plan.bin_hi = plan.n_cand = 0;
  plan.p_key = 0u;
  plan.z = 1.f;
  plan.mass_before = plan.mass_total = 0ull;
  for (int c = 0; c < SP_CHUNKS; ++c) plan.chunk_at[c] = 0;
  plan.inv_t = temp > 0.f ? 1.f / temp : 1.f;
  const SampleExtent ext = sp_extent(part_best + rowi * SP_CHUNKS, part_low + rowi * SP_CHUNKS, plan.inv_t);
  plan.best_i = ext.best.i;
  plan.best_v = ext.best.v;
  plan.bin_scale = ext.bin_scale;
  if (temp <= 0.f) {
    if (b == 0) plans[rowi] = plan;
    return;
  }
  const int k = top_k[rowi];
  const float p_lim = top_p[rowi];
  plan.k_active = k > 0 && k < vocab;
  plan.p_active = p_lim < 1.f;

  const size_t at = static_cast<size_t>(rowi) * SP_CHUNKS * SP_BINS + b;
  uint32_t per_chunk[SP_CHUNKS];
  sp_mass_t n_here = 0ull, m_here = 0ull;
#pragma unroll
  for (int c = 0; c < SP_CHUNKS; ++c) {
    per_chunk[c] = hist_count[at + c * SP_BINS];
    n_here += per_chunk[c];
    m_here += hist_mass[at + c * SP_BINS];
  }
  const sp_mass_t n_to = sp_block_scan(n_here, scan_scratch);  // tokens of the bins up to this one
  const sp_mass_t m_to = sp_block_scan(m_here, scan_scratch);  // and their mass
  __syncthreads();
  if (b == SP_BINS - 1) picked[0] = m_to;
  __syncthreads();
  plan.mass_total = picked[0];
  plan.z = static_cast<float>(static_cast<double>(plan.mass_total) * (1.0 / SP_ONE));
  if (!plan.k_active && !plan.p_active) {
    plan.path = SP_RACE;
    if (b == 0) plans[rowi] = plan;
    return;
  }
  // the running sums only grow: the first bin that reaches the wanted sum is found by
  // counting the bins that do not
  bool reached;
  if (plan.k_active) reached = n_to >= static_cast<sp_mass_t>(k);
  else reached = static_cast<double>(m_to) > static_cast<double>(p_lim) * static_cast<double>(plan.mass_total);
  const int first = static_cast<int>(block_sum(reached ? 0.f : 1.f, fscratch));
  if (first >= SP_BINS) {  // no bin reaches it (a row without a finite logit)
    plan.path = SP_WHOLE_ROW;
    if (b == 0) plans[rowi] = plan;
    return;
  }
  __syncthreads();
  if (b == first) {
    picked[0] = n_to;
    picked[1] = n_here;
    picked[2] = m_to - m_here;
  }
  __syncthreads();
  if (plan.k_active) {
    plan.bin_lo = 0;
    plan.bin_hi = first;
    plan.n_cand = static_cast<int>(min(picked[0], static_cast<sp_mass_t>(0x7fffffff)));
  } else {
    plan.bin_lo = plan.bin_hi = first;
    plan.n_cand = static_cast<int>(picked[1]);
    plan.mass_before = picked[2];
  }
  plan.path = plan.n_cand <= CAND_MAX ? SP_CANDS : SP_WHOLE_ROW;
  if (plan.path == SP_CANDS) {
    const bool mine = b >= plan.bin_lo && b <= plan.bin_hi;
    int from = 0;
#pragma unroll
    for (int c = 0; c < SP_CHUNKS; ++c) {
      plan.chunk_at[c] = from;
      from += static_cast<int>(block_sum(mine ? static_cast<float>(per_chunk[c]) : 0.f, fscratch));
    }
  }
  if (b == 0) plans[rowi] = plan;
}

// ---- 4: the candidates, in index order
__global__ __launch_bounds__(SP_THREADS) void sp_collect_kernel(
    const float* __restrict__ logits, int vocab, const SamplePlan* __restrict__ plans,
    uint32_t* __restrict__ cand_key, float* __restrict__ cand_e, int32_t* __restrict__ cand_idx) {
  __shared__ int wave_count[17];
  const int rowi = blockIdx.x, chunk = blockIdx.y;
  const SamplePlan& plan = plans[rowi];
  if (plan.path != SP_CANDS) return;
  const float inv_t = plan.inv_t, top = plan.best_v * inv_t, bin_scale = plan.bin_scale;
  const int bin_lo = plan.bin_lo, bin_hi = plan.bin_hi;
  const float* row = logits + static_cast<size_t>(rowi) * vocab;
  int lo, hi;
  sp_chunk(vocab, chunk, lo, hi);
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, n_waves = blockDim.x / 64;
  const int per_wave = (hi - lo + n_waves - 1) / n_waves;
  const int w_lo = min(hi, lo + wave * per_wave), w_hi = min(hi, w_lo + per_wave);
  int mine = 0;
  for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
    const int i = i0 + lane;
    bool hit = false;
    if (i < w_hi) {
      const int b = sp_bin(sp_exponent(row[i], inv_t, top), bin_scale);
      hit = b >= bin_lo && b <= bin_hi;
    }
    mine += __popcll(__ballot(hit));
  }
  if (lane == 0) wave_count[wave] = mine;
  __syncthreads();
  int at = plan.chunk_at[chunk];
  for (int w = 0; w < wave; ++w) at += wave_count[w];
  const size_t base = static_cast<size_t>(rowi) * CAND_MAX;
  for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
    const int i = i0 + lane;
    bool hit = false;
    float x = 0.f, a = 0.f;
    if (i < w_hi) {
      x = row[i];
      a = sp_exponent(x, inv_t, top);
      const int b = sp_bin(a, bin_scale);
      hit = b >= bin_lo && b <= bin_hi;
    }
    const unsigned long long mask = __ballot(hit);
    if (hit) {
      const int slot = at + __popcll(mask & ((1ull << lane) - 1ull));
      if (slot < CAND_MAX) {
        cand_key[base + slot] = order_key(x);
        cand_e[base + slot] = expf(a);
        cand_idx[base + slot] = i;
      }
    }
    at += __popcll(mask);
  }
}

// ---- 5: the exact thresholds among the candidates, by one wave; with top_k the race too
__global__ __launch_bounds__(64) void sp_choose_kernel(
    int vocab, const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
    const int32_t* __restrict__ seeds, const int32_t* __restrict__ draws,
    const uint32_t* __restrict__ cand_key, const float* __restrict__ cand_e,
    const int32_t* __restrict__ cand_idx, SamplePlan* __restrict__ plans, int32_t* __restrict__ out) {
  __shared__ uint32_t key[CAND_MAX];
  __shared__ float e[CAND_MAX];
  __shared__ int32_t idx[CAND_MAX];
  const int rowi = blockIdx.x, lane = threadIdx.x;
  const SamplePlan plan = plans[rowi];
  if (plan.path != SP_CANDS) return;
  const int n = min(plan.n_cand, CAND_MAX);
  const size_t base = static_cast<size_t>(rowi) * CAND_MAX;
  uint32_t k_low = 0xffffffffu, k_high = 0u;
  for (int j = lane; j < n; j += 64) {
    const uint32_t kj = cand_key[base + j];
    key[j] = kj;
    e[j] = cand_e[base + j];
    idx[j] = cand_idx[base + j];
    k_low = min(k_low, kj);
    k_high = max(k_high, kj);
  }
  __syncthreads();
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    k_low = min(k_low, static_cast<uint32_t>(__shfl_xor(k_low, o, 64)));
    k_high = max(k_high, static_cast<uint32_t>(__shfl_xor(k_high, o, 64)));
  }
  // a threshold is one of the candidates' keys: the bits they all share are settled
  const uint32_t differ = k_low ^ k_high;
  const int top_bit = differ ? 31 - __clz(differ) : -1;
  const uint32_t shared_bits = top_bit >= 31 ? 0u : (top_bit < 0 ? k_high : k_high & ~((2u << top_bit) - 1u));

  uint32_t k_key = 0u;
  sp_mass_t total = plan.mass_total;
  if (plan.k_active) {
    const int k = top_k[rowi];
    k_key = shared_bits;  // count(key >= k_key) >= k holds; raise it bit by bit where it still does
    for (int bit = top_bit; bit >= 0; --bit) {
      const uint32_t t = k_key | (1u << bit);
      int c = 0;
      for (int j = lane; j < n; j += 64) c += key[j] >= t ? 1 : 0;
      if (sp_wave_sum(c) >= k) k_key = t;
    }
    sp_mass_t m = 0ull;
    for (int j = lane; j < n; j += 64)
      if (key[j] >= k_key) m += sp_mass(e[j]);
    total = sp_wave_sum(m);
  }
  const float z = static_cast<float>(static_cast<double>(total) * (1.0 / SP_ONE));
  uint32_t p_key = k_key;
  if (plan.p_active) {
    // the largest key whose mass(key >= it) still exceeds top_p of the kept mass
    const double limit = static_cast<double>(top_p[rowi]) * static_cast<double>(total);
    uint32_t t0 = shared_bits;
    for (int bit = top_bit; bit >= 0; --bit) {
      const uint32_t t = t0 | (1u << bit);
      sp_mass_t m = 0ull;
      for (int j = lane; j < n; j += 64) {
        const uint32_t kj = key[j];
        if (kj >= t && kj >= k_key) m += sp_mass(e[j]);
      }
      m = plan.mass_before + sp_wave_sum(m);
      if (static_cast<double>(m) > limit) t0 = t;
    }
    p_key = t0;
  }
  if (!plan.k_active) {
    // top_p alone: the kept tokens are spread over the row, which the next kernel races over
    if (lane == 0) {
      plans[rowi].p_key = p_key;
      plans[rowi].z = z;
      plans[rowi].path = SP_RACE;
    }
    return;
  }
  const uint64_t seed_base = mix64((static_cast<uint64_t>(static_cast<uint32_t>(seeds[rowi])) << 32) |
                                   static_cast<uint32_t>(draws[rowi]));
  ArgMax win{-INFINITY, 0x7fffffff};
  for (int j = lane; j < n; j += 64) {
    const uint32_t kj = key[j];
    const int i = idx[j];
    bool keep = kj >= k_key;
    if (plan.p_active) keep = keep && (kj > p_key || i == plan.best_i);
    if (keep) {
      const uint64_t zz = mix64(seed_base + static_cast<uint64_t>(i));
      const float u = (static_cast<float>(zz >> 41) + 0.5f) * (1.f / 8388608.f);
      win = better(win, ArgMax{e[j] / z / -logf(u), i});
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax y;
    y.v = __shfl_xor(win.v, o, 64);
    y.i = __shfl_xor(win.i, o, 64);
    win = better(win, y);
  }
  if (lane == 0) {
    out[rowi] = win.i == 0x7fffffff ? plan.best_i : win.i;
    plans[rowi].path = SP_DONE;
  }
}

// ---- 6: the race over the whole row, chunk by chunk (no top_k: every token, or those above p_key)
__global__ __launch_bounds__(SP_THREADS) void sp_race_kernel(
    const float* __restrict__ logits, int vocab, const int32_t* __restrict__ seeds,
    const int32_t* __restrict__ draws, const SamplePlan* __restrict__ plans,
    ArgMax* __restrict__ race_part) {
  __shared__ ArgMax ascratch[17];
  const int rowi = blockIdx.x, chunk = blockIdx.y;
  const SamplePlan& plan = plans[rowi];
  if (plan.path != SP_RACE) return;
  const float inv_t = plan.inv_t, top = plan.best_v * inv_t, z = plan.z;
  const bool p_active = plan.p_active != 0;
  const uint32_t p_key = plan.p_key;
  const int best_i = plan.best_i;
  const uint64_t seed_base = mix64((static_cast<uint64_t>(static_cast<uint32_t>(seeds[rowi])) << 32) |
                                   static_cast<uint32_t>(draws[rowi]));
  const float* row = logits + static_cast<size_t>(rowi) * vocab;
  int lo, hi;
  sp_chunk(vocab, chunk, lo, hi);
  ArgMax win{-INFINITY, 0x7fffffff};
  for_each_logit(row + lo, hi - lo, [&](float x, int at) {
    const int i = lo + at;
    if (!p_active || order_key(x) > p_key || i == best_i) {
      const uint64_t zz = mix64(seed_base + static_cast<uint64_t>(i));
      const float u = (static_cast<float>(zz >> 41) + 0.5f) * (1.f / 8388608.f);
      win = better(win, ArgMax{expf(sp_exponent(x, inv_t, top)) / z / -logf(u), i});
    }
  });
  win = block_argmax(win, ascratch);
  if (threadIdx.x == 0) race_part[rowi * SP_CHUNKS + chunk] = win;
}

// What the divided path keeps between its kernels, for n_rows rows.
struct SampleWorkspace {
  sp_mass_t* hist_mass;
  SamplePlan* plans;
  uint32_t* hist_count;
  ArgMax* part_best;
  ArgMax* race_part;
  float* part_low;
  uint32_t* cand_key;
  float* cand_e;
  int32_t* cand_idx;
  size_t bytes;
};

static SampleWorkspace sample_workspace(void* base, size_t n_rows) {
  SampleWorkspace w;
  char* at = static_cast<char*>(base);
  auto take = [&](size_t bytes) {
    char* here = at;
    at += (bytes + 255) / 256 * 256;
    return here;
  };
  w.hist_mass = reinterpret_cast<sp_mass_t*>(take(n_rows * SP_CHUNKS * SP_BINS * sizeof(sp_mass_t)));
  w.plans = reinterpret_cast<SamplePlan*>(take(n_rows * sizeof(SamplePlan)));
  w.hist_count = reinterpret_cast<uint32_t*>(take(n_rows * SP_CHUNKS * SP_BINS * sizeof(uint32_t)));
  w.part_best = reinterpret_cast<ArgMax*>(take(n_rows * SP_CHUNKS * sizeof(ArgMax)));
  w.race_part = reinterpret_cast<ArgMax*>(take(n_rows * SP_CHUNKS * sizeof(ArgMax)));
  w.part_low = reinterpret_cast<float*>(take(n_rows * SP_CHUNKS * sizeof(float)));
  w.cand_key = reinterpret_cast<uint32_t*>(take(n_rows * CAND_MAX * sizeof(uint32_t)));
  w.cand_e = reinterpret_cast<float*>(take(n_rows * CAND_MAX * sizeof(float)));
  w.cand_idx = reinterpret_cast<int32_t*>(take(n_rows * CAND_MAX * sizeof(int32_t)));
  w.bytes = static_cast<size_t>(at - static_cast<char*>(base));
  return w;
}

// Bytes of workspace with which yk_sample divides the rows of a large vocabulary among
// workgroups (0: this vocabulary is left to one workgroup a row, which needs none).
extern "C" size_t yk_sample_workspace_bytes(int n_rows, int vocab) {
  if (n_rows <= 0 || vocab < SP_MIN_VOCAB) return 0;
  return sample_workspace(nullptr, static_cast<size_t>(n_rows)).bytes;
}

// workspace: yk_sample_workspace_bytes bytes, 256-byte aligned, or null (then, as with
// force_whole_row, every row is one workgroup's work).  paths_out (may be null) receives, for
// rows that were divided, which way each went (SamplePath); other rows are left untouched.
extern "C" int yk_sample(const float* logits, int32_t* out, int n_rows, int vocab,
                         const float* temperature, const int32_t* top_k, const float* top_p,
                         const int32_t* seeds, const int32_t* draws, int force_whole_row,
                         void* workspace, size_t workspace_bytes, int32_t* paths_out,
                         hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes");
  if (n_rows == 0) return 0;
  const size_t need = yk_sample_workspace_bytes(n_rows, vocab);
  const bool divide = need > 0 && !force_whole_row && workspace && workspace_bytes >= need && n_rows <= 65535;
  if (!divide) {
    sample_kernel<<<n_rows, 1024, 0, stream>>>(logits, out, vocab, temperature, top_k, top_p, seeds, draws,
                                               force_whole_row, nullptr, nullptr, nullptr);
    return yk_check_launch("sample");
  }
  YK_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, "sample: the workspace must be 256-byte aligned");
  const SampleWorkspace w = sample_workspace(workspace, static_cast<size_t>(n_rows));
  const dim3 chunks(n_rows, SP_CHUNKS);
  sp_extent_kernel<<<chunks, SP_THREADS, 0, stream>>>(logits, vocab, w.part_best, w.part_low);
  if (yk_check_launch("sample: extent")) return -1;
  sp_histogram_kernel<<<chunks, SP_THREADS, 0, stream>>>(logits, vocab, temperature, w.part_best, w.part_low,
                                                         w.hist_count, w.hist_mass);
  if (yk_check_launch("sample: histogram")) return -1;
  sp_plan_kernel<<<n_rows, SP_BINS, 0, stream>>>(vocab, temperature, top_k, top_p, w.part_best, w.part_low,
                                                 w.hist_count, w.hist_mass, w.plans);
  if (yk_check_launch("sample: plan")) return -1;
  sp_collect_kernel<<<chunks, SP_THREADS, 0, stream>>>(logits, vocab, w.plans, w.cand_key, w.cand_e, w.cand_idx);
  if (yk_check_launch("sample: collect")) return -1;
  sp_choose_kernel<<<n_rows, 64, 0, stream>>>(vocab, top_k, top_p, seeds, draws, w.cand_key, w.cand_e, w.cand_idx,
                                              w.plans, out);
  if (yk_check_launch("sample: choose")) return -1;
  sp_race_kernel<<<chunks, SP_THREADS, 0, stream>>>(logits, vocab, seeds, draws, w.plans, w.race_part);
  if (yk_check_launch("sample: race")) return -1;
  sample_kernel<<<n_rows, 1024, 0, stream>>>(logits, out, vocab, temperature, top_k, top_p, seeds, draws, 0,
                                             w.plans, w.race_part, paths_out);
  return yk_check_launch("sample");
}
