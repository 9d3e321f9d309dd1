// Machine probes for the benchmark: what a plain streaming read and a plain loop of
// matrix-core instructions reach on the card at hand.  The published peaks (8 TB/s,
// 2.5 PFLOP/s) are what the benchmark prices against; these two numbers say how much of
// them any kernel can get, so that a kernel's distance from the machine can be told from
// its distance from the data sheet.  Neither touches the model.
#include "common.h"

typedef __bf16 probe_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float probe_f32x4_t __attribute__((ext_vector_type(4)));

// Every workgroup reads one contiguous span, four 16-byte loads in flight per thread;
// NT: loads marked as not to be kept in the caches, as the decode products mark their weights.
typedef float probe_load_t __attribute__((ext_vector_type(4)));
template <bool NT>
__global__ __launch_bounds__(256) void probe_stream_read_kernel(const probe_load_t* __restrict__ data, size_t n_vec,
                                                                float* __restrict__ sink) {
  const size_t per = (n_vec + gridDim.x - 1) / gridDim.x;
  const size_t begin = per * blockIdx.x;
  const size_t end = begin + per < n_vec ? begin + per : n_vec;
  float acc = 0.f;
  for (size_t i = begin + threadIdx.x; i < end; i += 256 * 4) {
    probe_load_t v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = i + static_cast<size_t>(u) * 256;
      v[u] = probe_load_t{0.f, 0.f, 0.f, 0.f};
      if (j < end) v[u] = NT ? __builtin_nontemporal_load(data + j) : data[j];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc += v[u].x + v[u].y + v[u].z + v[u].w;
  }
  // the sum is stored only for a value that random data does not give: the loads stay, the
  // store does not happen
  if (acc == 123456.789f) sink[0] = acc;
}

// Four independent accumulator tiles per wave, so that one v_mfma_f32_16x16x32_bf16 can
// issue while the three before it are in flight; operands stay in registers.
__global__ __launch_bounds__(256) void probe_mfma_bf16_kernel(int iterations, float* __restrict__ sink) {
  probe_bf16x8_t a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = static_cast<__bf16>(static_cast<float>((threadIdx.x + i) % 7) * 0.125f);
    b[i] = static_cast<__bf16>(static_cast<float>((threadIdx.x + 3 * i) % 5) * 0.25f);
  }
  probe_f32x4_t acc0{0.f, 0.f, 0.f, 0.f}, acc1 = acc0, acc2 = acc0, acc3 = acc0;
  for (int it = 0; it < iterations; it += 16) {
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc1, 0, 0, 0);
      acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc2, 0, 0, 0);
      acc3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc3, 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) s += acc0[i] + acc1[i] + acc2[i] + acc3[i];
  if (s == 123456.789f) sink[0] = s;
}

// Reads `bytes` (a multiple of 16, 16-byte aligned) once with `workgroups` workgroups.
extern "C" int yk_probe_stream_read(const void* data, size_t bytes, int workgroups, int nontemporal, float* sink,
                                    hipStream_t stream) {
  YK_REQUIRE(data && sink, "probe_stream_read: null pointer");
  YK_REQUIRE(bytes % 16 == 0 && reinterpret_cast<uintptr_t>(data) % 16 == 0, "probe_stream_read: needs 16-byte pieces");
  YK_REQUIRE(workgroups >= 1 && workgroups <= (1 << 20), "probe_stream_read: bad workgroup count");
  if (bytes == 0) return 0;
  const probe_load_t* p = static_cast<const probe_load_t*>(data);
  if (nontemporal) probe_stream_read_kernel<true><<<workgroups, 256, 0, stream>>>(p, bytes / 16, sink);
  else probe_stream_read_kernel<false><<<workgroups, 256, 0, stream>>>(p, bytes / 16, sink);
  return yk_check_launch("probe_stream_read");
}

// Issues workgroups * 4 waves * iterations * 4 matrix-core instructions of 16,384 flop each.
extern "C" int yk_probe_mfma_bf16(int workgroups, int iterations, float* sink, hipStream_t stream) {
  YK_REQUIRE(sink, "probe_mfma_bf16: null pointer");
  YK_REQUIRE(workgroups >= 1 && workgroups <= (1 << 20) && iterations >= 16 && iterations % 16 == 0 && iterations <= (1 << 24),
             "probe_mfma_bf16: bad sizes (iterations in sixteens)");
  probe_mfma_bf16_kernel<<<workgroups, 256, 0, stream>>>(iterations, sink);
  return yk_check_launch("probe_mfma_bf16");
}
