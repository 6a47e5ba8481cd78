// Diagnostic: what the matrix pipe sustains on this GPU with nothing else going on.  Every wave issues `iters` rounds of
// four independent v_mfma_f32_32x32x16_bf16 on operands held in registers (no LDS, no memory traffic in the loop).  The
// operands come from `src` (1024 floats, e.g. N(0,1) samples) or are all zero when `src` is null: the clock, and with it
// the rate, depends on how much the operand bits toggle.  The caller times the launch; it executes
// grid * 4 waves * iters * 4 * 32768 FLOP.  Used by the benchmark to state the ceiling its roofline fractions are up against.
#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void probe_mfma_kernel(const float* __restrict__ src,
                                                                                         float* __restrict__ sink, int iters) {
  bf16x8 a, b;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    a[t] = (__bf16)(src ? src[(threadIdx.x * 8 + t) & 1023] : 0.f);
    b[t] = (__bf16)(src ? src[(threadIdx.x * 3 + t + 517) & 1023] : 0.f);
  }
  f32x16 c0, c1, c2, c3;
#pragma unroll
  for (int r = 0; r < 16; ++r) { c0[r] = 0.f; c1[r] = 0.f; c2[r] = 0.f; c3[r] = 0.f; }
  for (int i = 0; i < iters; ++i) {
    c0 = mfma32(a, b, c0);
    c1 = mfma32(a, b, c1);
    c2 = mfma32(a, b, c2);
    c3 = mfma32(a, b, c3);
  }
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) s += c0[r] + c1[r] + c2[r] + c3[r];
  sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// Diagnostic: what a kernel that only reads can pull from device memory.  Every lane keeps eight 16-byte loads with the
// streaming hint in flight and folds them into one word; `sink` is written only if that word has an unlikely value, so
// the loop cannot be dropped.  The caller times the launch over a buffer much larger than the caches.
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void probe_read_kernel(const u32x4* __restrict__ src, int64_t n_vec,
                                                                                         uint32_t* __restrict__ sink) {
  constexpr int kInFlight = 8;
  u32x4 acc = {0, 0, 0, 0};
  const int64_t stride = (int64_t)gridDim.x * 256 * kInFlight;
  for (int64_t i = (int64_t)blockIdx.x * 256 * kInFlight + threadIdx.x; i + 256 * (kInFlight - 1) < n_vec; i += stride) {
    u32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) v[u] = __builtin_nontemporal_load(src + i + 256 * u);
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) acc ^= v[u];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5eed1e55u) sink[0] = 1;
}

hipError_t launch_probe_read(const void* src, int64_t bytes, uint32_t* sink, int work_groups, hipStream_t stream) {
  hipLaunchKernelGGL(probe_read_kernel, dim3(work_groups), dim3(256), 0, stream, reinterpret_cast<const u32x4*>(src), bytes / 16, sink);
  return hipGetLastError();
}

hipError_t launch_probe_mfma(const float* src, float* sink, int work_groups, int iters, hipStream_t stream) {
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(work_groups), dim3(256), 0, stream, src, sink, iters);
  return hipGetLastError();
}

}  // namespace fba
