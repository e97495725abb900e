// Diagnostic kernels: what the matrix pipe of this chip sustains, with operands in registers only.
//
// Every SIMD of every CU gets two wavefronts that issue independent v_mfma_f32_32x32x16_bf16
// instructions -- alone, or interleaved with vector work in the ratio of the attention inner loop
// (per MFMA: 5 fma and 1 exp2).  No LDS, no memory traffic: the rate is bounded by instruction
// issue and by the clock the power management grants, and is the ceiling against which the
// attention kernel's own rate can be read (the published 2.5 PFLOP/s assumes 2.4 GHz).
#include "common.h"

namespace daisy {

template <int MIX>
__global__ __launch_bounds__(512) void matrix_rate_kernel(float* sink, unsigned long long* ticks, int iters) {
  float a[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = 0.5f + i * 0.001f + threadIdx.x * 1e-5f;
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  bf16x8 x, y;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    x[e] = (__bf16)(0.37f * ((threadIdx.x * 7 + e) % 13) - 2.f);
    y[e] = (__bf16)(0.11f * ((threadIdx.x * 3 + e) % 17) - 1.f);
  }
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[j & 3], 0, 0, 0);
      if (MIX) {
#pragma unroll
        for (int i = 0; i < 5; ++i) a[(j + i) & 7] = fmaf(a[(j + i) & 7], 0.999f, 0.001f);
        a[(j + 5) & 7] = fast_exp2(a[(j + 5) & 7]);
      }
    }
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += a[i];
#pragma unroll
  for (int j = 0; j < 4; ++j) s += acc[j][0];
  sink[(blockIdx.x * 512 + threadIdx.x) & 4095] = s;
  if (threadIdx.x == 0) {
    ticks[2 * blockIdx.x] = c1 - c0;       // shader clock counter
    ticks[2 * blockIdx.x + 1] = r1 - r0;   // constant 100 MHz counter
  }
}

// Read-only streaming: every workgroup sums its contiguous slab of the buffer with 8 x 16 bytes in
// flight per lane (non-temporal loads).  The rate this reaches is the practical ceiling of any
// kernel that only streams from HBM, such as the decode kernel.
__global__ __launch_bounds__(256) void read_rate_kernel(const u32x4* buf, size_t vec_per_wg, uint32_t* sink) {
  const u32x4* p = buf + (size_t)blockIdx.x * vec_per_wg + threadIdx.x;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (size_t i = 0; i < vec_per_wg; i += 256 * 8) {
    u32x4 r[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) r[u] = __builtin_nontemporal_load(p + i + 256 * u);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += r[u];
  }
  // The sum only keeps the loads alive; it is stored when it takes one particular value.
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[blockIdx.x & 4095] = acc.x;
}

}  // namespace daisy

using namespace daisy;

extern "C" int daisy_probe_read_rate(const void* buf, size_t bytes, int workgroups, void* sink, void* stream) {
  DAISY_CHECK_ARG(buf && sink, "probe: buf and sink (4096 x 4 bytes) must be non-NULL");
  DAISY_CHECK_ARG((reinterpret_cast<uintptr_t>(buf) & 15) == 0, "probe: buf must be 16-byte aligned");
  DAISY_CHECK_ARG(workgroups > 0 && bytes > 0 && bytes % ((size_t)workgroups * 256 * 8 * 16) == 0,
                  "probe: bytes=%zu must be a multiple of workgroups (%d) x 32 KiB", bytes, workgroups);
  hipLaunchKernelGGL(read_rate_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const u32x4*>(buf), bytes / 16 / (size_t)workgroups, reinterpret_cast<uint32_t*>(sink));
  DAISY_CHECK_LAUNCH("read_rate_kernel");
  return DAISY_OK;
}

extern "C" int daisy_probe_matrix_rate(int with_vector_mix, int workgroups, int iters,
                                       float* sink, unsigned long long* ticks, double* flop_out, void* stream) {
  DAISY_CHECK_ARG(sink && ticks, "probe: sink (4096 floats) and ticks (2 per workgroup) must be non-NULL");
  DAISY_CHECK_ARG(workgroups > 0 && iters > 0, "probe: workgroups=%d, iters=%d must be positive", workgroups, iters);
  hipStream_t s = (hipStream_t)stream;
  if (with_vector_mix) hipLaunchKernelGGL(matrix_rate_kernel<1>, dim3(workgroups), dim3(512), 0, s, sink, ticks, iters);
  else hipLaunchKernelGGL(matrix_rate_kernel<0>, dim3(workgroups), dim3(512), 0, s, sink, ticks, iters);
  DAISY_CHECK_LAUNCH("matrix_rate_kernel");
  if (flop_out) *flop_out = (double)workgroups * 8.0 * iters * 8.0 * 32768.0;   // 8 wavefronts x 8 MFMA x 2*32*32*16
  return DAISY_OK;
}
