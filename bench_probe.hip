// Diagnostic kernels: what the matrix pipe of this chip sustains, with operands in registers only.
//
// Every SIMD of every CU gets two wavefronts that issue independent v_mfma_f32_32x32x16_bf16
// instructions -- alone, or interleaved with vector work in the ratio of the attention inner loop
// (per MFMA: 5 fma and 1 exp2).  No LDS, no memory traffic: the rate is bounded by instruction
// issue and by the clock the power management grants, and is the ceiling against which the
// attention kernel's own rate can be read (the published 2.5 PFLOP/s assumes 2.4 GHz).
#include "daisy_amd/csrc/common.h"

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

// Register-only MFMAs whose operands CHANGE from one instruction to the next and hold the caller's data (eight A and
// eight B fragments per lane, loaded once from `data`).  With operands of random bits the multiplier arrays toggle as
// they do on real tensors; with a buffer of zeros or of one repeated value they do not.  The difference between the
// two sustained rates is what the chip's power management takes for the data alone.
template <int VARIANT>   // 0: A and B change with every instruction; 1: B stays the same (A changes); 2: A stays the same (B changes)
__global__ __launch_bounds__(512) void matrix_rate_data_kernel(const u32x4* data, float* sink, unsigned long long* ticks, int iters) {
  bf16x8 xs[8], ys[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    xs[j] = __builtin_bit_cast(bf16x8, data[(size_t)(2 * j) * 512 + threadIdx.x]);
    ys[j] = __builtin_bit_cast(bf16x8, data[(size_t)(2 * j + 1) * 512 + threadIdx.x]);
  }
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xs[VARIANT == 2 ? 0 : j], ys[VARIANT == 1 ? 0 : j], acc[j & 3], 0, 0, 0);
    // keep the sums bounded: the accumulators are cleared every 64 iterations (a handful of vector moves per 512 MFMAs)
    if ((it & 63) == 63) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] *= 0.f;
    }
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) s += acc[j][0];
  sink[(blockIdx.x * 512 + threadIdx.x) & 4095] = s;
  if (threadIdx.x == 0) {
    ticks[2 * blockIdx.x] = c1 - c0;
    ticks[2 * blockIdx.x + 1] = r1 - r0;
  }
}

// The same with the attention loop's LDS operand traffic: per MFMA 3 fma and 1 exp2, and the A operand
// of every MFMA comes from LDS with the kernel's own access patterns -- a 16-byte read of a swizzled
// row-major tile (the K operand) for even MFMAs, two 8-byte transposing reads (the V operand) for
// odd ones -- requested eight MFMAs before its use.  No global memory, no barriers, no masks: the
// rate of this stream is what the layout of prefill_tile_kernel (two or three wavefronts per SIMD) can reach at
// best with its instruction mix.
typedef short probe_s16x4 __attribute__((ext_vector_type(4)));
// data: NULL, or 64 x 128 + 512 x 8 bf16 values that fill the LDS tile and the B operands (N(0,1) values make the
// operand bits toggle as they do on real tensors; without it the tile holds a few repeated values).
__global__ __launch_bounds__(512) void attention_mix_kernel(const uint16_t* data, float* sink, unsigned long long* ticks, int iters) {
  __shared__ __attribute__((aligned(1024))) uint16_t tile[64 * 128];
  for (int i = threadIdx.x; i < 64 * 128; i += 512) tile[i] = data ? data[i] : (uint16_t)(0x3c00 + (i & 63));
  __syncthreads();
  const int lane = threadIdx.x & 63, lq = lane & 31, lh = lane >> 5;
  typedef __attribute__((address_space(3))) const uint16_t* lptr;
  // K pattern: row lq of a 32-row block, 16-byte chunk (2s + lh) ^ (lq & 15), s = 0..7 by immediate.
  lptr kp[2];
  kp[0] = (lptr)&tile[0] + lq * 128 + 8 * ((0 + lh) ^ (lq & 15));
  kp[1] = (lptr)&tile[0] + lq * 128 + 8 * ((2 + lh) ^ (lq & 15));
  // V pattern: lane i of a block of 16 addresses key i/4, channels 4*(i%4)..+3.
  const int i16 = lane & 15, vrow = 4 * lh + (i16 >> 2);
  lptr vp = (lptr)&tile[0] + vrow * 128 + 8 * ((2 * ((lane >> 4) & 1) + ((i16 & 3) >> 1)) ^ (4 * (vrow & 3))) + 4 * (i16 & 1);
  auto read_operand = [&](int j) -> bf16x8 {
    if ((j & 1) == 0) {
      return __builtin_bit_cast(bf16x8, *(const u32x4 __attribute__((address_space(3)))*)(kp[(j >> 1) & 1] + 32 * 128 * ((j >> 2) & 1)));
    } else {
      const probe_s16x4 a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((probe_s16x4 __attribute__((address_space(3)))*)(vp + 16 * 128 * (j >> 1)));
      const probe_s16x4 a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((probe_s16x4 __attribute__((address_space(3)))*)(vp + 16 * 128 * (j >> 1) + 8 * 128));
      const u32x2 b0 = __builtin_bit_cast(u32x2, a0), b1 = __builtin_bit_cast(u32x2, a1);
      const u32x4 av = {b0.x, b0.y, b1.x, b1.y};
      return __builtin_bit_cast(bf16x8, av);
    }
  };
  float a[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = 0.5f + i * 0.001f + threadIdx.x * 1e-5f;
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  bf16x8 y;
#pragma unroll
  for (int e = 0; e < 8; ++e) y[e] = (__bf16)(0.11f * ((threadIdx.x * 3 + e) % 17) - 1.f);
  if (data) y = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(data + 64 * 128 + 8 * threadIdx.x));
  bf16x8 opa[8], opb[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) opa[j] = read_operand(j);
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  auto block = [&](bf16x8* use, bf16x8* fill) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      fill[j] = read_operand(j);
      acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(use[j], y, acc[j & 3], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 3; ++i) a[(j + i) & 7] = fmaf(a[(j + i) & 7], 0.999f, 0.001f);
      a[(j + 3) & 7] = fast_exp2(a[(j + 3) & 7]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  for (int it = 0; it < iters; it += 2) {
    block(opa, opb);
    block(opb, opa);
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += a[i];
#pragma unroll
  for (int j = 0; j < 4; ++j) s += acc[j][0];
  sink[(blockIdx.x * 512 + threadIdx.x) & 4095] = s;
  if (threadIdx.x == 0) {
    ticks[2 * blockIdx.x] = c1 - c0;
    ticks[2 * blockIdx.x + 1] = r1 - r0;
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

extern "C" int daisy_probe_matrix_rate_data(const void* data, size_t data_bytes, int variant, int workgroups, int iters,
                                            float* sink, unsigned long long* ticks, double* flop_out, void* stream) {
  DAISY_CHECK_ARG(data && sink && ticks, "probe: data, sink (4096 floats) and ticks (2 per workgroup) must be non-NULL");
  DAISY_CHECK_ARG(data_bytes >= 16 * 512 * 16 && (reinterpret_cast<uintptr_t>(data) & 15) == 0,
                  "probe: data must hold 16 x 512 x 16 bytes, 16-byte aligned");
  DAISY_CHECK_ARG(workgroups > 0 && iters > 0, "probe: workgroups=%d, iters=%d must be positive", workgroups, iters);
  const u32x4* d = reinterpret_cast<const u32x4*>(data);
  hipStream_t s = (hipStream_t)stream;
  if (variant == 3) {   // the attention loop's mix: vector work and LDS operand reads next to the MFMAs, on the caller's data
    iters = (iters + 1) & ~1;
    hipLaunchKernelGGL(attention_mix_kernel, dim3(workgroups), dim3(512), 0, s, reinterpret_cast<const uint16_t*>(data), sink, ticks, iters);
  } else if (variant == 1) hipLaunchKernelGGL(matrix_rate_data_kernel<1>, dim3(workgroups), dim3(512), 0, s, d, sink, ticks, iters);
  else if (variant == 2) hipLaunchKernelGGL(matrix_rate_data_kernel<2>, dim3(workgroups), dim3(512), 0, s, d, sink, ticks, iters);
  else hipLaunchKernelGGL(matrix_rate_data_kernel<0>, dim3(workgroups), dim3(512), 0, s, d, sink, ticks, iters);
  DAISY_CHECK_LAUNCH("matrix_rate_data_kernel");
  if (flop_out) *flop_out = (double)workgroups * 8.0 * iters * 8.0 * 32768.0;
  return DAISY_OK;
}

extern "C" int daisy_probe_matrix_rate(int with_vector_mix, int workgroups, int iters,
                                       float* sink, unsigned long long* ticks, double* flop_out, void* stream) {
  DAISY_CHECK_ARG(sink && ticks, "probe: sink (4096 floats) and ticks (2 per workgroup) must be non-NULL");
  DAISY_CHECK_ARG(workgroups > 0 && iters > 0, "probe: workgroups=%d, iters=%d must be positive", workgroups, iters);
  hipStream_t s = (hipStream_t)stream;
  if (with_vector_mix == 2) hipLaunchKernelGGL(attention_mix_kernel, dim3(workgroups), dim3(512), 0, s, (const uint16_t*)nullptr, sink, ticks, (iters + 1) & ~1);
  else if (with_vector_mix) hipLaunchKernelGGL(matrix_rate_kernel<1>, dim3(workgroups), dim3(512), 0, s, sink, ticks, iters);
  else hipLaunchKernelGGL(matrix_rate_kernel<0>, dim3(workgroups), dim3(512), 0, s, sink, ticks, iters);
  DAISY_CHECK_LAUNCH("matrix_rate_kernel");
  if (with_vector_mix == 2) iters = (iters + 1) & ~1;
  if (flop_out) *flop_out = (double)workgroups * 8.0 * iters * 8.0 * 32768.0;   // 8 wavefronts x 8 MFMA x 2*32*32*16
  return DAISY_OK;
}
