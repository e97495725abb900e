// Kernel 3: chunked Kimi Delta Attention forward and its log-decay gate (gfx950).
#include "common.h"

namespace daisy {

// out = -exp(A_log[h]) * softplus(g + bias[h, d]); one thread per element.
template <bool BF16>
__global__ __launch_bounds__(256) void kda_gate_kernel(const void* g, const float* A_log, const float* bias, void* out,
                                                       int64_t total, int H, int Dk, float sp_beta, float threshold) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int d = i % Dk;
  const int h = (i / Dk) % H;
  float x = BF16 ? bf16lo_to_f32(((const uint16_t*)g)[i]) : ((const float*)g)[i];
  if (bias != nullptr) x += bias[h * Dk + d];
  const float bx = x * sp_beta;
  const float sp = (bx > threshold) ? x : log1pf(expf(bx)) / sp_beta;
  const float y = -expf(A_log[h]) * sp;
  if (BF16) ((uint16_t*)out)[i] = (uint16_t)(pack_bf16x2(y, 0.f) & 0xffffu);
  else ((float*)out)[i] = y;
}

}  // namespace daisy

using namespace daisy;

extern "C" int daisy_kda_gate_fwd(const void* g, const float* A_log, const float* bias, void* out,
                                  int64_t rows, int H, int Dk, int io_is_bf16,
                                  float softplus_beta, float threshold, void* stream) {
  DAISY_CHECK_ARG(g && A_log && out, "kda_gate: g, A_log and out must be non-NULL");
  DAISY_CHECK_ARG(rows >= 0 && H > 0 && Dk > 0, "kda_gate: rows=%lld, H=%d, Dk=%d invalid", (long long)rows, H, Dk);
  DAISY_CHECK_ARG(softplus_beta > 0.f, "kda_gate: softplus beta must be positive");
  const int64_t total = rows * H * Dk;
  if (total == 0) return DAISY_OK;
  const int64_t nblk = (total + 255) / 256;
  DAISY_CHECK_ARG(nblk <= 0x7fffffff, "kda_gate: too many elements");
  hipStream_t s = (hipStream_t)stream;
  if (io_is_bf16)
    hipLaunchKernelGGL(kda_gate_kernel<true>, dim3((unsigned)nblk), dim3(256), 0, s, g, A_log, bias, out, total, H, Dk, softplus_beta, threshold);
  else
    hipLaunchKernelGGL(kda_gate_kernel<false>, dim3((unsigned)nblk), dim3(256), 0, s, g, A_log, bias, out, total, H, Dk, softplus_beta, threshold);
  DAISY_CHECK_LAUNCH("kda_gate_kernel");
  return DAISY_OK;
}

extern "C" size_t daisy_kda_workspace_bytes(int B, int T, int H, int Dk, int Dv, int chunk) {
  (void)B; (void)T; (void)H; (void)Dk; (void)Dv; (void)chunk;
  return 0;
}

extern "C" int daisy_kda_chunk_fwd(const void* q, const void* k, const void* v,
                                   const void* g, int g_is_bf16, const float* beta,
                                   const float* initial_state, void* o, float* final_state,
                                   int B, int T, int H, int Dk, int Dv, int chunk,
                                   float scale, int l2norm_qk, float l2_eps,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  set_error("kda_chunk_fwd: not built yet");
  return DAISY_ERR_UNSUPPORTED;
}
