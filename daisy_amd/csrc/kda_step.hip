// Token-by-token Kimi Delta Attention for decode (and short prompts) on gfx950.
//
// The recurrence of the chunked kernel, one token at a time with the fp32 state held in
// registers for the whole call:
//     S <- diag(exp(g_t)) S;   S <- S + beta_t k_t (v_t - S^T k_t)^T;   o_t = scale * S^T q_t
// This is the "fused_recurrent" mode that models/daisy/attention_kimi.py:70,144 names but does
// not support; a generation loop calls it with T = 1 per step.  At T = 1 the call is bound by
// HBM: it reads and writes the [Dk, Dv] fp32 state of every (batch, head) once (128 KiB each).
//
// Workgroup = one (batch, head) and one slab of 128 value columns (value columns are independent of each
// other; key channels beyond Dk read as zeros, whose state rows stay zero), 4 wavefronts; wavefront w
// owns value columns [32w, 32w+32) of the slab.
// Lane (dq = lane/8, jc = lane%8) holds S[16dq .. 16dq+15][32w+4jc .. +3] as 16 float4: state
// loads and stores are 128-byte row segments, the per-token vectors k, q, exp(g) are 16
// consecutive floats per lane read from LDS, and the two matrix-vector products reduce over the
// 8 dq lanes of a column group with cross-lane moves.
#include "common.h"

namespace daisy {

constexpr int RD = 128;   // key channels and value columns a workgroup works on

struct KdaStepParams {
  const uint16_t* q; const uint16_t* k; const uint16_t* v;
  const void* g; int g_bf16;
  const float* beta;
  const float* s_in; float* s_out;
  uint16_t* o;
  int B, T, H;
  int Dk, Dv;   // the tensors' own widths (Dk <= 128)
  float scale; int l2norm; float l2eps;
  // Packed sequences (B == 1, T = all tokens): workgroup (s, h) walks rows cu[s] .. cu[s+1]-1.
  const int32_t* cu; int n_seq;
};

// Sum over the 8 lanes that share jc (lane bits 3, 4, 5).
__device__ __forceinline__ float sum_over_dq(float x) {
  x = dpp_add<0x128>(x);                 // row_ror 8: lane ^ 8 inside a row of 16
  x += __shfl_xor(x, 16);
  x += __shfl_xor(x, 32);
  return x;
}

__global__ __launch_bounds__(256) void kda_recurrent_kernel(KdaStepParams p) {
  __shared__ __attribute__((aligned(16))) float kf[RD];
  __shared__ __attribute__((aligned(16))) float qf[RD];
  __shared__ __attribute__((aligned(16))) float eg[RD];
  __shared__ float red[2][4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int dq = lane >> 3, jc = lane & 7;
  const int h = blockIdx.x % p.H, b = blockIdx.x / p.H;
  const int col = RD * blockIdx.y + 32 * wave + 4 * jc;     // first of this lane's four value columns
  const bool col_live = col < p.Dv;                         // (Dv is a multiple of 8: four columns are live or dead together)
  const int64_t sbase = ((int64_t)(b * p.H + h) * p.Dk + 16 * dq) * p.Dv + col;

  f32x4 S[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    S[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (p.s_in != nullptr && col_live && 16 * dq + i < p.Dk)
      S[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p.s_in + sbase + (int64_t)i * p.Dv));
  }

  // Token rows of this recurrence on the flattened token axis; bounds read from the device are
  // forced into 0 <= first <= end <= T so that no input can lead outside the tensors.
  int tok0 = b * p.T, tok_end = tok0 + p.T;
  if (p.cu != nullptr) {
    tok0 = min(max(p.cu[b], 0), p.T);
    tok_end = min(max(p.cu[b + 1], tok0), p.T);
  }
  for (int tok = tok0; tok < tok_end; ++tok) {
    const int64_t row = (int64_t)tok * p.H + h;
    // ---- stage k, q (L2-normalised) and exp(g) of this token in LDS ---------
    float kx = 0.f, qx = 0.f;
    if (tid < RD) {
      float gx = 0.f;
      if (tid < p.Dk) {
        kx = bf16lo_to_f32(p.k[row * p.Dk + tid]);
        qx = bf16lo_to_f32(p.q[row * p.Dk + tid]);
        gx = p.g_bf16 ? bf16lo_to_f32(reinterpret_cast<const uint16_t*>(p.g)[row * p.Dk + tid])
                      : reinterpret_cast<const float*>(p.g)[row * p.Dk + tid];
      }
      eg[tid] = __expf(gx);
    }
    if (p.l2norm) {
      float ks = kx * kx, qs = qx * qx;      // zero in wavefronts 2 and 3
#pragma unroll
      for (int m = 1; m < 64; m <<= 1) { ks += __shfl_xor(ks, m); qs += __shfl_xor(qs, m); }
      if (lane == 0) { red[0][wave] = ks; red[1][wave] = qs; }
      __syncthreads();
      const float kn = rsqrtf(red[0][0] + red[0][1] + p.l2eps);
      const float qn = rsqrtf(red[1][0] + red[1][1] + p.l2eps);
      kx *= kn;
      qx *= qn;
    }
    if (tid < RD) { kf[tid] = kx; qf[tid] = qx; }
    u32x2 vraw = {0u, 0u};
    if (col_live) vraw = *reinterpret_cast<const u32x2*>(p.v + row * p.Dv + col);
    const f32x4 v4 = {bf16lo_to_f32(vraw.x), bf16hi_to_f32(vraw.x), bf16lo_to_f32(vraw.y), bf16hi_to_f32(vraw.y)};
    const float beta = p.beta[row];
    __syncthreads();

    // ---- decay, prediction S^T k ------------------------------------------------
    f32x4 pred = {0.f, 0.f, 0.f, 0.f};
    float kk[16];
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4 e4 = *reinterpret_cast<const f32x4*>(&eg[16 * dq + 4 * i4]);
      const f32x4 k4 = *reinterpret_cast<const f32x4*>(&kf[16 * dq + 4 * i4]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * i4 + e;
        kk[i] = k4[e];
        S[i] *= e4[e];
        pred += S[i] * k4[e];
      }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) pred[c] = sum_over_dq(pred[c]);
    const f32x4 delta = (v4 - pred) * beta;

    // ---- rank-one update, read-out S^T q -----------------------------------------
    f32x4 out = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4 q4 = *reinterpret_cast<const f32x4*>(&qf[16 * dq + 4 * i4]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * i4 + e;
        S[i] += delta * kk[i];
        out += S[i] * q4[e];
      }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) out[c] = sum_over_dq(out[c]) * p.scale;
    if (dq == 0 && col_live) {
      u32x2 w = {pack_bf16x2(out[0], out[1]), pack_bf16x2(out[2], out[3])};
      *reinterpret_cast<u32x2*>(p.o + row * p.Dv + col) = w;
    }
    __syncthreads();   // kf / qf / eg are rewritten by the next token
  }

  if (p.s_out != nullptr && col_live) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (16 * dq + i < p.Dk) __builtin_nontemporal_store(S[i], reinterpret_cast<f32x4*>(p.s_out + sbase + (int64_t)i * p.Dv));
  }
}

}  // namespace daisy

using namespace daisy;

// Shared by the two entry points.  cu_seqlens == NULL: B sequences of T tokens each; otherwise
// B sequences packed into T tokens in all.
static int recurrent_launch(const void* q, const void* k, const void* v,
                            const void* g, int g_is_bf16, const float* beta, const int32_t* cu_seqlens,
                            const float* initial_state, void* o, float* final_state,
                            int B, int T, int H, int Dk, int Dv,
                            float scale, int l2norm_qk, float l2_eps, void* stream) {
  DAISY_CHECK_SUPPORTED(Dk >= 8 && Dk <= RD && Dk % 8 == 0 && Dv >= 8 && Dv % 8 == 0,
                        "kda_recurrent: Dk=%d, Dv=%d not supported (Dk: a multiple of 8 up to %d; Dv: a multiple of 8)", Dk, Dv, RD);
  DAISY_CHECK_ARG(q && k && v && g && beta && o, "kda_recurrent: q, k, v, g, beta and o must be non-NULL");
  DAISY_CHECK_ARG(B > 0 && T > 0 && H > 0, "kda_recurrent: B=%d, T=%d, H=%d must be positive", B, T, H);
  DAISY_CHECK_ARG((int64_t)B * H <= 0x7fffffff && (int64_t)B * T <= 0x7fffffff, "kda_recurrent: B*H or B*T too large");
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(al16(o) && al16(v) && al16(initial_state) && al16(final_state), "kda_recurrent: v, o and the states must be 16-byte aligned");
  KdaStepParams p;
  p.q = (const uint16_t*)q; p.k = (const uint16_t*)k; p.v = (const uint16_t*)v;
  p.g = g; p.g_bf16 = g_is_bf16; p.beta = beta;
  p.s_in = initial_state; p.s_out = final_state; p.o = (uint16_t*)o;
  p.B = B; p.T = T; p.H = H; p.Dk = Dk; p.Dv = Dv;
  p.scale = scale; p.l2norm = l2norm_qk; p.l2eps = l2_eps;
  p.cu = cu_seqlens; p.n_seq = cu_seqlens ? B : 0;
  DAISY_CHECK_ARG((Dv + RD - 1) / RD <= 65535, "kda_recurrent: Dv=%d too wide", Dv);
  hipLaunchKernelGGL(kda_recurrent_kernel, dim3((unsigned)(B * H), (unsigned)((Dv + RD - 1) / RD)), dim3(256), 0, (hipStream_t)stream, p);
  DAISY_CHECK_LAUNCH("kda_recurrent_kernel");
  return DAISY_OK;
}

extern "C" int daisy_kda_recurrent_fwd(const void* q, const void* k, const void* v,
                                       const void* g, int g_is_bf16, const float* beta,
                                       const float* initial_state, void* o, float* final_state,
                                       int B, int T, int H, int Dk, int Dv,
                                       float scale, int l2norm_qk, float l2_eps, void* stream) {
  return recurrent_launch(q, k, v, g, g_is_bf16, beta, nullptr, initial_state, o, final_state, B, T, H, Dk, Dv,
                          scale, l2norm_qk, l2_eps, stream);
}

extern "C" int daisy_kda_recurrent_varlen_fwd(const void* q, const void* k, const void* v,
                                              const void* g, int g_is_bf16, const float* beta,
                                              const int32_t* cu_seqlens, int n_seq,
                                              const float* initial_state, void* o, float* final_state,
                                              int T, int H, int Dk, int Dv,
                                              float scale, int l2norm_qk, float l2_eps, void* stream) {
  DAISY_CHECK_ARG(cu_seqlens != nullptr && n_seq >= 1, "kda_recurrent_varlen: cu_seqlens and n_seq >= 1 are required");
  return recurrent_launch(q, k, v, g, g_is_bf16, beta, cu_seqlens, initial_state, o, final_state, n_seq, T, H, Dk, Dv,
                          scale, l2norm_qk, l2_eps, stream);
}
