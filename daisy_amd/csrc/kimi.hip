// Streaming kernels of the KDA layer around the delta-rule core (gfx950).
//
// models/daisy/attention_kimi.py:155-158,136-137 puts three depthwise short convolutions
// (q, k, v: 4 taps, causal, SiLU) in front of chunk_kda and a gated RMS norm behind it; both
// come from a package that is absent from the reference checkout, so what is restated here is
// their documented arithmetic:
//   conv :  y[t, c] = silu( bias[c] + sum_j w[c, j] * x[t - (K-1) + j, c] ),  x[<0] from the
//           carried window (the last K-1 inputs of the previous call) or zero
//   norm :  out = x * rsqrt(mean(x^2) + eps) * weight * sigmoid(gate)      over the last dim
// Both are one pass over their tensors: 16-byte loads and stores, no LDS.
#include "common.h"

namespace daisy {

struct ConvParams {
  const uint16_t* x; int64_t x_sb, x_st;       // [B, T, C], channel stride 1
  const uint16_t* w;                           // [C, K]
  const uint16_t* bias;                        // [C] or null
  const uint16_t* cache_in;                    // [B, C, K] or null: the last K inputs before t = 0 (the first is unused)
  uint16_t* y; int64_t y_sb, y_st;             // [B, T, C]
  uint16_t* cache_out;                         // [B, C, K] or null: the last K inputs of the extended sequence
  int B, T, C, silu;
};

constexpr int kConvSeg = 32;   // time steps per thread

// A thread owns 8 consecutive channels and kConvSeg consecutive time steps; the K-1 inputs
// before its first step come from the sequence itself or from the carried window.  The sum is
// taken in fp32 and rounded to bf16 before the activation, which is again evaluated in fp32 and
// rounded (the two roundings of a bf16 convolution followed by a bf16 SiLU).
template <int K>
__global__ __launch_bounds__(256) void short_conv_kernel(ConvParams p) {
  const int cg = blockIdx.x * 256 + threadIdx.x;        // group of 8 channels
  const int c0 = 8 * cg;
  if (c0 >= p.C) return;
  const int b = blockIdx.z;
  const int t0 = blockIdx.y * kConvSeg;
  const int t1 = min(t0 + kConvSeg, p.T);

  float w[K][8], acc0[8];
  {
    // channel c's taps are K consecutive values; 8 channels = 8K consecutive bf16
    const uint16_t* wp = p.w + (int64_t)c0 * K;
    if (K == 4) {   // 64 contiguous bytes: four 16-byte loads, two channels each
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float f[8];
        unpack8(*reinterpret_cast<const u32x4*>(wp + 8 * v), f);
#pragma unroll
        for (int j = 0; j < K; ++j) { w[j][2 * v] = f[j % 8]; w[j][2 * v + 1] = f[(4 + j) % 8]; }
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int j = 0; j < K; ++j) w[j][e] = bf16lo_to_f32(wp[e * K + j]);
    }
    if (p.bias != nullptr) unpack8(*reinterpret_cast<const u32x4*>(p.bias + c0), acc0);
    else {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc0[e] = 0.f;
    }
  }
  // The carried window of 8 channels is 8K contiguous values; for K = 4 it is read and written
  // as four 16-byte pieces (two channels each).
  float carried[K][8];
  if (K == 4 && p.cache_in != nullptr && t0 < K - 1) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float f[8];
      unpack8(*reinterpret_cast<const u32x4*>(p.cache_in + ((int64_t)b * p.C + c0) * K + 8 * v), f);
#pragma unroll
      for (int j = 0; j < K; ++j) { carried[j][2 * v] = f[j % 8]; carried[j][2 * v + 1] = f[(4 + j) % 8]; }
    }
  }
  // Input at time ti (may be negative: carried window or zero).
  auto input_at = [&](int ti, float* f) {
    if (ti >= 0) {
      unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.x + b * p.x_sb + (int64_t)ti * p.x_st + c0)), f);
    } else if (p.cache_in != nullptr) {
      if (K == 4) {
#pragma unroll
        for (int j = 1; j < K; ++j)
          if (K + ti == j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = carried[j][e];
          }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = bf16lo_to_f32(p.cache_in[((int64_t)b * p.C + c0 + e) * K + K + ti]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = 0.f;
    }
  };

  float win[K - 1][8];   // win[j] = input at t - (K-1) + j for the step t about to be computed
#pragma unroll
  for (int j = 0; j < K - 1; ++j) input_at(t0 - (K - 1) + j, win[j]);
  constexpr int U = 8;   // steps whose inputs are in flight together
  for (int tb = t0; tb < t1; tb += U) {
    u32x4 raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = min(tb + u, p.T - 1);   // steps past the end re-read the last row and are not stored
      raw[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.x + b * p.x_sb + (int64_t)t * p.x_st + c0));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float xin[8], out[8];
      unpack8(raw[u], xin);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float a = acc0[e];
#pragma unroll
        for (int j = 0; j < K - 1; ++j) a = fmaf(w[j][e], win[j][e], a);
        a = round_bf16(fmaf(w[K - 1][e], xin[e], a));
        if (p.silu) a = a * __builtin_amdgcn_rcpf(1.f + __expf(-a));
        out[e] = a;
      }
      if (tb + u < t1) *reinterpret_cast<u32x4*>(p.y + b * p.y_sb + (int64_t)(tb + u) * p.y_st + c0) = pack8(out);
#pragma unroll
      for (int j = 0; j + 1 < K - 1; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) win[j][e] = win[j + 1][e];
#pragma unroll
      for (int e = 0; e < 8; ++e) win[K - 2][e] = xin[e];
    }
  }
  // The thread that reaches the end of the sequence leaves the window for the next call.
  if (p.cache_out != nullptr && t1 == p.T) {
    float last[K][8];
#pragma unroll
    for (int j = 0; j < K; ++j) input_at(p.T - K + j, last[j]);
    if (K == 4) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float f[8];
#pragma unroll
        for (int j = 0; j < K; ++j) { f[j % 8] = last[j][2 * v]; f[(4 + j) % 8] = last[j][2 * v + 1]; }
        *reinterpret_cast<u32x4*>(p.cache_out + ((int64_t)b * p.C + c0) * K + 8 * v) = pack8(f);
      }
    } else {
#pragma unroll
      for (int j = 0; j < K; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          p.cache_out[((int64_t)b * p.C + c0 + e) * K + j] = (uint16_t)(pack_bf16x2(last[j][e], 0.f) & 0xffffu);
    }
  }
}

// Sequences packed along T of a batch of one: the taps of a step must not reach across the start of
// the step's sequence (they read the sequence's carried window [n_seq, C, K] or zero instead), and
// every sequence leaves its own window.  The bounds cu [n_seq + 1] are read on the device and forced
// into 0..T; a thread finds the sequence of its first step by bisection and walks on from there.
// Taps are re-read from global memory (they hit the cache) instead of kept in registers, which keeps
// the boundary handling in one place.
template <int K>
__global__ __launch_bounds__(256) void short_conv_varlen_kernel(ConvParams p, const int32_t* cu, int n_seq) {
  const int cg = blockIdx.x * 256 + threadIdx.x;
  const int c0 = 8 * cg;
  if (c0 >= p.C) return;
  const int t0 = blockIdx.y * kConvSeg;
  const int t1 = min(t0 + kConvSeg, p.T);
  auto bound = [&](int i) { return min(max(cu[i], 0), p.T); };

  float w[K][8], acc0[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int j = 0; j < K; ++j) w[j][e] = bf16lo_to_f32(p.w[(int64_t)(c0 + e) * K + j]);
    acc0[e] = p.bias ? bf16lo_to_f32(p.bias[c0 + e]) : 0.f;
  }
  // Input of sequence `seq` (first row `start`) at row ti; rows before the start come from the window.
  auto input_at = [&](int seq, int start, int ti, float* f) {
    if (ti >= start) {
      unpack8(*reinterpret_cast<const u32x4*>(p.x + (int64_t)ti * p.x_st + c0), f);
    } else {
      const int slot = K + (ti - start);     // window slot: K-1 is the input just before the sequence
#pragma unroll
      for (int e = 0; e < 8; ++e)
        f[e] = (p.cache_in != nullptr && seq < n_seq && slot >= 0) ? bf16lo_to_f32(p.cache_in[((int64_t)seq * p.C + c0 + e) * K + slot]) : 0.f;
    }
  };
  auto leave_window = [&](int seq, int start, int end) {
#pragma unroll
    for (int j = 0; j < K; ++j) {
      float f[8];
      input_at(seq, start, end - K + j, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) p.cache_out[((int64_t)seq * p.C + c0 + e) * K + j] = (uint16_t)(pack_bf16x2(f[e], 0.f) & 0xffffu);
    }
  };

  // smallest seq in [0, n_seq] whose end lies beyond t0 (n_seq: rows behind the last bound, a sequence
  // of their own without a window)
  int lo = 0, hi = n_seq;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (bound(mid + 1) > t0) hi = mid; else lo = mid + 1;
  }
  int seq = lo;
  int start = bound(min(seq, n_seq)), end = seq < n_seq ? bound(seq + 1) : p.T;
  for (int t = t0; t < t1; ++t) {
    while (t >= end && seq < n_seq) {
      ++seq;
      start = bound(min(seq, n_seq));
      end = seq < n_seq ? bound(seq + 1) : p.T;
    }
    float a[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = acc0[e];
#pragma unroll
    for (int j = 0; j < K; ++j) {
      float f[8];
      input_at(seq, start, t - (K - 1) + j, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) a[e] = fmaf(w[j][e], f[e], a[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[e] = round_bf16(a[e]);
      if (p.silu) a[e] = a[e] * __builtin_amdgcn_rcpf(1.f + __expf(-a[e]));
    }
    *reinterpret_cast<u32x4*>(p.y + (int64_t)t * p.y_st + c0) = pack8(a);
    if (p.cache_out != nullptr && seq < n_seq && t == end - 1) leave_window(seq, start, end);
  }
  // Empty sequences keep their window; the threads of the first time segment see to it.
  if (p.cache_out != nullptr && blockIdx.y == 0) {
    for (int i = 0; i < n_seq; ++i) {
      const int b0 = bound(i), b1 = bound(i + 1);
      if (b1 <= b0) leave_window(i, b0, b0);
    }
  }
}

struct GatedNormParams {
  const uint16_t* x; const uint16_t* gate; const uint16_t* weight; uint16_t* out;
  int64_t rows; float eps;
};

// D/8 lanes share a row; statistics in fp32 over the row, one rounding at the end.
template <int D>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(GatedNormParams p) {
  constexpr int LPR = D / 8;
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  const int c = threadIdx.x % LPR;
  const int64_t r = row < p.rows ? row : p.rows - 1;   // surplus lanes redo the last row (the sums need full groups)
  float x[8], g[8], w[8], o[8];
  unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.x + r * D + 8 * c)), x);
  unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.gate + r * D + 8 * c)), g);
  unpack8(*reinterpret_cast<const u32x4*>(p.weight + 8 * c), w);
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss = fmaf(x[e], x[e], ss);
  ss = group_sum<LPR>(ss);
  const float rstd = rsqrtf(ss / (float)D + p.eps);
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = x[e] * rstd * w[e] * __builtin_amdgcn_rcpf(1.f + __expf(-g[e]));
  if (row < p.rows) *reinterpret_cast<u32x4*>(p.out + r * D + 8 * c) = pack8(o);
}

}  // namespace daisy

using namespace daisy;

extern "C" int daisy_short_conv_fwd(const void* x, const int64_t* x_strides, const void* weight, const void* bias,
                                    const void* cache_in, void* y, const int64_t* y_strides, void* cache_out,
                                    int B, int T, int C, int K, int apply_silu, void* stream) {
  DAISY_CHECK_ARG(x && weight && y && x_strides && y_strides, "short_conv: x, weight, y and the stride arrays must be non-NULL");
  DAISY_CHECK_ARG(B > 0 && T > 0 && C > 0, "short_conv: B=%d, T=%d, C=%d must be positive", B, T, C);
  DAISY_CHECK_SUPPORTED(K >= 2 && K <= 4, "short_conv: kernel size %d not supported (2..4)", K);
  DAISY_CHECK_SUPPORTED(C % 8 == 0, "short_conv: channels (%d) must be a multiple of 8", C);
  DAISY_CHECK_ARG(B <= 65535, "short_conv: B must be <= 65535");
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(al16(x) && al16(y) && al16(bias) && al16(weight) && al16(cache_in) && al16(cache_out),
                  "short_conv: x, y, weight, bias and the windows must be 16-byte aligned");
  for (int i = 0; i < 2; ++i)
    DAISY_CHECK_ARG(x_strides[i] % 8 == 0 && y_strides[i] % 8 == 0, "short_conv: strides must be multiples of 8 elements");
  // Updating the window in place is safe only while the thread that writes it is the one that read it.
  DAISY_CHECK_ARG(cache_out == nullptr || cache_out != cache_in || T <= kConvSeg,
                  "short_conv: the window can be updated in place for T <= %d only (T=%d)", kConvSeg, T);
  ConvParams p;
  p.x = (const uint16_t*)x; p.x_sb = x_strides[0]; p.x_st = x_strides[1];
  p.w = (const uint16_t*)weight; p.bias = (const uint16_t*)bias; p.cache_in = (const uint16_t*)cache_in;
  p.y = (uint16_t*)y; p.y_sb = y_strides[0]; p.y_st = y_strides[1];
  p.cache_out = (uint16_t*)cache_out;
  p.B = B; p.T = T; p.C = C; p.silu = apply_silu;
  const dim3 grid((unsigned)((C / 8 + 255) / 256), (unsigned)((T + kConvSeg - 1) / kConvSeg), (unsigned)B);
  DAISY_CHECK_ARG(grid.y <= 65535, "short_conv: T=%d too long for one launch", T);
  hipStream_t s = (hipStream_t)stream;
  if (K == 4) hipLaunchKernelGGL(short_conv_kernel<4>, grid, dim3(256), 0, s, p);
  else if (K == 3) hipLaunchKernelGGL(short_conv_kernel<3>, grid, dim3(256), 0, s, p);
  else hipLaunchKernelGGL(short_conv_kernel<2>, grid, dim3(256), 0, s, p);
  DAISY_CHECK_LAUNCH("short_conv_kernel");
  return DAISY_OK;
}

extern "C" int daisy_short_conv_varlen_fwd(const void* x, int64_t x_row_stride, const void* weight, const void* bias,
                                           const int32_t* cu_seqlens, int n_seq, const void* cache_in,
                                           void* y, int64_t y_row_stride, void* cache_out,
                                           int T, int C, int K, int apply_silu, void* stream) {
  DAISY_CHECK_ARG(x && weight && y, "short_conv_varlen: x, weight and y must be non-NULL");
  DAISY_CHECK_ARG(cu_seqlens != nullptr && n_seq >= 1, "short_conv_varlen: cu_seqlens and n_seq >= 1 are required");
  DAISY_CHECK_ARG(T > 0 && C > 0, "short_conv_varlen: T=%d, C=%d must be positive", T, C);
  DAISY_CHECK_SUPPORTED(K >= 2 && K <= 4, "short_conv_varlen: kernel size %d not supported (2..4)", K);
  DAISY_CHECK_SUPPORTED(C % 8 == 0, "short_conv_varlen: channels (%d) must be a multiple of 8", C);
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(al16(x) && al16(y) && x_row_stride % 8 == 0 && y_row_stride % 8 == 0,
                  "short_conv_varlen: x and y must be 16-byte aligned with row strides that are multiples of 8 elements");
  DAISY_CHECK_ARG(cache_out == nullptr || cache_out != cache_in, "short_conv_varlen: the windows cannot be updated in place");
  ConvParams p;
  p.x = (const uint16_t*)x; p.x_sb = 0; p.x_st = x_row_stride;
  p.w = (const uint16_t*)weight; p.bias = (const uint16_t*)bias; p.cache_in = (const uint16_t*)cache_in;
  p.y = (uint16_t*)y; p.y_sb = 0; p.y_st = y_row_stride;
  p.cache_out = (uint16_t*)cache_out;
  p.B = 1; p.T = T; p.C = C; p.silu = apply_silu;
  const dim3 grid((unsigned)((C / 8 + 255) / 256), (unsigned)((T + kConvSeg - 1) / kConvSeg), 1);
  DAISY_CHECK_ARG(grid.y <= 65535, "short_conv_varlen: T=%d too long for one launch", T);
  hipStream_t s = (hipStream_t)stream;
  if (K == 4) hipLaunchKernelGGL(short_conv_varlen_kernel<4>, grid, dim3(256), 0, s, p, cu_seqlens, n_seq);
  else if (K == 3) hipLaunchKernelGGL(short_conv_varlen_kernel<3>, grid, dim3(256), 0, s, p, cu_seqlens, n_seq);
  else hipLaunchKernelGGL(short_conv_varlen_kernel<2>, grid, dim3(256), 0, s, p, cu_seqlens, n_seq);
  DAISY_CHECK_LAUNCH("short_conv_varlen_kernel");
  return DAISY_OK;
}

extern "C" int daisy_gated_rmsnorm_fwd(const void* x, const void* gate, const void* weight, void* out,
                                       int64_t rows, int D, float eps, void* stream) {
  DAISY_CHECK_ARG(x && gate && weight && out, "gated_rmsnorm: x, gate, weight and out must be non-NULL");
  DAISY_CHECK_ARG(rows > 0, "gated_rmsnorm: rows=%lld must be positive", (long long)rows);
  DAISY_CHECK_SUPPORTED(D == 32 || D == 64 || D == 128 || D == 256, "gated_rmsnorm: last dim %d not supported (32, 64, 128 or 256)", D);
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(al16(x) && al16(gate) && al16(weight) && al16(out), "gated_rmsnorm: tensors must be 16-byte aligned");
  GatedNormParams p;
  p.x = (const uint16_t*)x; p.gate = (const uint16_t*)gate; p.weight = (const uint16_t*)weight; p.out = (uint16_t*)out;
  p.rows = rows; p.eps = eps;
  const int64_t nwg = (rows * (D / 8) + 255) / 256;
  DAISY_CHECK_ARG(nwg <= 0x7fffffff, "gated_rmsnorm: too many rows (%lld)", (long long)rows);
  hipStream_t s = (hipStream_t)stream;
  if (D == 128) hipLaunchKernelGGL(gated_rmsnorm_kernel<128>, dim3((unsigned)nwg), dim3(256), 0, s, p);
  else if (D == 256) hipLaunchKernelGGL(gated_rmsnorm_kernel<256>, dim3((unsigned)nwg), dim3(256), 0, s, p);
  else if (D == 32) hipLaunchKernelGGL(gated_rmsnorm_kernel<32>, dim3((unsigned)nwg), dim3(256), 0, s, p);
  else hipLaunchKernelGGL(gated_rmsnorm_kernel<64>, dim3((unsigned)nwg), dim3(256), 0, s, p);
  DAISY_CHECK_LAUNCH("gated_rmsnorm_kernel");
  return DAISY_OK;
}
