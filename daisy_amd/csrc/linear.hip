// Projection of a few activation rows for gfx950: y[m][n] = sum_k x[m][k] * w[n][k].
//
// A decode step multiplies one activation row per sequence with the layer's weight matrices
// (models/daisy/attention.py:119-120, the QKV projection, and :201, the output projection): with
// one to eight rows the work is reading the weights once, and the bound is HBM bandwidth
// (N * K * 2 bytes per call).  A wavefront (a workgroup of its own) owns R consecutive weight rows;
// lane l takes the 16-byte pieces l, l + 64, ... of every row, P pieces per row in flight (P R loads
// of 16 bytes per lane before the first multiply: a matrix of a few MB is requested in one go and the
// call lasts one memory round trip plus the transfer), multiplies them with the matching pieces of the
// activation rows and keeps R x M partial sums; the 64 lanes are summed with cross-lane adds at the end.  Products
// accumulate in fp32 and the result is rounded once to bf16, like a library GEMM with fp32
// accumulation (the order of the sums differs from the library's: results agree to the last bf16
// bit except where the fp32 sums straddle a rounding boundary).
#include "common.h"

namespace daisy {

struct LinearParams {
  const uint16_t* x; int64_t x_sm;
  const uint16_t* w; int64_t w_sn;
  uint16_t* y; int64_t y_sm;
  int N, K;
};

constexpr int kLinearMaxRows = 8;

__device__ __forceinline__ float wave_sum(float x) {
  x = group_sum<32>(x);
  return x + __shfl_xor(x, 32);
}

// M activation rows, R weight rows per wavefront, P 16-byte pieces of every row in flight per lane; one wavefront
// per workgroup.
template <int M, int R, int P>
__global__ __launch_bounds__(64) void linear_rows_kernel(LinearParams p) {
  const int lane = threadIdx.x;
  const int row0 = blockIdx.x * R;
  const int pieces = p.K / 8;

  const uint16_t* wr[R];
#pragma unroll
  for (int r = 0; r < R; ++r) wr[r] = p.w + (int64_t)min(row0 + r, p.N - 1) * p.w_sn;   // rows past the end redo the last one

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.f;

  const u32x4 zero = {0u, 0u, 0u, 0u};
  for (int c = lane; c < pieces; c += 64 * P) {
    u32x4 wv[P][R], xv[P][M];
#pragma unroll
    for (int j = 0; j < P; ++j) {
      const bool live = c + 64 * j < pieces;
#pragma unroll
      for (int m = 0; m < M; ++m)
        xv[j][m] = live ? *reinterpret_cast<const u32x4*>(p.x + m * p.x_sm + 8 * (c + 64 * j)) : zero;
    }
#pragma unroll
    for (int j = 0; j < P; ++j) {
      const bool live = c + 64 * j < pieces;
#pragma unroll
      for (int r = 0; r < R; ++r) wv[j][r] = live ? *reinterpret_cast<const u32x4*>(wr[r] + 8 * (c + 64 * j)) : zero;
    }
#pragma unroll
    for (int j = 0; j < P; ++j) {
      float xf[M][8];
#pragma unroll
      for (int m = 0; m < M; ++m) unpack8(xv[j][m], xf[m]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float wf[8];
        unpack8(wv[j][r], wf);
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[r][m] = fmaf(wf[i], xf[m][i], acc[r][m]);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = wave_sum(acc[r][m]);

  if (lane == 0) {
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (row0 + r < p.N) p.y[m * p.y_sm + row0 + r] = (uint16_t)(pack_bf16x2(acc[r][m], 0.f) & 0xffffu);
  }
}

template <int M, int R, int P>
static void launch_linear(const LinearParams& p, hipStream_t s) {
  hipLaunchKernelGGL((linear_rows_kernel<M, R, P>), dim3((p.N + R - 1) / R), dim3(64), 0, s, p);
}

// Rows per wavefront from a sweep (M = 1, 2, 4; N = 768 ... 50304; K = 768 ... 6144): one row -- as many
// wavefronts as the matrix has rows, each with all of its loads in flight at once -- unless several activation
// rows meet a long matrix, where sharing the activation pieces among two or four weight rows wins.
template <int M>
static void launch_linear_rows(const LinearParams& p, hipStream_t s) {
  constexpr int P = M <= 2 ? 4 : 2;
  if (M >= 3 && p.N >= 16384) launch_linear<M, 4, P>(p, s);
  else if ((M == 2 && p.N >= 16384) || (M >= 3 && p.N >= 4096)) launch_linear<M, 2, P>(p, s);
  else launch_linear<M, 1, P>(p, s);
}

}  // namespace daisy

using namespace daisy;

extern "C" int daisy_linear_rows_fwd(const void* x, int64_t x_row_stride, const void* w, int64_t w_row_stride,
                                     void* y, int64_t y_row_stride, int M, int N, int K, void* stream) {
  DAISY_CHECK_ARG(x && w && y, "linear_rows: x, w and y must be non-NULL");
  DAISY_CHECK_ARG(M >= 1 && N >= 1 && K >= 8, "linear_rows: M=%d, N=%d, K=%d must be positive (K at least 8)", M, N, K);
  DAISY_CHECK_SUPPORTED(M <= kLinearMaxRows, "linear_rows: at most %d activation rows, got %d (use a library GEMM)",
                        kLinearMaxRows, M);
  DAISY_CHECK_SUPPORTED(K % 8 == 0, "linear_rows: K=%d must be a multiple of 8", K);
  DAISY_CHECK_ARG((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 &&
                      x_row_stride % 8 == 0 && w_row_stride % 8 == 0,
                  "linear_rows: rows of x and w must start on 16-byte boundaries (strides %lld, %lld elements)",
                  (long long)x_row_stride, (long long)w_row_stride);
  DAISY_CHECK_ARG(w_row_stride >= K && (M == 1 || (x_row_stride >= K && y_row_stride >= N)),
                  "linear_rows: row strides (%lld, %lld, %lld) shorter than the rows (K=%d, N=%d)",
                  (long long)x_row_stride, (long long)w_row_stride, (long long)y_row_stride, K, N);
  LinearParams p{(const uint16_t*)x, x_row_stride, (const uint16_t*)w, w_row_stride, (uint16_t*)y, y_row_stride, N, K};
  hipStream_t s = (hipStream_t)stream;
  switch (M) {
    case 1: launch_linear_rows<1>(p, s); break;
    case 2: launch_linear_rows<2>(p, s); break;
    case 3: launch_linear_rows<3>(p, s); break;
    case 4: launch_linear_rows<4>(p, s); break;
    case 5: launch_linear_rows<5>(p, s); break;
    case 6: launch_linear_rows<6>(p, s); break;
    case 7: launch_linear_rows<7>(p, s); break;
    default: launch_linear_rows<8>(p, s); break;
  }
  DAISY_CHECK_LAUNCH("linear_rows_kernel");
  return DAISY_OK;
}
