// Fused pre-attention elementwise pass for gfx950.
//
// One pass over the QKV projection output does what the reference spreads over a dozen
// elementwise kernels (models/daisy/attention.py:116-135):
//   q, k, v = norm(q), norm(k), norm(v)          functional.py:6-7, weightless RMS norm
//   q, k    = rope(q), rope(k)                   attention.py:16-20 at positions pos0 + t
//   v       = g * v + (1 - g) * ve               attention.py:132-135 (only when ve is given)
// Every intermediate is rounded to bf16 where the reference materialises a bf16 tensor (after
// the norm, after each product and the sum of the mix), so the outputs carry the same roundings.
// The pass is pure streaming: 16-byte loads and stores, no LDS, sums inside a group of lanes by
// DPP; it is bound by HBM bandwidth (3 rows in, 3 rows out, plus the ve row, per token and head).
#include "common.h"

namespace daisy {

struct PrepParams {
  const uint16_t* q; int64_t q_sb, q_st, q_sh;
  const uint16_t* k; int64_t k_sb, k_st, k_sh;
  const uint16_t* v; int64_t v_sb, v_st, v_sh;
  const uint16_t* ve; int64_t e_sb, e_st, e_sh;
  const float* gate;
  const float* cos; const float* sin;
  uint16_t* qo; int64_t qo_sb, qo_st, qo_sh;
  uint16_t* ko; int64_t ko_sb, ko_st, ko_sh;
  uint16_t* vo; int64_t vo_sb, vo_st, vo_sh;
  int B, T, H, pos0;
  // When set, the first position is read from device memory at run time (so that a recorded
  // launch can be replayed for later positions) and held inside the table's rows.
  const int32_t* pos0_dev; int table_rows;
  int32_t* status;   // optional: receives DAISY_STATUS_* bits the kernel raises
  int64_t rows;
  float eps;
};

// One row of D channels is shared by LPR = D/16 lanes; lane c holds channels [8c, 8c+8) and
// their RoPE partners [D/2 + 8c, D/2 + 8c + 8), so the rotation needs no exchange.
template <int D>
__global__ __launch_bounds__(256) void qkv_prep_kernel(PrepParams p) {
  constexpr int LPR = D / 16, HALF = D / 2;
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  const int c = threadIdx.x % LPR;
  // Lanes past the last row redo the last row (same values, same addresses): the cross-lane
  // sums below need every lane of a group to take part.
  const int64_t r = row < p.rows ? row : p.rows - 1;
  const int h = (int)(r % p.H);
  const int64_t bt = r / p.H;
  const int t = (int)(bt % p.T);
  const int64_t b = bt / p.T;

  auto load_row = [&](const uint16_t* base, int64_t sb, int64_t st, int64_t sh, float* lo, float* hi) {
    const uint16_t* src = base + b * sb + t * st + h * sh + 8 * c;
    // streamed once: keep the rows out of the way of the tables in the caches
    const u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src));
    const u32x4 d = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + HALF));
    unpack8(a, lo);
    unpack8(d, hi);
  };
  auto store_row = [&](uint16_t* base, int64_t sb, int64_t st, int64_t sh, const float* lo, const float* hi) {
    uint16_t* dst = base + b * sb + t * st + h * sh + 8 * c;
    *reinterpret_cast<u32x4*>(dst) = pack8(lo);
    *reinterpret_cast<u32x4*>(dst + HALF) = pack8(hi);
  };
  // x * rsqrt(mean(x^2) + eps), rounded to bf16 (the reference's norm output dtype).
  auto rms_normalise = [&](float* lo, float* hi) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += lo[e] * lo[e];
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += hi[e] * hi[e];
    ss = group_sum<LPR>(ss);
    const float rstd = rsqrtf(ss / (float)D + p.eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      lo[e] = round_bf16(lo[e] * rstd);
      hi[e] = round_bf16(hi[e] * rstd);
    }
  };

  float ql[8], qh[8], kl[8], kh[8], vl[8], vh[8], el[8], eh[8];
  load_row(p.q, p.q_sb, p.q_st, p.q_sh, ql, qh);
  load_row(p.k, p.k_sb, p.k_st, p.k_sh, kl, kh);
  load_row(p.v, p.v_sb, p.v_st, p.v_sh, vl, vh);
  if (p.ve != nullptr) load_row(p.ve, p.e_sb, p.e_st, p.e_sh, el, eh);
  float cs[8], sn[8];
  if (p.cos != nullptr) {
    int pos0 = p.pos0;
    bool past_tables = false;
    if (p.pos0_dev != nullptr) {
      // Rows past the rotation tables read the tables' end (memory safety) and are reported: the status
      // word gets its bit and the rotated outputs are NaN.
      const int want = max(0, p.pos0_dev[0]);
      past_tables = want > p.table_rows - p.T;
      pos0 = min(want, p.table_rows - p.T);
      if (past_tables && p.status != nullptr && blockIdx.x == 0 && threadIdx.x == 0)
        __hip_atomic_fetch_or(p.status, DAISY_STATUS_POSITION_PAST_TABLES, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const int64_t off = (int64_t)(pos0 + t) * HALF + 8 * c;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(p.cos + off), c1 = *reinterpret_cast<const f32x4*>(p.cos + off + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(p.sin + off), s1 = *reinterpret_cast<const f32x4*>(p.sin + off + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { cs[e] = c0[e]; cs[4 + e] = c1[e]; sn[e] = s0[e]; sn[4 + e] = s1[e]; }
    if (past_tables) {
#pragma unroll
      for (int e = 0; e < 8; ++e) cs[e] = __builtin_nanf("");
    }
  }

  rms_normalise(ql, qh);
  rms_normalise(kl, kh);
  rms_normalise(vl, vh);

  if (p.cos != nullptr) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float q1 = ql[e], q2 = qh[e], k1 = kl[e], k2 = kh[e];
      ql[e] = rope_lo(q1, q2, cs[e], sn[e]);
      qh[e] = rope_hi(q1, q2, cs[e], sn[e]);
      kl[e] = rope_lo(k1, k2, cs[e], sn[e]);
      kh[e] = rope_hi(k1, k2, cs[e], sn[e]);
    }
  }
  if (p.ve != nullptr) {
    // g*v + (1-g)*ve the way a bf16 tensor library evaluates it: each product, the
    // difference and the sum are separate bf16 results.
    const float g = p.gate[0];
    const float og = round_bf16(1.0f - g);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      vl[e] = round_bf16(g * vl[e]) + round_bf16(og * el[e]);
      vh[e] = round_bf16(g * vh[e]) + round_bf16(og * eh[e]);
    }
  }
  if (row < p.rows) {
    store_row(p.qo, p.qo_sb, p.qo_st, p.qo_sh, ql, qh);
    store_row(p.ko, p.ko_sb, p.ko_st, p.ko_sh, kl, kh);
    store_row(p.vo, p.vo_sb, p.vo_st, p.vo_sh, vl, vh);
  }
}

}  // namespace daisy

using namespace daisy;

static int prep_launch(const void* q, const int64_t* q_strides,
                       const void* k, const int64_t* k_strides,
                       const void* v, const int64_t* v_strides,
                       const void* ve, const int64_t* ve_strides, const float* gate,
                       const float* cos, const float* sin, int pos0, const int32_t* pos0_dev, int table_rows, int32_t* status,
                       void* q_out, const int64_t* q_out_strides,
                       void* k_out, const int64_t* k_out_strides,
                       void* v_out, const int64_t* v_out_strides,
                       int B, int T, int H, int D, float eps, void* stream) {
  DAISY_CHECK_ARG(q && k && v && q_out && k_out && v_out, "qkv_prep: q, k, v and the three outputs must be non-NULL");
  DAISY_CHECK_ARG(q_strides && k_strides && v_strides && q_out_strides && k_out_strides && v_out_strides,
                  "qkv_prep: stride arrays must be non-NULL");
  DAISY_CHECK_ARG(B > 0 && T > 0 && H > 0, "qkv_prep: B=%d, T=%d, H=%d must be positive", B, T, H);
  DAISY_CHECK_ARG((cos == nullptr) == (sin == nullptr), "qkv_prep: cos and sin must both be given or both NULL");
  DAISY_CHECK_ARG((ve == nullptr) == (gate == nullptr), "qkv_prep: ve and gate must both be given or both NULL");
  DAISY_CHECK_ARG(ve == nullptr || ve_strides != nullptr, "qkv_prep: ve needs ve_strides");
  DAISY_CHECK_ARG(pos0 >= 0, "qkv_prep: pos0=%d must be >= 0", pos0);
  DAISY_CHECK_SUPPORTED(D == 64 || D == 128, "qkv_prep: head_dim %d not supported (64 or 128)", D);
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(al16(q) && al16(k) && al16(v) && al16(ve) && al16(cos) && al16(sin) && al16(q_out) && al16(k_out) && al16(v_out),
                  "qkv_prep: tensors must be 16-byte aligned");
  for (int i = 0; i < 3; ++i) {
    DAISY_CHECK_ARG(q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 &&
                        q_out_strides[i] % 8 == 0 && k_out_strides[i] % 8 == 0 && v_out_strides[i] % 8 == 0 &&
                        (!ve || ve_strides[i] % 8 == 0),
                    "qkv_prep: strides must be multiples of 8 elements");
  }

  PrepParams p;
  p.q = (const uint16_t*)q; p.q_sb = q_strides[0]; p.q_st = q_strides[1]; p.q_sh = q_strides[2];
  p.k = (const uint16_t*)k; p.k_sb = k_strides[0]; p.k_st = k_strides[1]; p.k_sh = k_strides[2];
  p.v = (const uint16_t*)v; p.v_sb = v_strides[0]; p.v_st = v_strides[1]; p.v_sh = v_strides[2];
  p.ve = (const uint16_t*)ve;
  p.e_sb = ve ? ve_strides[0] : 0; p.e_st = ve ? ve_strides[1] : 0; p.e_sh = ve ? ve_strides[2] : 0;
  p.gate = gate; p.cos = cos; p.sin = sin;
  p.qo = (uint16_t*)q_out; p.qo_sb = q_out_strides[0]; p.qo_st = q_out_strides[1]; p.qo_sh = q_out_strides[2];
  p.ko = (uint16_t*)k_out; p.ko_sb = k_out_strides[0]; p.ko_st = k_out_strides[1]; p.ko_sh = k_out_strides[2];
  p.vo = (uint16_t*)v_out; p.vo_sb = v_out_strides[0]; p.vo_st = v_out_strides[1]; p.vo_sh = v_out_strides[2];
  p.B = B; p.T = T; p.H = H; p.pos0 = pos0; p.eps = eps;
  p.pos0_dev = pos0_dev; p.table_rows = table_rows; p.status = status;
  p.rows = (int64_t)B * T * H;
  const int lpr = D / 16;
  const int64_t nwg = (p.rows * lpr + 255) / 256;
  DAISY_CHECK_ARG(nwg <= 0x7fffffff, "qkv_prep: too many rows (%lld)", (long long)p.rows);
  hipStream_t s = (hipStream_t)stream;
  if (D == 128) hipLaunchKernelGGL(qkv_prep_kernel<128>, dim3((unsigned)nwg), dim3(256), 0, s, p);
  else hipLaunchKernelGGL(qkv_prep_kernel<64>, dim3((unsigned)nwg), dim3(256), 0, s, p);
  DAISY_CHECK_LAUNCH("qkv_prep_kernel");
  return DAISY_OK;
}

extern "C" int daisy_qkv_prep_fwd(const void* q, const int64_t* q_strides,
                                  const void* k, const int64_t* k_strides,
                                  const void* v, const int64_t* v_strides,
                                  const void* ve, const int64_t* ve_strides, const float* gate,
                                  const float* cos, const float* sin, int pos0,
                                  void* q_out, const int64_t* q_out_strides,
                                  void* k_out, const int64_t* k_out_strides,
                                  void* v_out, const int64_t* v_out_strides,
                                  int B, int T, int H, int D, float eps, void* stream) {
  return prep_launch(q, q_strides, k, k_strides, v, v_strides, ve, ve_strides, gate, cos, sin, pos0, nullptr, 0, nullptr,
                     q_out, q_out_strides, k_out, k_out_strides, v_out, v_out_strides, B, T, H, D, eps, stream);
}

extern "C" int daisy_qkv_prep_fwd_at(const void* q, const int64_t* q_strides,
                                     const void* k, const int64_t* k_strides,
                                     const void* v, const int64_t* v_strides,
                                     const void* ve, const int64_t* ve_strides, const float* gate,
                                     const float* cos, const float* sin, const int32_t* pos0, int table_rows, int32_t* status,
                                     void* q_out, const int64_t* q_out_strides,
                                     void* k_out, const int64_t* k_out_strides,
                                     void* v_out, const int64_t* v_out_strides,
                                     int B, int T, int H, int D, float eps, void* stream) {
  DAISY_CHECK_ARG(pos0 != nullptr, "qkv_prep_at: the device position pointer must be non-NULL");
  DAISY_CHECK_ARG(cos && sin, "qkv_prep_at: the rotary tables are required");
  DAISY_CHECK_ARG(table_rows >= T, "qkv_prep_at: table_rows=%d must cover the %d rows of the call", table_rows, T);
  return prep_launch(q, q_strides, k, k_strides, v, v_strides, ve, ve_strides, gate, cos, sin, 0, pos0, table_rows, status,
                     q_out, q_out_strides, k_out, k_out_strides, v_out, v_out_strides, B, T, H, D, eps, stream);
}
