// Kernel 1: sliding-window causal flash-attention prefill with fused RoPE (gfx950).
//
// Work decomposition
//   workgroup = 4 wavefronts = 128 consecutive query rows of one (batch, head);
//   wavefront = 32 query rows.  Key/value rows are visited in tiles of 64, and
//   only tiles that intersect [lo(q_first), q_last] are loaded at all, where
//   lo(q) = max(q - window + 1, doc_start[q], 0) is non-decreasing in q.
//
// MFMA formulation (v_mfma_f32_32x32x16_bf16, wave64)
//   The kernel computes the TRANSPOSED products  S^T = K Q^T  and
//   O^T = V^T P^T.  In the 32x32 accumulator layout a lane owns one column, so
//   every lane owns one QUERY: lane l holds query (l % 32) and, per accumulator
//   register r, key row 8*(r/4) + 4*(l/32) + (r%4).  Row max / row sum are
//   therefore per-lane loops plus one exchange between lanes l and l^32, the
//   rescale of O^T is a per-lane scalar, and the accumulator registers of S^T,
//   converted to bf16, already ARE the B operand of the second product: the
//   contraction index of an MFMA may be enumerated in any order as long as the
//   A and B operands agree, so V^T is stored in LDS with key rows permuted to
//   match (swap bits 2 and 3 of the key index inside each group of 16).
//
// LDS (double buffered): K tile [64][D+8] bf16 row major, V^T tile [D][64+8]
// bf16.  The +8 element pad makes the 16-byte operand reads of 8 consecutive
// lanes fall into distinct banks.  V is transposed in registers as 4x4 blocks
// on its way from global memory to LDS.
//
// Algorithmic work: 4*D flops per visible (query, key) pair.
#include "common.h"

namespace daisy {

struct PrefillParams {
  const uint16_t* q; int64_t q_sb, q_st, q_sh;
  const uint16_t* k; int64_t k_sb, k_st, k_sh;
  const uint16_t* v; int64_t v_sb, v_st, v_sh;
  const float* cos; const float* sin;
  const int32_t* doc_start;
  uint16_t* o; int64_t o_sb, o_st, o_sh;
  uint16_t* k_out; int64_t ko_sb, ko_st, ko_sh;
  int B, T, H, D, window, nqb;
  float scale_log2e;
};

constexpr int kBM = 128;  // query rows per workgroup
constexpr int kBN = 64;   // key rows per tile
constexpr int kPrefillThreads = 256;

__device__ __forceinline__ int row_lo(const PrefillParams& p, int q) {
  int lo = (p.window > 0) ? max(q - p.window + 1, 0) : 0;
  if (p.doc_start != nullptr) lo = max(lo, p.doc_start[q]);
  return lo;
}

// Exchange with the lane that holds the other half of this query's keys.
__device__ __forceinline__ float pair_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_int(x), __float_as_int(x), false, false);
  return fmaxf(__int_as_float(r[0]), __int_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_int(x), __float_as_int(x), false, false);
  return __int_as_float(r[0]) + __int_as_float(r[1]);
}

// Position inside a V^T row of key row `kv` (0..63): bits 2 and 3 swapped.
__device__ __forceinline__ int vt_pos(int kv) { return (kv & ~12) | ((kv & 4) << 1) | ((kv & 8) >> 1); }

template <int D, bool ROPE_K>
__global__ __launch_bounds__(kPrefillThreads, 2) void prefill_mfma_kernel(PrefillParams p) {
  constexpr int KS = D + 8;        // K tile row stride (elements)
  constexpr int VS = kBN + 8;      // V^T tile row stride (elements)
  constexpr int NS = D / 16;       // MFMA steps over the head dim for S^T
  constexpr int NDT = D / 32;      // 32-row tiles of O^T
  constexpr int HALF = D / 2;
  constexpr int CPR = D / 8;       // 16-byte chunks per K row
  constexpr int NKC = ROPE_K ? (kBN * CPR / 2) / kPrefillThreads : (kBN * CPR) / kPrefillThreads;
  constexpr int NVB = (kBN / 4) * (D / 4) / kPrefillThreads;  // 4x4 V blocks per thread

  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][kBN * KS];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[2][D * VS];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int lq = lane & 31, lh = lane >> 5;

  // ---- workgroup -> (batch, head, query block); XCD-aware ------------------
  // Workgroups are dealt round-robin to the 8 XCDs.  Give each XCD a contiguous
  // run of (batch, head, query block) ids so that the query blocks sharing K/V
  // rows also share an L2, and start with the heaviest query blocks.
  int vid = blockIdx.x;
  {
    const int nwg = gridDim.x;
    if ((nwg & 7) == 0) vid = (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3);
  }
  const int qb = p.nqb - 1 - (vid % p.nqb);
  const int bh = vid / p.nqb;
  const int h = bh % p.H, b = bh / p.H;

  const int q0 = qb * kBM;
  const int qw0 = q0 + wave * 32;
  const int qrow = min(qw0 + lq, p.T - 1);
  const int lo_q = row_lo(p, qrow);
  const int lo_w_min = __builtin_amdgcn_readlane(lo_q, 0);
  const int lo_w_max = __builtin_amdgcn_readlane(lo_q, 31);
  const int q_w_min = min(qw0, p.T - 1), q_w_max = min(qw0 + 31, p.T - 1);
  const bool wave_live = qw0 < p.T;

  const int t_lo = row_lo(p, q0) / kBN;
  const int t_hi = min(q0 + kBM - 1, p.T - 1) / kBN;

  // ---- Q fragment (B operand), RoPE fused ----------------------------------
  bf16x8 qreg[NS];
  {
    const uint16_t* qptr = p.q + b * p.q_sb + (int64_t)qrow * p.q_st + h * p.q_sh + 8 * lh;
    u32x4 raw[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) raw[s] = *reinterpret_cast<const u32x4*>(qptr + 16 * s);
    if (p.cos != nullptr) {
      const float* cr = p.cos + (int64_t)qrow * HALF + 8 * lh;
      const float* sr = p.sin + (int64_t)qrow * HALF + 8 * lh;
#pragma unroll
      for (int s = 0; s < NS / 2; ++s) {
        float x1[8], x2[8], y1[8], y2[8];
        unpack8(raw[s], x1);
        unpack8(raw[s + NS / 2], x2);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = cr[16 * s + e], sn = sr[16 * s + e];
          y1[e] = rope_lo(x1[e], x2[e], c, sn);
          y2[e] = rope_hi(x1[e], x2[e], c, sn);
        }
        raw[s] = pack8(y1);
        raw[s + NS / 2] = pack8(y2);
      }
    }
#pragma unroll
    for (int s = 0; s < NS; ++s) qreg[s] = __builtin_bit_cast(bf16x8, raw[s]);
  }

  const uint16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
  const uint16_t* vbase = p.v + b * p.v_sb + h * p.v_sh;

  // ---- staging registers ----------------------------------------------------
  u32x4 kst[ROPE_K ? 2 * NKC : NKC];
  u32x4 cst[ROPE_K ? 2 * NKC : 1], sst[ROPE_K ? 2 * NKC : 1];
  u32x2 vst[NVB][4];

  // V 4x4 block coordinates of this thread (see the bank analysis above VS).
  int v_db[NVB], v_kb[NVB];
  {
    const int l16 = tid & 15, grp = tid >> 4;
    constexpr int DBH = (D / 4) / 8;  // number of groups of 8 channel blocks
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
      const int idx = grp + 16 * i;             // 0 .. DBH*8-1
      const int db_hi = idx % DBH;
      const int rest = idx / DBH;               // 3 bits: kb bit0, bit2, bit3
      v_db[i] = db_hi * 8 + (l16 & 7);
      v_kb[i] = (rest & 1) | ((l16 >> 3) << 1) | (((rest >> 1) & 1) << 2) | (((rest >> 2) & 1) << 3);
    }
  }

  auto load_tile = [&](int tile) {
    const int kv0 = tile * kBN;
    if constexpr (!ROPE_K) {
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int c = tid + kPrefillThreads * i;
        const int row = min(kv0 + c / CPR, p.T - 1);
        kst[i] = *reinterpret_cast<const u32x4*>(kbase + (int64_t)row * p.k_st + 8 * (c % CPR));
      }
    } else {
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int c = tid + kPrefillThreads * i;
        const int row = min(kv0 + c / (CPR / 2), p.T - 1);
        const int dc = 8 * (c % (CPR / 2));
        const uint16_t* kp = kbase + (int64_t)row * p.k_st + dc;
        kst[2 * i] = *reinterpret_cast<const u32x4*>(kp);
        kst[2 * i + 1] = *reinterpret_cast<const u32x4*>(kp + HALF);
        const float* cp = p.cos + (int64_t)row * HALF + dc;
        const float* sp = p.sin + (int64_t)row * HALF + dc;
        cst[2 * i] = *reinterpret_cast<const u32x4*>(cp);
        cst[2 * i + 1] = *reinterpret_cast<const u32x4*>(cp + 4);
        sst[2 * i] = *reinterpret_cast<const u32x4*>(sp);
        sst[2 * i + 1] = *reinterpret_cast<const u32x4*>(sp + 4);
      }
    }
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int row = min(kv0 + 4 * v_kb[i] + j, p.T - 1);
        vst[i][j] = *reinterpret_cast<const u32x2*>(vbase + (int64_t)row * p.v_st + 4 * v_db[i]);
      }
    }
  };

  auto store_tile = [&](int tile, int buf) {
    if constexpr (!ROPE_K) {
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int c = tid + kPrefillThreads * i;
        *reinterpret_cast<u32x4*>(&Ks[buf][(c / CPR) * KS + 8 * (c % CPR)]) = kst[i];
      }
    } else {
      // This workgroup also publishes the rotated keys of its own query rows.
      const bool publish = p.k_out != nullptr && (tile * kBN) / kBM == qb;
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int c = tid + kPrefillThreads * i;
        const int r = c / (CPR / 2), dc = 8 * (c % (CPR / 2));
        float x1[8], x2[8], y1[8], y2[8];
        unpack8(kst[2 * i], x1);
        unpack8(kst[2 * i + 1], x2);
        const float cs[8] = {__uint_as_float(cst[2 * i].x), __uint_as_float(cst[2 * i].y), __uint_as_float(cst[2 * i].z),
                             __uint_as_float(cst[2 * i].w), __uint_as_float(cst[2 * i + 1].x), __uint_as_float(cst[2 * i + 1].y),
                             __uint_as_float(cst[2 * i + 1].z), __uint_as_float(cst[2 * i + 1].w)};
        const float sn[8] = {__uint_as_float(sst[2 * i].x), __uint_as_float(sst[2 * i].y), __uint_as_float(sst[2 * i].z),
                             __uint_as_float(sst[2 * i].w), __uint_as_float(sst[2 * i + 1].x), __uint_as_float(sst[2 * i + 1].y),
                             __uint_as_float(sst[2 * i + 1].z), __uint_as_float(sst[2 * i + 1].w)};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          y1[e] = rope_lo(x1[e], x2[e], cs[e], sn[e]);
          y2[e] = rope_hi(x1[e], x2[e], cs[e], sn[e]);
        }
        const u32x4 a = pack8(y1), bb = pack8(y2);
        *reinterpret_cast<u32x4*>(&Ks[buf][r * KS + dc]) = a;
        *reinterpret_cast<u32x4*>(&Ks[buf][r * KS + dc + HALF]) = bb;
        const int grow = tile * kBN + r;
        if (publish && grow < p.T) {
          uint16_t* op = p.k_out + b * p.ko_sb + (int64_t)grow * p.ko_st + h * p.ko_sh + dc;
          *reinterpret_cast<u32x4*>(op) = a;
          *reinterpret_cast<u32x4*>(op + HALF) = bb;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
      const u32x2 r0 = vst[i][0], r1 = vst[i][1], r2 = vst[i][2], r3 = vst[i][3];
      u32x2 c0, c1, c2, c3;
      c0.x = (r0.x & 0xffffu) | (r1.x << 16);         c0.y = (r2.x & 0xffffu) | (r3.x << 16);
      c1.x = (r0.x >> 16) | (r1.x & 0xffff0000u);     c1.y = (r2.x >> 16) | (r3.x & 0xffff0000u);
      c2.x = (r0.y & 0xffffu) | (r1.y << 16);         c2.y = (r2.y & 0xffffu) | (r3.y << 16);
      c3.x = (r0.y >> 16) | (r1.y & 0xffff0000u);     c3.y = (r2.y >> 16) | (r3.y & 0xffff0000u);
      uint16_t* dst = &Vt[buf][(4 * v_db[i]) * VS + vt_pos(4 * v_kb[i])];
      *reinterpret_cast<u32x2*>(dst) = c0;
      *reinterpret_cast<u32x2*>(dst + VS) = c1;
      *reinterpret_cast<u32x2*>(dst + 2 * VS) = c2;
      *reinterpret_cast<u32x2*>(dst + 3 * VS) = c3;
    }
  };

  // ---- accumulators -----------------------------------------------------------
  f32x16 oacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY;  // running max of scale*log2e*s for this lane's query
  float l_run = 0.f;        // this lane's share of the running sum

  load_tile(t_lo);
  store_tile(t_lo, 0);
  __syncthreads();

  for (int tile = t_lo; tile <= t_hi; ++tile) {
    const int buf = (tile - t_lo) & 1;
    if (tile < t_hi) load_tile(tile + 1);

    const int kv0 = tile * kBN;
    // Sub-blocks of 32 keys this wavefront needs (wave-uniform).
    bool need[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int kmin = kv0 + 32 * sb, kmax = kmin + 31;
      need[sb] = wave_live && kmin <= q_w_max && kmax >= lo_w_min;
    }

    if (need[0] || need[1]) {
      f32x16 sacc[2];
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[sb][r] = 0.f;
        if (need[sb]) {
          const uint16_t* kp = &Ks[buf][(32 * sb + lq) * KS + 8 * lh];
#pragma unroll
          for (int s = 0; s < NS; ++s) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(kp + 16 * s));
            sacc[sb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[s], sacc[sb], 0, 0, 0);
          }
          const int kmin = kv0 + 32 * sb, kmax = kmin + 31;
          const bool full = kmax <= q_w_min && kmin >= lo_w_max;
          if (!full) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int kv = kmin + 8 * (r >> 2) + 4 * lh + (r & 3);
              if (kv > qrow || kv < lo_q) sacc[sb][r] = -INFINITY;
            }
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[sb][r] = -INFINITY;
        }
      }

      // ---- online softmax (log2 domain) --------------------------------------
      float mt = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mt = fmaxf(mt, sacc[sb][r]);
      mt = pair_max(mt) * p.scale_log2e;
      const float m_new = fmaxf(m_run, mt);
      const float mu = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2(m_run - mu);
      m_run = m_new;
      float lsum = 0.f;
      bf16x8 pfrag[2][2];
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
        float pv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          pv[r] = fast_exp2(fmaf(sacc[sb][r], p.scale_log2e, -mu));
          lsum += pv[r];
        }
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          u32x4 pk;
          pk.x = pack_bf16x2(pv[8 * m + 0], pv[8 * m + 1]);
          pk.y = pack_bf16x2(pv[8 * m + 2], pv[8 * m + 3]);
          pk.z = pack_bf16x2(pv[8 * m + 4], pv[8 * m + 5]);
          pk.w = pack_bf16x2(pv[8 * m + 6], pv[8 * m + 7]);
          pfrag[sb][m] = __builtin_bit_cast(bf16x8, pk);
        }
      }
      l_run = l_run * alpha + lsum;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;

      // ---- O^T += V^T P^T ---------------------------------------------------------
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
        if (need[sb]) {
#pragma unroll
          for (int m = 0; m < 2; ++m) {
            const int m16 = 2 * sb + m;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
              const uint16_t* vp = &Vt[buf][(32 * dt + lq) * VS + 16 * m16 + 8 * lh];
              const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(vp));
              oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pfrag[sb][m], oacc[dt], 0, 0, 0);
            }
          }
        }
      }
    }

    if (tile < t_hi) store_tile(tile + 1, buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue ---------------------------------------------------------------
  const float l_tot = pair_sum(l_run);
  const float inv = 1.f / l_tot;
  if (qw0 + lq < p.T) {
    uint16_t* op = p.o + b * p.o_sb + (int64_t)(qw0 + lq) * p.o_st + h * p.o_sh + 4 * lh;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w.x = pack_bf16x2(oacc[dt][4 * g + 0] * inv, oacc[dt][4 * g + 1] * inv);
        w.y = pack_bf16x2(oacc[dt][4 * g + 2] * inv, oacc[dt][4 * g + 3] * inv);
        *reinterpret_cast<u32x2*>(op + 32 * dt + 8 * g) = w;
      }
    }
  }
}

// Rotates keys once and stores them with the caller's output strides.
template <int D>
__global__ __launch_bounds__(256) void rope_k_kernel(PrefillParams p) {
  constexpr int HALF = D / 2;
  constexpr int CH = HALF / 8;  // pair chunks per row
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)p.B * p.T * p.H * CH;
  if (idx >= total) return;
  const int ch = idx % CH;
  const int h = (idx / CH) % p.H;
  const int t = (idx / ((int64_t)CH * p.H)) % p.T;
  const int b = idx / ((int64_t)CH * p.H * p.T);
  const uint16_t* kp = p.k + b * p.k_sb + (int64_t)t * p.k_st + h * p.k_sh + 8 * ch;
  uint16_t* op = p.k_out + b * p.ko_sb + (int64_t)t * p.ko_st + h * p.ko_sh + 8 * ch;
  float x1[8], x2[8], y1[8], y2[8];
  unpack8(*reinterpret_cast<const u32x4*>(kp), x1);
  unpack8(*reinterpret_cast<const u32x4*>(kp + HALF), x2);
  const float* cr = p.cos + (int64_t)t * HALF + 8 * ch;
  const float* sr = p.sin + (int64_t)t * HALF + 8 * ch;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float c = cr[e], s = sr[e];
    y1[e] = rope_lo(x1[e], x2[e], c, s);
    y2[e] = rope_hi(x1[e], x2[e], c, s);
  }
  *reinterpret_cast<u32x4*>(op) = pack8(y1);
  *reinterpret_cast<u32x4*>(op + HALF) = pack8(y2);
}

// Scalar kernel for head dims the MFMA kernel does not cover (any even D <= 256).
// One wavefront per (batch, head, query); lanes split the head dim.  Slow by
// design: it serves tiny shapes only.
__global__ __launch_bounds__(64) void prefill_scalar_kernel(PrefillParams p) {
  const int t = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x;
  const int D = p.D, HALF = D / 2;
  constexpr int MAXPL = 4;  // channels per lane (D <= 256)
  float qv[MAXPL], acc[MAXPL];
  const uint16_t* qp = p.q + b * p.q_sb + (int64_t)t * p.q_st + h * p.q_sh;
  auto rot_load = [&](const uint16_t* vec, int pos, int d) -> float {
    float x = bf16lo_to_f32(vec[d]);
    if (p.cos != nullptr) {
      const bool lower = d < HALF;
      const float xp = bf16lo_to_f32(vec[lower ? d + HALF : d - HALF]);
      const float c = p.cos[(int64_t)pos * HALF + (lower ? d : d - HALF)];
      const float s = p.sin[(int64_t)pos * HALF + (lower ? d : d - HALF)];
      x = round_bf16(lower ? rope_lo(x, xp, c, s) : rope_hi(xp, x, c, s));
    }
    return x;
  };
#pragma unroll
  for (int i = 0; i < MAXPL; ++i) {
    const int d = lane + 64 * i;
    qv[i] = (d < D) ? rot_load(qp, t, d) * p.scale_log2e : 0.f;
    acc[i] = 0.f;
  }
  if (p.k_out != nullptr && p.cos != nullptr) {
    const uint16_t* kp = p.k + b * p.k_sb + (int64_t)t * p.k_st + h * p.k_sh;
    uint16_t* op = p.k_out + b * p.ko_sb + (int64_t)t * p.ko_st + h * p.ko_sh;
    for (int d = lane; d < D; d += 64) op[d] = (uint16_t)(pack_bf16x2(rot_load(kp, t, d), 0.f) & 0xffffu);
  }
  float m = -INFINITY, l = 0.f;
  const int lo = row_lo(p, t);
  for (int kv = lo; kv <= t; ++kv) {
    const uint16_t* kp = p.k + b * p.k_sb + (int64_t)kv * p.k_st + h * p.k_sh;
    const uint16_t* vp = p.v + b * p.v_sb + (int64_t)kv * p.v_st + h * p.v_sh;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < MAXPL; ++i) {
      const int d = lane + 64 * i;
      if (d < D) s = fmaf(qv[i], rot_load(kp, kv, d), s);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off);
    const float mn = fmaxf(m, s);
    const float alpha = fast_exp2(m - mn);
    const float pw = fast_exp2(s - mn);
    l = l * alpha + pw;
#pragma unroll
    for (int i = 0; i < MAXPL; ++i) {
      const int d = lane + 64 * i;
      if (d < D) acc[i] = acc[i] * alpha + pw * bf16lo_to_f32(vp[d]);
    }
    m = mn;
  }
  uint16_t* op = p.o + b * p.o_sb + (int64_t)t * p.o_st + h * p.o_sh;
#pragma unroll
  for (int i = 0; i < MAXPL; ++i) {
    const int d = lane + 64 * i;
    if (d < D) op[d] = (uint16_t)(pack_bf16x2(acc[i] / l, 0.f) & 0xffffu);
  }
}

template <int D>
static int launch_mfma(PrefillParams p, bool rope_in_kernel, hipStream_t s) {
  const int64_t nwg = (int64_t)p.nqb * p.H * p.B;
  if (nwg > 0x7fffffff) {
    set_error("prefill: too many workgroups (%lld)", (long long)nwg);
    return DAISY_ERR_INVALID_ARGUMENT;
  }
  if (p.cos != nullptr && !rope_in_kernel) {
    // Pre-pass: rotate K once into k_out, then attend over k_out.
    const int64_t total = (int64_t)p.B * p.T * p.H * (D / 16);
    hipLaunchKernelGGL(rope_k_kernel<D>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, p);
    DAISY_CHECK_LAUNCH("rope_k_kernel");
    p.k = p.k_out; p.k_sb = p.ko_sb; p.k_st = p.ko_st; p.k_sh = p.ko_sh;
    hipLaunchKernelGGL((prefill_mfma_kernel<D, false>), dim3((unsigned)nwg), dim3(kPrefillThreads), 0, s, p);
  } else if (p.cos != nullptr) {
    hipLaunchKernelGGL((prefill_mfma_kernel<D, true>), dim3((unsigned)nwg), dim3(kPrefillThreads), 0, s, p);
  } else {
    hipLaunchKernelGGL((prefill_mfma_kernel<D, false>), dim3((unsigned)nwg), dim3(kPrefillThreads), 0, s, p);
  }
  DAISY_CHECK_LAUNCH("prefill_mfma_kernel");
  return DAISY_OK;
}

}  // namespace daisy

using namespace daisy;

extern "C" int daisy_prefill_fwd(const void* q, const int64_t* q_strides,
                                 const void* k, const int64_t* k_strides,
                                 const void* v, const int64_t* v_strides,
                                 const float* cos, const float* sin,
                                 const int32_t* doc_start,
                                 void* o, const int64_t* o_strides,
                                 void* k_out, const int64_t* k_out_strides,
                                 int B, int T, int H, int D,
                                 int window, float scale, int flags, void* stream) {
  DAISY_CHECK_ARG(q && k && v && o, "prefill: q, k, v and o must be non-NULL");
  DAISY_CHECK_ARG(q_strides && k_strides && v_strides && o_strides, "prefill: stride arrays must be non-NULL");
  DAISY_CHECK_ARG(B > 0 && T > 0 && H > 0, "prefill: B=%d, T=%d, H=%d must be positive", B, T, H);
  DAISY_CHECK_ARG((cos == nullptr) == (sin == nullptr), "prefill: cos and sin must both be given or both NULL");
  DAISY_CHECK_ARG(k_out == nullptr || k_out_strides != nullptr, "prefill: k_out needs k_out_strides");
  DAISY_CHECK_SUPPORTED(D >= 2 && D <= 256 && D % 2 == 0, "prefill: head_dim %d not supported (even, 2..256)", D);

  PrefillParams p;
  p.q = (const uint16_t*)q; p.q_sb = q_strides[0]; p.q_st = q_strides[1]; p.q_sh = q_strides[2];
  p.k = (const uint16_t*)k; p.k_sb = k_strides[0]; p.k_st = k_strides[1]; p.k_sh = k_strides[2];
  p.v = (const uint16_t*)v; p.v_sb = v_strides[0]; p.v_st = v_strides[1]; p.v_sh = v_strides[2];
  p.cos = cos; p.sin = sin; p.doc_start = doc_start;
  p.o = (uint16_t*)o; p.o_sb = o_strides[0]; p.o_st = o_strides[1]; p.o_sh = o_strides[2];
  p.k_out = (uint16_t*)k_out;
  p.ko_sb = k_out ? k_out_strides[0] : 0; p.ko_st = k_out ? k_out_strides[1] : 0; p.ko_sh = k_out ? k_out_strides[2] : 0;
  p.B = B; p.T = T; p.H = H; p.D = D; p.window = window;
  p.nqb = (T + kBM - 1) / kBM;
  p.scale_log2e = scale * kLog2e;
  hipStream_t s = (hipStream_t)stream;

  if (D == 64 || D == 128) {
    auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    DAISY_CHECK_ARG(al16(q) && al16(k) && al16(v) && al16(o) && al16(k_out) && al16(cos) && al16(sin),
                    "prefill: tensors must be 16-byte aligned");
    for (int i = 0; i < 3; ++i) {
      DAISY_CHECK_ARG(q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 && o_strides[i] % 8 == 0 &&
                          (!k_out || k_out_strides[i] % 8 == 0),
                      "prefill: strides must be multiples of 8 elements");
    }
    const bool rope_in_kernel = (flags & DAISY_PREFILL_ROTATE_K_IN_KERNEL) != 0 || k_out == nullptr;
    return D == 128 ? launch_mfma<128>(p, rope_in_kernel, s) : launch_mfma<64>(p, rope_in_kernel, s);
  }

  DAISY_CHECK_ARG(B <= 65535 && H <= 65535, "prefill: B and H must each be <= 65535 for the scalar kernel");
  hipLaunchKernelGGL(prefill_scalar_kernel, dim3(T, H, B), dim3(64), 0, s, p);
  DAISY_CHECK_LAUNCH("prefill_scalar_kernel");
  return DAISY_OK;
}
