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
//   A and B operands agree, so the V^T operand simply fetches, per lane, the key
//   rows 16m + 8g + 4*(l/32) + 0..3 that the lane's P registers hold.
//
// LDS (double buffered): K and V tiles [64][D] bf16, row major, filled by direct
// global->LDS copies (global_load_lds_dwordx4: no staging registers, no LDS
// store instructions); the 16-byte chunks of each row are XOR-swizzled so that
// operand reads are bank-conflict free.  V^T operands come out of the row-major
// V tile through LDS transpose reads (ds_read_b64_tr_b16): inside a block of 16
// lanes, lane L receives element L%4 of the four 8-byte chunks addressed by
// lanes L/4, L/4+4, L/4+8, L/4+12; with lane i of a block addressing key i/4,
// channels 4*(i%4)..+3, lane i receives channel i of four consecutive keys.
//
// Two kernels share this structure: prefill_pipe_kernel (keys need no rotation
// here; software pipelined) and prefill_mfma_kernel<D, true> (keys are rotated
// while they are staged into LDS).
//
// Algorithmic work: 4*D flops per visible (query, key) pair.
#include "common.h"

#include <type_traits>

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
  int period;    // tiles in a full window's range (0 = no window): the rotation period of the tile order
  int n_light;   // leading query blocks that see fewer keys than a full window (0 = order by block only)
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

// Workgroup -> (batch*head, query block).  Workgroups are dealt round-robin to the 8 XCDs, each
// with its own L2: an XCD is given a contiguous group of (batch, head) pairs so that the query
// blocks sharing K/V rows share an L2.  Inside a group the blocks with a full window of keys
// come first, pair by pair from the last block down; the n_light shorter blocks at the start of
// every sequence come last, longest first across the whole group, and fill the tail of the grid.
__device__ __forceinline__ void workgroup_to_block(const PrefillParams& p, int& bh, int& qb) {
  const int nbh = p.B * p.H;
  int group = 0, gsize = nbh, idx = blockIdx.x;
  if ((nbh & 7) == 0) { group = blockIdx.x & 7; gsize = nbh >> 3; idx = blockIdx.x >> 3; }
  const int n_full = p.nqb - p.n_light;
  int local;
  if (idx < gsize * n_full) {
    local = idx / n_full;
    qb = p.nqb - 1 - idx % n_full;
  } else {
    const int j = idx - gsize * n_full;
    qb = p.n_light - 1 - j / gsize;
    local = j % gsize;
  }
  bh = group * gsize + local;
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

// LDS transpose read (ds_read_b64_tr_b16); semantics in the header comment.
typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t* p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)p);
  return __builtin_bit_cast(u32x2, v);
}

typedef __attribute__((address_space(3))) const uint16_t* lds_u16_ptr;
__device__ __forceinline__ u32x2 lds_read_tr16_as3(lds_u16_ptr p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)p);
  return __builtin_bit_cast(u32x2, v);
}

template <int D, bool ROPE_K>
__global__ __launch_bounds__(kPrefillThreads, 2) void prefill_mfma_kernel(PrefillParams p) {
  // LDS tiles are [64 rows][D] bf16 without padding; the 16-byte chunks of a row are stored
  // XOR-swizzled (chunk c of row r sits at position c ^ f(r)) so that operand reads are free
  // of bank conflicts.  The LDS has 64 banks of 4 bytes, i.e. 256 bytes per clock:
  //   K: a 16-byte read serves 16 lanes per clock = 16 consecutive rows, same chunk
  //      -> those rows must land in 16 different 16-byte slots of the 256-byte bank window;
  //   V: an 8-byte transpose read serves 32 lanes per clock = 4 consecutive rows x 64 bytes
  //      -> those rows must land in 4 different 64-byte slots.
  constexpr int NS = D / 16;       // MFMA steps over the head dim for S^T
  constexpr int NDT = D / 32;      // 32-row tiles of O^T
  constexpr int HALF = D / 2;
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int RPL = 64 / CPR;    // rows covered by one wavefront copy (1 KiB)
  constexpr int NLD = kBN / RPL / 4;   // wavefront copies per tensor, tile and wavefront
  constexpr int TILE = kBN * D;    // elements per LDS tile
  auto swz_k = [](int r) { return D == 128 ? (r & 15) : ((r >> 1) & 7); };
  auto swz_v = [](int r) { return D == 128 ? 4 * (r & 3) : 4 * ((r >> 1) & 1); };

  __shared__ __attribute__((aligned(1024))) uint16_t Ks[2][TILE];
  __shared__ __attribute__((aligned(1024))) uint16_t Vs[2][TILE];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  int bh, qb;
  workgroup_to_block(p, bh, qb);
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

  // ---- global -> LDS staging --------------------------------------------------
  // Wavefront copy j (0 .. 64/RPL-1) of a tile moves rows RPL*j .. RPL*j+RPL-1; lane i lands
  // at chunk position i % CPR of row i / CPR, so it fetches the chunk that belongs there.
  const int ld_row = lane / CPR, ld_pos = lane % CPR;
  int k_lane_off[NLD], v_lane_off[NLD];   // element offsets inside a tile's rows, per copy
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int r = RPL * (4 * i + wave) + ld_row;
    k_lane_off[i] = 8 * (ld_pos ^ swz_k(r));
    v_lane_off[i] = 8 * (ld_pos ^ swz_v(r));
  }

  u32x4 kst[ROPE_K ? 2 * ((kBN * CPR / 2) / kPrefillThreads) : 1];
  u32x4 cst[ROPE_K ? 2 * ((kBN * CPR / 2) / kPrefillThreads) : 1], sst[ROPE_K ? 2 * ((kBN * CPR / 2) / kPrefillThreads) : 1];
  constexpr int NKC = (kBN * CPR / 2) / kPrefillThreads;   // (row, channel-pair chunk) items per thread when rotating K

  // Per-lane source offsets of the wavefront copies relative to the first row of a tile
  // (32-bit; the tile base is uniform, so the copy can use scalar-base addressing).
  int k_src_off[NLD], v_src_off[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int row = RPL * (4 * i + wave) + ld_row;
    k_src_off[i] = row * (int)p.k_st + k_lane_off[i];
    v_src_off[i] = row * (int)p.v_st + v_lane_off[i];
  }

  const uint32_t ks_lds = lds_address(&Ks[0][0]), vs_lds = lds_address(&Vs[0][0]);

  auto issue_copies = [&](int tile, auto buf_tag) {
    constexpr int buf = decltype(buf_tag)::value;
    const int kv0 = tile * kBN;
    const uint16_t* kt = kbase + (int64_t)kv0 * p.k_st;
    const uint16_t* vt = vbase + (int64_t)kv0 * p.v_st;
    if (kv0 + kBN <= p.T) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const uint32_t dst = 2 * (buf * TILE + (4 * i + wave) * 512);
        if constexpr (!ROPE_K) copy16_to_lds_async(kt, 2 * k_src_off[i], ks_lds + dst);
        copy16_to_lds_async(vt, 2 * v_src_off[i], vs_lds + dst);
      }
    } else {
      // The tile reaches past the last row: clamp (the surplus rows are masked by causality).
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const uint32_t dst = 2 * (buf * TILE + (4 * i + wave) * 512);
        const int row = min(RPL * (4 * i + wave) + ld_row, p.T - 1 - kv0);
        if constexpr (!ROPE_K) copy16_to_lds_async(kt, 2 * (row * (int)p.k_st + k_lane_off[i]), ks_lds + dst);
        copy16_to_lds_async(vt, 2 * (row * (int)p.v_st + v_lane_off[i]), vs_lds + dst);
      }
    }
    if constexpr (ROPE_K) {
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
  };

  // Completes the staging of a tile: waits for the asynchronous copies and, when K is rotated
  // here, rotates the register-staged K rows into LDS (and publishes this workgroup's own rows).
  auto finish_copies = [&](int tile, auto buf_tag) {
    constexpr int buf = decltype(buf_tag)::value;
    if constexpr (ROPE_K) {
      const bool publish = p.k_out != nullptr && (tile * kBN) / kBM == qb;
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int c = tid + kPrefillThreads * i;
        const int r = c / (CPR / 2), cc = c % (CPR / 2), dc = 8 * cc;
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
        *reinterpret_cast<u32x4*>(&Ks[buf][r * D + 8 * (cc ^ swz_k(r))]) = a;
        *reinterpret_cast<u32x4*>(&Ks[buf][r * D + 8 * ((cc + CPR / 2) ^ swz_k(r))]) = bb;
        const int grow = tile * kBN + r;
        if (publish && grow < p.T) {
          uint16_t* op = p.k_out + b * p.ko_sb + (int64_t)grow * p.ko_st + h * p.ko_sh + dc;
          *reinterpret_cast<u32x4*>(op) = a;
          *reinterpret_cast<u32x4*>(op + HALF) = bb;
        }
      }
    }
    // vmcnt(0) as a compiler-visible wait (encoding: vmcnt = 0, expcnt = 7, lgkmcnt = 15): the
    // asynchronous copies have landed, and the compiler also learns that no earlier vector
    // load is pending, so it places no conservative vmcnt waits inside the tile loop (those
    // would wait for the copies of the NEXT tile, which it cannot see).
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
  };

  // ---- accumulators -----------------------------------------------------------
  f32x16 oacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY;  // reference maximum (scaled, log2 domain) of this lane's query
  float l_run = 0.f;        // this lane's share of the running sum

  // Per-lane LDS element offsets of the operand reads (inside one tile).
  //   K (A operand of S^T): row = key lq of the 32-key sub-block, step s wants chunk 2s + lh.
  //   V (A operand of O^T, LDS transpose read): the lane's block of 16 covers output channels
  //   32dt + 16*(block & 1) + 0..15 and keys 4*lh + 0..3 (+8, +16, ... as immediates); lane i of
  //   the block addresses key i/4, channels 4*(i%4)..+3 and receives channel i, four keys.
  const uint16_t* k_rd[NS];
  const uint16_t* v_rd[NDT];
#pragma unroll
  for (int s = 0; s < NS; ++s) k_rd[s] = &Ks[0][0] + lq * D + 8 * ((2 * s + lh) ^ swz_k(lq));
  {
    const int i16 = lane & 15, vrow = 4 * lh + (i16 >> 2);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const int chunk = 4 * dt + 2 * ((lane >> 4) & 1) + ((i16 & 3) >> 1);
      v_rd[dt] = &Vs[0][0] + vrow * D + 8 * (chunk ^ swz_v(vrow)) + 4 * (i16 & 1);
    }
  }

  // One tile of 64 keys.  MASKED = false: both 32-key sub-blocks are needed by this
  // wavefront and fully visible to all of its queries (no mask, no skipping).
  auto process_tile = [&](auto buf_tag, int kv0, auto masked_tag) {
    constexpr int buf = decltype(buf_tag)::value;
    constexpr bool MASKED = decltype(masked_tag)::value;
    bool need[2] = {true, true};
    if constexpr (MASKED) {
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
        const int kmin = kv0 + 32 * sb, kmax = kmin + 31;
        need[sb] = kmin <= q_w_max && kmax >= lo_w_min;
      }
    }
    f32x16 sacc[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[sb][r] = 0.f;
      if (!MASKED || need[sb]) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
          const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(k_rd[s] + (buf * TILE + 32 * sb * D)));
          sacc[sb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[s], sacc[sb], 0, 0, 0);
        }
        if constexpr (MASKED) {
          const int kmin = kv0 + 32 * sb;
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

    // ---- online softmax (log2 domain, lazy rescale) ------------------------------
    // The reference maximum m_run only moves when some query of the wavefront sees a
    // score more than 8 (log2 units) above it; until then probabilities are at most 2^8,
    // which bf16 and the fp32 sums hold without loss, and O is not touched.
    float mt = -INFINITY;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mt = fmaxf(mt, sacc[sb][r]);
    mt = pair_max(mt) * p.scale_log2e;
    if (__builtin_amdgcn_ballot_w64(mt > m_run + 8.f) != 0) {
      const float m_new = fmaxf(m_run, mt);
      const float mu = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2(m_run - mu);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
    }
    const float mu = (m_run == -INFINITY) ? 0.f : m_run;
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
    l_run += lsum;

    // ---- O^T += V^T P^T ---------------------------------------------------------
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      if (!MASKED || need[sb]) {
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          const int voff = buf * TILE + (32 * sb + 16 * m) * D;
#pragma unroll
          for (int dt = 0; dt < NDT; ++dt) {
            const u32x2 a0 = lds_read_tr16(v_rd[dt] + voff);            // keys 16m + 4lh + 0..3
            const u32x2 a1 = lds_read_tr16(v_rd[dt] + voff + 8 * D);    // keys 16m + 8 + 4lh + 0..3
            const u32x4 av = {a0.x, a0.y, a1.x, a1.y};
            oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av), pfrag[sb][m], oacc[dt], 0, 0, 0);
          }
        }
      }
    }
  };

  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, 1>;
  issue_copies(t_lo, Buf0{});
  finish_copies(t_lo, Buf0{});
  __syncthreads();

  // One iteration: start the copies of the next tile into the other buffer, compute on this
  // buffer, then wait for the copies and meet the other wavefronts.
  auto iteration = [&](int tile, auto buf_tag) {
    constexpr int buf = decltype(buf_tag)::value;
    using Other = std::integral_constant<int, buf ^ 1>;
    if (tile < t_hi) issue_copies(tile + 1, Other{});
    const int kv0 = tile * kBN;
    if (wave_live && kv0 <= q_w_max && kv0 + kBN - 1 >= lo_w_min) {
      const bool clean = kv0 + kBN - 1 <= q_w_min && kv0 >= lo_w_max;
      if (clean) process_tile(buf_tag, kv0, std::false_type{});
      else process_tile(buf_tag, kv0, std::true_type{});
    }
    if (tile < t_hi) finish_copies(tile + 1, Other{});
    __syncthreads();
  };
  for (int tile = t_lo; tile <= t_hi; tile += 2) {
    iteration(tile, Buf0{});
    if (tile + 1 <= t_hi) iteration(tile + 1, Buf1{});
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

// Software-pipelined variant (keys already rotated or no RoPE on keys): the O^T += V^T P^T
// product of tile i-1 is issued in the same basic block as the softmax of tile i, so the matrix
// pipe works while the vector ALU does max / exp2 / sum / convert, inside one wavefront and
// not only across the two wavefronts that share a SIMD.  V therefore runs one tile behind K:
//   iteration i:  copies  K(i+1) -> Kbuf[(i+1)&1],  V(i) -> Vbuf[i&1]
//                 S(i) = K(i) Q^T;   then   O += V(i-1)^T P(i-1)  ||  P(i) = softmax(S(i))
// A rescale of O that the softmax of tile i asks for is applied at the start of the next fused
// block (before P(i) is accumulated), which keeps that block free of branches.
// A wavefront works on the contiguous tile range [tw_lo, tw_hi] that its 32 queries can see
// (inside the workgroup's range); both 32-key halves of a tile in that range are computed and
// masked per element where needed.
template <int D>
__global__ __launch_bounds__(kPrefillThreads, 2) void prefill_pipe_kernel(PrefillParams p) {
  constexpr int NS = D / 16, NDT = D / 32, HALF = D / 2, CPR = D / 8;
  constexpr int RPL = 64 / CPR, NLD = kBN / RPL / 4, TILE = kBN * D;
  auto swz_k = [](int r) { return D == 128 ? (r & 15) : ((r >> 1) & 7); };
  auto swz_v = [](int r) { return D == 128 ? 4 * (r & 3) : 4 * ((r >> 1) & 1); };

  __shared__ __attribute__((aligned(1024))) uint16_t Ks[2][TILE];
  __shared__ __attribute__((aligned(1024))) uint16_t Vs[2][TILE];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  int bh, qb;
  workgroup_to_block(p, bh, qb);
  const int h = bh % p.H, b = bh / p.H;

  const int q0 = qb * kBM;
  const int qw0 = q0 + wave * 32;
  const int qrow = min(qw0 + lq, p.T - 1);
  const int lo_q = row_lo(p, qrow);
  const int lo_w_min = __builtin_amdgcn_readlane(lo_q, 0);
  const int lo_w_max = __builtin_amdgcn_readlane(lo_q, 31);
  const int q_w_min = min(qw0, p.T - 1), q_w_max = min(qw0 + 31, p.T - 1);

  const int t_lo = row_lo(p, q0) / kBN;
  const int t_hi = min(q0 + kBM - 1, p.T - 1) / kBN;
  // This wavefront's own tile range (empty when all of its rows are past the end).
  const int tw_lo = lo_w_min / kBN;
  const int tw_hi = (qw0 < p.T) ? q_w_max / kBN : -1;

  // Tiles are visited in rotated order: start at the tile whose index is a multiple of the
  // window's tile count (one exists in every full range), run up to t_hi, wrap to t_lo.  The
  // online softmax does not care about the order, and the query blocks of one (batch, head)
  // that run side by side then read the same K/V tile at the same step, so one fetch into the
  // L2 serves all of them.  With no window every range starts at tile 0 and nothing is rotated.
  const int n_tiles = t_hi - t_lo + 1;
  int t_first = t_lo;
  if (p.period > 0) {
    const int c = (t_lo + p.period - 1) / p.period * p.period;
    if (c <= t_hi) t_first = c;
  }

  const uint16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
  const uint16_t* vbase = p.v + b * p.v_sb + h * p.v_sh;

  // ---- global -> LDS copies (layout as in prefill_mfma_kernel) ---------------------------
  const int ld_row = lane / CPR, ld_pos = lane % CPR;
  int k_src_off[NLD], v_src_off[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int r = RPL * (4 * i + wave) + ld_row;
    k_src_off[i] = r * (int)p.k_st + 8 * (ld_pos ^ swz_k(r));
    v_src_off[i] = r * (int)p.v_st + 8 * (ld_pos ^ swz_v(r));
  }
  const uint32_t ks_lds = lds_address(&Ks[0][0]), vs_lds = lds_address(&Vs[0][0]);

  auto copy_tile = [&](const uint16_t* base, int stride, const int* src_off, bool is_k, uint32_t lds, int tile, int buf) {
    const int kv0 = tile * kBN;
    const uint16_t* tb = base + (int64_t)kv0 * stride;
    const uint32_t dst = lds + 2 * (buf * TILE + wave * 512);
    if (kv0 + kBN <= p.T) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) copy16_to_lds_async(tb, 2 * src_off[i], dst + 2 * (4 * i * 512));
    } else {
      // The tile reaches past the last row: clamp (the surplus rows are masked by causality).
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int r = RPL * (4 * i + wave) + ld_row;
        const int row = min(r, p.T - 1 - kv0);
        const int chunk = ld_pos ^ (is_k ? swz_k(r) : swz_v(r));
        copy16_to_lds_async(tb, 2 * (row * stride + 8 * chunk), dst + 2 * (4 * i * 512));
      }
    }
  };
  auto copy_k = [&](int tile, int buf) { copy_tile(kbase, (int)p.k_st, k_src_off, true, ks_lds, tile, buf); };
  auto copy_v = [&](int tile, int buf) { copy_tile(vbase, (int)p.v_st, v_src_off, false, vs_lds, tile, buf); };
  auto copies_landed = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0), visible to the compiler's wait-count model
    asm volatile("" ::: "memory");
  };

  // The first two K tiles go out before anything else so that their latency overlaps the Q loads.
  auto tile_of = [&](int n) { const int t = t_first + n; return t <= t_hi ? t : t - n_tiles; };
  copy_k(t_first, 0);
  if (n_tiles > 1) copy_k(tile_of(1), 1);

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

  // Per-lane LDS read pointers into buffer 0 (32-bit LDS addresses).
  lds_u16_ptr k_rd[NS];
  lds_u16_ptr v_rd[NDT];
#pragma unroll
  for (int s = 0; s < NS; ++s) k_rd[s] = (lds_u16_ptr)&Ks[0][0] + lq * D + 8 * ((2 * s + lh) ^ swz_k(lq));
  {
    const int i16 = lane & 15, vrow = 4 * lh + (i16 >> 2);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const int chunk = 4 * dt + 2 * ((lane >> 4) & 1) + ((i16 & 3) >> 1);
      v_rd[dt] = (lds_u16_ptr)&Vs[0][0] + vrow * D + 8 * (chunk ^ swz_v(vrow)) + 4 * (i16 & 1);
    }
  }

  f32x16 oacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  f32x16 sc[2];                    // S of the tile this step turns into P; refilled in place for the next tile
  float m_run = -INFINITY, l_run = 0.f;
  float alpha_pend = 1.f;          // rescale of O asked for by the last softmax, not applied yet
  bool rescale_pend = false;       // wave-uniform
  bool pending = false;            // wave-uniform: pfrag holds a P that has not been multiplied into O yet
  bf16x8 pfrag[2][2];              // P of the previous tile (B operands of the delayed product)
  {
    const u32x4 z = {0, 0, 0, 0};
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int m = 0; m < 2; ++m) pfrag[sb][m] = __builtin_bit_cast(bf16x8, z);
  }

  auto apply_pending_rescale = [&]() {
    if (rescale_pend) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha_pend;
      rescale_pend = false;
    }
  };

  // One 32-key half of S^T = K Q^T into sc[sb], K from buffer offset kofs (elements).
  auto qk_half = [&](int kofs, int sb) {
    constexpr int KPF = 3;   // K fragments are read KPF contraction slices ahead of their MFMAs
    bf16x8 ka[KPF];
    auto read_k = [&](int s) {
      ka[s % KPF] = __builtin_bit_cast(bf16x8, *(const u32x4 __attribute__((address_space(3)))*)(k_rd[s] + kofs + 32 * sb * D));
    };
#pragma unroll
    for (int s = 0; s < KPF; ++s) read_k(s);
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[sb][r] = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      sc[sb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[s % KPF], qreg[s], sc[sb], 0, 0, 0);
      if (s + KPF < NS) read_k(s + KPF);
    }
  };

  // Half of O^T += V^T P^T: the 32 keys of block sb, V from buffer offset vofs (elements).
  auto pv_half = [&](int vofs, int sb) {
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        lds_u16_ptr vp = v_rd[dt] + vofs;
        const u32x2 a0 = lds_read_tr16_as3(vp + (32 * sb + 16 * m) * D);
        const u32x2 a1 = lds_read_tr16_as3(vp + (32 * sb + 16 * m + 8) * D);
        const u32x4 av = {a0.x, a0.y, a1.x, a1.y};
        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av), pfrag[sb][m], oacc[dt], 0, 0, 0);
      }
    }
  };

  // Online-softmax bookkeeping for the tile held in sc (after masking): returns the exponent offset.
  // Lazy rescale: the reference maximum only moves when some query of the wavefront sees a score
  // more than 8 (log2 units) above it; until then probabilities stay below 2^8, which bf16 and
  // the fp32 sums hold without loss, and O is not touched.
  auto update_maximum = [&]() {
    float mt = -INFINITY;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mt = fmaxf(mt, sc[sb][r]);
    mt = pair_max(mt) * p.scale_log2e;
    const bool move = __builtin_amdgcn_ballot_w64(mt > m_run + 8.f) != 0;
    const float m_new = move ? fmaxf(m_run, mt) : m_run;
    const float mu = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - mu);      // 1 when the maximum did not move, 0 on the first tile
    m_run = m_new;
    alpha_pend = alpha;
    rescale_pend = move;
    l_run *= alpha;
    return mu;
  };
  // P of one 32-key half: exp2, row sums, bf16 B operands of the delayed product.
  auto probabilities_half = [&](int sb, float mu) {
    float pv[16];
    float lsum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      pv[r] = fast_exp2(fmaf(sc[sb][r], p.scale_log2e, -mu));
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
    l_run += lsum;
  };
  auto mask_scores = [&](int kv0) {
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      // element r of this lane is key kv0 + 32sb + 4lh + c_r with c_r = 8*(r/4) + r%4
      const int hi = qrow - (kv0 + 32 * sb + 4 * lh);    // visible iff lo <= c_r <= hi
      const int lo = lo_q - (kv0 + 32 * sb + 4 * lh);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 8 * (r >> 2) + (r & 3);
        if (c > hi || c < lo) sc[sb][r] = -INFINITY;
      }
    }
  };

  auto is_active = [&](int n) {
    if (n < 0 || n >= n_tiles) return false;
    const int t = tile_of(n);
    return t >= tw_lo && t <= tw_hi;
  };
  // Step n: K(n+2) and V(n) start on their way; at the end they have landed and all wavefronts meet.
  // K(n+1) was published by the previous step, V(n-1) too.
  auto step_begin = [&](int n) {
    if (n + 2 < n_tiles) copy_k(tile_of(n + 2), n & 1);
    copy_v(tile_of(n), n & 1);
  };
  auto step_end = [&]() {
    copies_landed();
    __syncthreads();
  };

  // Generic step (tiles at the edges of a wavefront's range, masked tiles, idle steps): the three
  // pieces one after the other.
  auto generic_steps = [&](int from, int to) {
    for (int n = from; n <= to; ++n) {
      const int par = n & 1;
      step_begin(n);
      if (pending) {
        apply_pending_rescale();
        pv_half((par ^ 1) * TILE, 0);
        pv_half((par ^ 1) * TILE, 1);
        pending = false;
      }
      if (is_active(n)) {
        const int kv0 = tile_of(n) * kBN;
        if (!(kv0 + kBN - 1 <= q_w_min && kv0 >= lo_w_max)) mask_scores(kv0);
        const float mu = update_maximum();
        probabilities_half(0, mu);
        probabilities_half(1, mu);
        pending = true;
      }
      if (is_active(n + 1)) {
        qk_half((par ^ 1) * TILE, 0);
        qk_half((par ^ 1) * TILE, 1);
      }
      step_end();
    }
  };
  // Hot step: tile n fully visible, the previous and the next tile belong to this wavefront too.
  // One basic block holds the delayed product of tile n-1, the softmax of tile n and S of tile
  // n+1 (written into the registers of S(n) as soon as each half has been turned into P), so
  // that the matrix pipe has work all along the vector work of the same wavefront.
  auto hot_steps = [&](int from, int to) {
    for (int n = from; n <= to; ++n) {
      const int par = n & 1;
      const int other = (par ^ 1) * TILE;   // V(n-1) and K(n+1) both sit in the other buffer
      step_begin(n);
      apply_pending_rescale();
      const float mu = update_maximum();
      pv_half(other, 0);
      probabilities_half(0, mu);   // frees sc[0] ...
      pv_half(other, 1);
      qk_half(other, 0);           // ... for S(n+1), first half
      probabilities_half(1, mu);
      qk_half(other, 1);
      step_end();
    }
  };

  copies_landed();
  __syncthreads();
  if (is_active(0)) {
    qk_half(0, 0);
    qk_half(0, 1);
  }

  // Fully visible tiles of this wavefront: first key >= every row's lower bound, last key <=
  // the first row.  A hot step needs such a tile with active neighbours in the same run of
  // consecutive tiles (the rotated order has two runs: t_first..t_hi, then t_lo..t_first-1).
  const int c_lo = max((lo_w_max + kBN - 1) / kBN, max(tw_lo, t_lo));
  const int c_hi = min((q_w_min + 1) / kBN - 1, min(tw_hi, t_hi));
#pragma nounroll
  for (int run = 0; run < 2; ++run) {
    const int a = run == 0 ? t_first : t_lo;
    const int b = run == 0 ? t_hi : t_first - 1;
    const int n0 = run == 0 ? 0 : t_hi - t_first + 1;     // step of tile a
    if (b < a) continue;
    int ha = max(max(c_lo, a + 1), tw_lo + 1);
    int hb = min(min(c_hi, b - 1), tw_hi - 1);
    if (hb < ha) { ha = b + 1; hb = b; }                   // no hot tile in this run
    generic_steps(n0, n0 + ha - 1 - a);
    hot_steps(n0 + ha - a, n0 + hb - a);
    generic_steps(n0 + hb + 1 - a, n0 + b - a);
  }
  if (pending) {
    apply_pending_rescale();
    pv_half(((n_tiles - 1) & 1) * TILE, 0);
    pv_half(((n_tiles - 1) & 1) * TILE, 1);
  }

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
  // The unrotated keys are not needed again: read them past the caches, so that q, v and the
  // rotated keys this pass writes are what the attention kernel finds there.
  unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp)), x1);
  unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp + HALF)), x2);
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

// Scalar kernel for head dims the MFMA kernel does not cover (any even D <= 256) and for fp32
// tensors.  One wavefront per (batch, head, query); lanes split the head dim.  Slow by
// design: it serves tiny shapes and the full-precision mode only.  E = uint16_t (bf16 bits;
// rotated values are rounded to bf16 as the bf16 tensors of the reference are) or float
// (nothing is rounded: fp32 in, fp32 arithmetic, fp32 out).
template <typename E>
__global__ __launch_bounds__(64) void prefill_scalar_kernel(PrefillParams p) {
  const int t = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x;
  const int D = p.D, HALF = D / 2;
  constexpr int MAXPL = 4;  // channels per lane (D <= 256)
  float qv[MAXPL], acc[MAXPL];
  const E* qbase = reinterpret_cast<const E*>(p.q);
  const E* kbase = reinterpret_cast<const E*>(p.k);
  const E* vbase = reinterpret_cast<const E*>(p.v);
  const E* qp = qbase + b * p.q_sb + (int64_t)t * p.q_st + h * p.q_sh;
  auto rot_load = [&](const E* vec, int pos, int d) -> float {
    float x = load_elem<E>(vec, d);
    if (p.cos != nullptr) {
      const bool lower = d < HALF;
      const float xp = load_elem<E>(vec, lower ? d + HALF : d - HALF);
      const float c = p.cos[(int64_t)pos * HALF + (lower ? d : d - HALF)];
      const float s = p.sin[(int64_t)pos * HALF + (lower ? d : d - HALF)];
      x = round_elem<E>(lower ? rope_lo(x, xp, c, s) : rope_hi(xp, x, c, s));
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
    const E* kp = kbase + b * p.k_sb + (int64_t)t * p.k_st + h * p.k_sh;
    E* op = reinterpret_cast<E*>(p.k_out) + b * p.ko_sb + (int64_t)t * p.ko_st + h * p.ko_sh;
    for (int d = lane; d < D; d += 64) store_elem<E>(op, d, rot_load(kp, t, d));
  }
  float m = -INFINITY, l = 0.f;
  const int lo = row_lo(p, t);
  for (int kv = lo; kv <= t; ++kv) {
    const E* kp = kbase + b * p.k_sb + (int64_t)kv * p.k_st + h * p.k_sh;
    const E* vp = vbase + b * p.v_sb + (int64_t)kv * p.v_st + h * p.v_sh;
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
      if (d < D) acc[i] = acc[i] * alpha + pw * load_elem<E>(vp, d);
    }
    m = mn;
  }
  E* op = reinterpret_cast<E*>(p.o) + b * p.o_sb + (int64_t)t * p.o_st + h * p.o_sh;
#pragma unroll
  for (int i = 0; i < MAXPL; ++i) {
    const int d = lane + 64 * i;
    if (d < D) store_elem<E>(op, d, acc[i] / l);
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
    hipLaunchKernelGGL((prefill_pipe_kernel<D>), dim3((unsigned)nwg), dim3(kPrefillThreads), 0, s, p);
    DAISY_CHECK_LAUNCH("prefill_pipe_kernel");
  } else if (p.cos != nullptr) {
    hipLaunchKernelGGL((prefill_mfma_kernel<D, true>), dim3((unsigned)nwg), dim3(kPrefillThreads), 0, s, p);
    DAISY_CHECK_LAUNCH("prefill_mfma_kernel");
  } else {
    hipLaunchKernelGGL((prefill_pipe_kernel<D>), dim3((unsigned)nwg), dim3(kPrefillThreads), 0, s, p);
    DAISY_CHECK_LAUNCH("prefill_pipe_kernel");
  }
  return DAISY_OK;
}

// Argument checks and parameter block shared by the bf16 and the fp32 entry point.
static int fill_prefill_params(PrefillParams& p, const void* q, const int64_t* q_strides,
                               const void* k, const int64_t* k_strides,
                               const void* v, const int64_t* v_strides,
                               const float* cos, const float* sin, const int32_t* doc_start,
                               void* o, const int64_t* o_strides,
                               void* k_out, const int64_t* k_out_strides,
                               int B, int T, int H, int D, int window, float scale) {
  DAISY_CHECK_ARG(q && k && v && o, "prefill: q, k, v and o must be non-NULL");
  DAISY_CHECK_ARG(q_strides && k_strides && v_strides && o_strides, "prefill: stride arrays must be non-NULL");
  DAISY_CHECK_ARG(B > 0 && T > 0 && H > 0, "prefill: B=%d, T=%d, H=%d must be positive", B, T, H);
  DAISY_CHECK_ARG((cos == nullptr) == (sin == nullptr), "prefill: cos and sin must both be given or both NULL");
  DAISY_CHECK_ARG(k_out == nullptr || k_out_strides != nullptr, "prefill: k_out needs k_out_strides");
  DAISY_CHECK_SUPPORTED(D >= 2 && D <= 256 && D % 2 == 0, "prefill: head_dim %d not supported (even, 2..256)", D);
  p.q = (const uint16_t*)q; p.q_sb = q_strides[0]; p.q_st = q_strides[1]; p.q_sh = q_strides[2];
  p.k = (const uint16_t*)k; p.k_sb = k_strides[0]; p.k_st = k_strides[1]; p.k_sh = k_strides[2];
  p.v = (const uint16_t*)v; p.v_sb = v_strides[0]; p.v_st = v_strides[1]; p.v_sh = v_strides[2];
  p.cos = cos; p.sin = sin; p.doc_start = doc_start;
  p.o = (uint16_t*)o; p.o_sb = o_strides[0]; p.o_st = o_strides[1]; p.o_sh = o_strides[2];
  p.k_out = (uint16_t*)k_out;
  p.ko_sb = k_out ? k_out_strides[0] : 0; p.ko_st = k_out ? k_out_strides[1] : 0; p.ko_sh = k_out ? k_out_strides[2] : 0;
  p.B = B; p.T = T; p.H = H; p.D = D; p.window = window;
  p.nqb = (T + kBM - 1) / kBM;
  p.period = (window > 0 && window < T) ? (kBM - 1) / kBN + 1 + (window - 1 + kBN - 1) / kBN : 0;
  p.n_light = (window > 0 && window < T) ? min((window - 1 + kBM - 1) / kBM, p.nqb) : 0;
  p.scale_log2e = scale * kLog2e;
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
  PrefillParams p;
  const int rc = fill_prefill_params(p, q, q_strides, k, k_strides, v, v_strides, cos, sin, doc_start, o, o_strides,
                                     k_out, k_out_strides, B, T, H, D, window, scale);
  if (rc != DAISY_OK) return rc;
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
  hipLaunchKernelGGL(prefill_scalar_kernel<uint16_t>, dim3(T, H, B), dim3(64), 0, s, p);
  DAISY_CHECK_LAUNCH("prefill_scalar_kernel");
  return DAISY_OK;
}

extern "C" int daisy_prefill_fwd_f32(const float* q, const int64_t* q_strides,
                                     const float* k, const int64_t* k_strides,
                                     const float* v, const int64_t* v_strides,
                                     const float* cos, const float* sin,
                                     const int32_t* doc_start,
                                     float* o, const int64_t* o_strides,
                                     float* k_out, const int64_t* k_out_strides,
                                     int B, int T, int H, int D,
                                     int window, float scale, void* stream) {
  PrefillParams p;
  const int rc = fill_prefill_params(p, q, q_strides, k, k_strides, v, v_strides, cos, sin, doc_start, o, o_strides,
                                     k_out, k_out_strides, B, T, H, D, window, scale);
  if (rc != DAISY_OK) return rc;
  DAISY_CHECK_ARG(B <= 65535 && H <= 65535, "prefill: B and H must each be <= 65535 for the fp32 kernel");
  hipLaunchKernelGGL(prefill_scalar_kernel<float>, dim3(T, H, B), dim3(64), 0, (hipStream_t)stream, p);
  DAISY_CHECK_LAUNCH("prefill_scalar_kernel<float>");
  return DAISY_OK;
}
