// Kernel 1: sliding-window causal flash-attention prefill with fused RoPE (gfx950).
//
// Work decomposition
//   workgroup = 4 wavefronts = 128 consecutive query rows of one (batch, head);
//   wavefront = 32 query rows.  Key/value rows are visited in tiles of 32 rows, and
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
// LDS (double buffered): K and V tiles [rows][D] bf16, row major, filled by direct
// global->LDS copies (global_load_lds_dwordx4: no staging registers, no LDS
// store instructions); the 16-byte chunks of each row are XOR-swizzled so that
// operand reads are bank-conflict free.  V^T operands come out of the row-major
// V tile through LDS transpose reads (ds_read_b64_tr_b16): inside a block of 16
// lanes, lane L receives element L%4 of the four 8-byte chunks addressed by
// lanes L/4, L/4+4, L/4+8, L/4+12; with lane i of a block addressing key i/4,
// channels 4*(i%4)..+3, lane i receives channel i of four consecutive keys.
//
// Keys reach prefill_tile_kernel rotated: by the caller, or by rope_k_kernel, a
// pre-pass that writes the rotated keys the reference's prefill returns anyway.
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
  int period;    // 32-key tiles in a full window's range (0 = no window): the rotation period of the tile order
  int n_light;   // leading query blocks that see fewer keys than a full window (0 = order by block only)
  float scale_log2e;
};

constexpr int kBM = 128;  // query rows per workgroup
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
typedef __attribute__((address_space(3))) const uint16_t* lds_u16_ptr;
__device__ __forceinline__ u32x2 lds_read_tr16_as3(lds_u16_ptr p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)p);
  return __builtin_bit_cast(u32x2, v);
}

// Main kernel (keys already rotated, or no RoPE on keys).  32-key tiles, and nothing of a step is
// overlapped inside a wavefront: scores, softmax and the product of one tile follow each other.  The
// kernel is small instead -- 167 VGPRs and 48 KiB of LDS at D = 128 -- so that THREE workgroups fit a
// CU, three wavefronts a SIMD, and the latencies of one wavefront's step (the issue of its tile
// copies, the LDS operand reads, the softmax chain, the barrier) are covered by the other two: matrix
// instructions of one wavefront and vector instructions of another do run side by side on a SIMD.
//   step n:  copies K(n+1), V(n+1) -> the other buffer;  S = K(n) Q^T;  P = softmax(S);  O += V(n)^T P;
//            wait for the copies, barrier.
// A wavefront computes only the tiles its 32 queries can see; a tile at the window / document edge or
// on the diagonal is masked per element.  The Q block at the start and the O block at the end pass
// through an LDS area of the wavefront's own, so that every global access of the kernel covers whole
// rows (a CU's memory path, shared by its three workgroups, is busy per cache line touched).
constexpr int kTBN = 32;   // key rows per tile of prefill_tile_kernel
template <int D>
__global__ __launch_bounds__(kPrefillThreads, 3) void prefill_tile_kernel(PrefillParams p) {
  constexpr int NS = D / 16, NDT = D / 32, HALF = D / 2, CPR = D / 8;
  constexpr int RPL = 64 / CPR, NLD = kTBN / RPL / 4, TILE = kTBN * D;
  static_assert(NLD >= 1, "a tile is at least one copy per wavefront");
  auto swz_k = [](int r) { return D == 128 ? (r & 15) : ((r >> 1) & 7); };
  auto swz_v = [](int r) { return D == 128 ? 4 * (r & 3) : 4 * ((r >> 1) & 1); };

  __shared__ __attribute__((aligned(1024))) uint16_t Ks[2][TILE];
  __shared__ __attribute__((aligned(1024))) uint16_t Vs[2][TILE];
  // Two more tile-sized areas: with Ks[1] and Vs[1] they give every wavefront 32 rows x D of its own for
  // turning the row-major Q block into operand fragments at the start (while the first K/V tile lands in
  // Ks[0] / Vs[0]) and the accumulators into row-major O at the end.
  __shared__ __attribute__((aligned(1024))) uint16_t Xs[2][TILE];

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

  // Tiles are visited in rotated order: start at the tile whose index is a multiple of the
  // window's tile count (one exists in every full range), run up to t_hi, wrap to t_lo.  The
  // online softmax does not care about the order, and the query blocks of one (batch, head)
  // that run side by side then read the same K/V tile at the same step, so one fetch into the
  // L2 serves all of them.  With no window every range starts at tile 0 and nothing is rotated.
  const int t_lo = row_lo(p, q0) / kTBN;
  const int t_hi = min(q0 + kBM - 1, p.T - 1) / kTBN;
  const int n_tiles = t_hi - t_lo + 1;
  int t_first = t_lo;
  if (p.period > 0) {
    const int c = (t_lo + p.period - 1) / p.period * p.period;
    if (c <= t_hi) t_first = c;
  }

  const uint16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
  const uint16_t* vbase = p.v + b * p.v_sb + h * p.v_sh;

  // ---- global -> LDS copies ------------------------------------------------------------------
  // Wavefront copy j of a tile moves rows RPL*j .. RPL*j+RPL-1 (1 KiB); lane i lands at chunk
  // position i % CPR of row i / CPR, so it fetches the chunk that belongs there (the swizzle is
  // applied on the global side).  This wavefront issues the copies wave, wave + 4, ...: their rows
  // are 16 apart, the swizzles of such rows coincide, so one per-lane offset serves all of them and
  // the row step goes into the wavefront-uniform base.
  const int ld_row = lane / CPR, ld_pos = lane % CPR;
  const int r0 = RPL * wave + ld_row;
  const int k_off = 2 * (r0 * (int)p.k_st + 8 * (ld_pos ^ swz_k(r0)));   // bytes
  const int v_off = 2 * (r0 * (int)p.v_st + 8 * (ld_pos ^ swz_v(r0)));
  const uint32_t ks_lds = lds_address(&Ks[0][0]) + 1024 * wave, vs_lds = lds_address(&Vs[0][0]) + 1024 * wave;
  // The copies walk the tiles in visiting order; the source pointers move by one tile per step and go
  // back to the first tile of the range once (kept incrementally: the scalar unit would otherwise
  // rebuild two 64-bit products per step).
  const int64_t k_step = (int64_t)kTBN * p.k_st, v_step = (int64_t)kTBN * p.v_st;
  const uint16_t* const k_lo = kbase + t_lo * k_step;
  const uint16_t* const v_lo = vbase + t_lo * v_step;
  int t_cp = t_first;                                   // tile the next copy_tiles() call fetches
  const uint16_t* kt = kbase + t_first * k_step;
  const uint16_t* vt = vbase + t_first * v_step;
  auto copy_tiles = [&](int buf) {
    const int kv0 = t_cp * kTBN;
    if (kv0 + kTBN <= p.T) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        copy16_to_lds_async(kt + (int64_t)(4 * RPL * i) * p.k_st, k_off, ks_lds + 2 * (buf * TILE) + 4096 * i);
        copy16_to_lds_async(vt + (int64_t)(4 * RPL * i) * p.v_st, v_off, vs_lds + 2 * (buf * TILE) + 4096 * i);
      }
    } else {
      // The tile reaches past the last row: clamp (the surplus rows are masked by causality).
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int r = r0 + 4 * RPL * i;
        const int row = min(r, p.T - 1 - kv0);
        copy16_to_lds_async(kt, 2 * (row * (int)p.k_st + 8 * (ld_pos ^ swz_k(r))), ks_lds + 2 * (buf * TILE) + 4096 * i);
        copy16_to_lds_async(vt, 2 * (row * (int)p.v_st + 8 * (ld_pos ^ swz_v(r))), vs_lds + 2 * (buf * TILE) + 4096 * i);
      }
    }
    if (++t_cp > t_hi) { t_cp = t_lo; kt = k_lo; vt = v_lo; }
    else { kt += k_step; vt += v_step; }
  };
  auto copies_landed = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0), visible to the compiler's wait-count model
    asm volatile("" ::: "memory");
  };
  // The first tile goes out before anything else so that its latency overlaps the Q loads.
  copy_tiles(0);
  int t_cur = t_first;                                  // tile the next iteration works on

  // ---- Q fragments (B operand), RoPE fused -------------------------------------------------------
  // Global loads with whole rows per group of lanes (lane -> row lane / CH, pair chunk lane % CH: the
  // 16 bytes at channel 8 ch and the 16 bytes at HALF + 8 ch, with the matching 32 bytes of the cos and
  // sin rows), rotated in that layout, written to this wavefront's own LDS area in the K tile layout
  // and read back as fragments.  Fetching the fragments straight from global memory would touch 32
  // rows with every instruction (32 bytes of each), and the CU's memory path, which the other
  // workgroups' tile copies share, would be busy four times as long.
  constexpr int CH = HALF / 8;          // pair chunks per row
  constexpr int QRI = 64 / CH;          // rows per load instruction
  constexpr int QT = 32 / QRI;          // loads of each kind per lane
  const uint32_t x_lds = wave == 0 ? lds_address(&Ks[1][0]) : wave == 1 ? lds_address(&Vs[1][0])
                                                                         : lds_address(&Xs[wave - 2][0]);
  bf16x8 qreg[NS];
  {
    const int qr = lane / CH, qc = lane % CH;
    u32x4 x1[QT], x2[QT];
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      const int row = min(qw0 + QRI * j + qr, p.T - 1);
      const uint16_t* qptr = p.q + b * p.q_sb + (int64_t)row * p.q_st + h * p.q_sh + 8 * qc;
      x1[j] = *reinterpret_cast<const u32x4*>(qptr);
      x2[j] = *reinterpret_cast<const u32x4*>(qptr + HALF);
    }
    if (p.cos != nullptr) {
#pragma unroll
      for (int j = 0; j < QT; ++j) {
        const int row = min(qw0 + QRI * j + qr, p.T - 1);
        const float* cr = p.cos + (int64_t)row * HALF + 8 * qc;
        const float* sr = p.sin + (int64_t)row * HALF + 8 * qc;
        float a1[8], a2[8], y1[8], y2[8];
        unpack8(x1[j], a1);
        unpack8(x2[j], a2);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = cr[e], sn = sr[e];
          y1[e] = rope_lo(a1[e], a2[e], c, sn);
          y2[e] = rope_hi(a1[e], a2[e], c, sn);
        }
        x1[j] = pack8(y1);
        x2[j] = pack8(y2);
      }
    }
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      const int r = QRI * j + qr;
      *(u32x4 __attribute__((address_space(3)))*)(size_t)(x_lds + 2 * (r * D + 8 * (qc ^ swz_k(r)))) = x1[j];
      *(u32x4 __attribute__((address_space(3)))*)(size_t)(x_lds + 2 * (r * D + 8 * ((CH + qc) ^ swz_k(r)))) = x2[j];
    }
    const uint32_t q_a0 = x_lds + 2 * (lq * D + 8 * (lh ^ swz_k(lq)));
#pragma unroll
    for (int s = 0; s < NS; ++s)
      qreg[s] = __builtin_bit_cast(bf16x8, *(const u32x4 __attribute__((address_space(3)))*)(size_t)(q_a0 ^ (32u * s)));
  }

  // Operand addresses inside a tile (LDS byte addresses of buffer 0).  The swizzles are XORs on the
  // chunk index, so the K fragment of contraction slice s sits at k_a0 ^ (32 s) and the V fragment of
  // output tile dt at v_a0 ^ (64 dt): one register each instead of one per fragment.
  //   K (A operand of S^T): row = key lq, slice s wants chunk (2s + lh) ^ swz_k(lq).
  //   V (A operand of O^T, LDS transpose read): the lane's block of 16 covers output channels
  //   32dt + 16*(block & 1) + 0..15 and keys 4*lh + 0..3 (+8, +16 as immediates); lane i of the
  //   block addresses key i/4, channels 4*(i%4)..+3 and receives channel i, four keys.
  const uint32_t k_a0 = lds_address(&Ks[0][0]) + 2 * (lq * D + 8 * (lh ^ swz_k(lq)));
  uint32_t v_a0;
  {
    const int i16 = lane & 15, vrow = 4 * lh + (i16 >> 2);
    const int chunk = 2 * ((lane >> 4) & 1) + ((i16 & 3) >> 1);
    v_a0 = lds_address(&Vs[0][0]) + 2 * (vrow * D + 8 * (chunk ^ swz_v(vrow)) + 4 * (i16 & 1));
  }

  f32x16 oacc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY;  // reference maximum (scaled, log2 domain) of this lane's query
  float l_run = 0.f;        // this lane's share of the running sum

  // One tile of 32 keys.  There is ONE code path for clean and masked tiles (the mask is a small
  // conditional region): two instantiations of the products would make the compiler keep a second
  // copy of the accumulators across the join.
  auto process_tile = [&](auto buf_tag, int kv0, bool masked) {
    constexpr int buf = decltype(buf_tag)::value;
    f32x16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
    // K fragments: four reads ahead of the products (an LDS read takes about as long as four MFMAs;
    // left alone the compiler keeps one fragment register set and waits for every read in turn).
    {
      bf16x8 kf[NS];
#pragma unroll
      for (int s = 0; s < NS; ++s)
        kf[s] = __builtin_bit_cast(bf16x8, *(const u32x4 __attribute__((address_space(3)))*)(size_t)((k_a0 ^ (32u * s)) + 2 * buf * TILE));
#pragma unroll
      for (int s = 0; s < NS; ++s) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s], qreg[s], sacc, 0, 0, 0);
      constexpr int AHEAD = NS < 4 ? NS : 4;
      __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);          // DS reads
#pragma unroll
      for (int s = 0; s < NS - AHEAD; ++s) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);            // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
    }
    if (masked) {
      // element r of this lane is key kv0 + 4lh + c_r with c_r = 8*(r/4) + r%4; visible iff lo <= c_r <= hi
      const int hi = qrow - (kv0 + 4 * lh);
      const int lo = lo_q - (kv0 + 4 * lh);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 8 * (r >> 2) + (r & 3);
        if (c > hi || c < lo) sacc[r] = -INFINITY;
      }
    }
    // Online softmax (log2 domain, lazy rescale): the reference maximum m_run only moves when some
    // query of the wavefront sees a score more than 8 (log2 units) above it; until then
    // probabilities are at most 2^8, which bf16 and the fp32 sums hold without loss, and O is not
    // touched.
    float mt = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) mt = fmaxf(mt, sacc[r]);
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
    bf16x8 pfrag[2];
    float lsum = 0.f;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      float pv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pv[e] = fast_exp2(fmaf(sacc[8 * m + e], p.scale_log2e, -mu));
        lsum += pv[e];
      }
      pfrag[m] = __builtin_bit_cast(bf16x8, pack8(pv));
    }
    l_run += lsum;
    // O^T += V^T P^T
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        lds_u16_ptr vp = (lds_u16_ptr)(size_t)((v_a0 ^ (64u * dt)) + 2 * (buf * TILE + 16 * m * D));
        const u32x2 a0 = lds_read_tr16_as3(vp);            // keys 16m + 4lh + 0..3
        const u32x2 a1 = lds_read_tr16_as3(vp + 8 * D);    // keys 16m + 8 + 4lh + 0..3
        const u32x4 av = {a0.x, a0.y, a1.x, a1.y};
        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av), pfrag[m], oacc[dt], 0, 0, 0);
      }
    }
  };

  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, 1>;
  copies_landed();
  __syncthreads();
  auto iteration = [&](int n, auto buf_tag) {
    constexpr int buf = decltype(buf_tag)::value;
    if (n + 1 < n_tiles) copy_tiles(buf ^ 1);
    const int kv0 = t_cur * kTBN;
    t_cur = t_cur < t_hi ? t_cur + 1 : t_lo;
    if (wave_live && kv0 <= q_w_max && kv0 + kTBN - 1 >= lo_w_min) {
      const bool clean = kv0 + kTBN - 1 <= q_w_min && kv0 >= lo_w_max;
      process_tile(buf_tag, kv0, !clean);
    }
    copies_landed();
    __syncthreads();
  };
  for (int n = 0; n < n_tiles; n += 2) {
    iteration(n, Buf0{});
    if (n + 1 < n_tiles) iteration(n + 1, Buf1{});
  }

  // Epilogue: normalise, turn the accumulators (a lane holds four channels of one query per register
  // group) into row-major bf16 through this wavefront's LDS area, and store 16 bytes per lane with whole
  // rows per group of lanes.  The tile buffers are free: the loop ends with a barrier.
  const float l_tot = pair_sum(l_run);
  const float inv = 1.f / l_tot;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w.x = pack_bf16x2(oacc[dt][4 * g + 0] * inv, oacc[dt][4 * g + 1] * inv);
      w.y = pack_bf16x2(oacc[dt][4 * g + 2] * inv, oacc[dt][4 * g + 3] * inv);
      // channels 32 dt + 8 g + 4 lh + 0..3 of query lq: chunk 4 dt + g, half lh
      *(u32x2 __attribute__((address_space(3)))*)(size_t)(x_lds + 2 * (lq * D + 8 * ((4 * dt + g) ^ swz_k(lq)) + 4 * lh)) = w;
    }
  }
  uint16_t* obase = p.o + b * p.o_sb + h * p.o_sh + 8 * ld_pos;
#pragma unroll
  for (int i = 0; i < 32 / RPL; ++i) {
    const int r = RPL * i + ld_row;
    const u32x4 w = *(const u32x4 __attribute__((address_space(3)))*)(size_t)(x_lds + 2 * (r * D + 8 * (ld_pos ^ swz_k(r))));
    // whole rows, written once and not read again by this kernel: streaming stores leave the last-level
    // cache to q, k and v (the same store from the accumulator layout, 16 bytes per row, must not be
    // streaming: such partial lines are then no longer merged on their way out)
    if (qw0 + r < p.T) __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(obase + (int64_t)(qw0 + r) * p.o_st));
  }
}

// Rotates keys once and stores them with the caller's output strides.  A thread takes one pair chunk
// (8 + 8 channels) of HPT heads of one position: the cos and sin values are fetched once for them.
template <int D, int HPT>
__global__ __launch_bounds__(256) void rope_k_kernel(PrefillParams p) {
  constexpr int HALF = D / 2;
  constexpr int CH = HALF / 8;  // pair chunks per row
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int HG = p.H / HPT;
  const int64_t total = (int64_t)p.B * p.T * HG * CH;
  if (idx >= total) return;
  const int ch = idx % CH;
  const int hg = (idx / CH) % HG;
  const int t = (idx / ((int64_t)CH * HG)) % p.T;
  const int b = idx / ((int64_t)CH * HG * p.T);
  u32x4 r1[HPT], r2[HPT];
  // The unrotated keys are not needed again: read them past the caches, so that q, v and the
  // rotated keys this pass writes are what the attention kernel finds there.
#pragma unroll
  for (int j = 0; j < HPT; ++j) {
    const uint16_t* kp = p.k + b * p.k_sb + (int64_t)t * p.k_st + (hg + j * HG) * p.k_sh + 8 * ch;
    r1[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp));
    r2[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp + HALF));
  }
  const float* cr = p.cos + (int64_t)t * HALF + 8 * ch;
  const float* sr = p.sin + (int64_t)t * HALF + 8 * ch;
  float c[8], sn[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { c[e] = cr[e]; sn[e] = sr[e]; }
#pragma unroll
  for (int j = 0; j < HPT; ++j) {
    float x1[8], x2[8], y1[8], y2[8];
    unpack8(r1[j], x1);
    unpack8(r2[j], x2);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      y1[e] = rope_lo(x1[e], x2[e], c[e], sn[e]);
      y2[e] = rope_hi(x1[e], x2[e], c[e], sn[e]);
    }
    uint16_t* op = p.k_out + b * p.ko_sb + (int64_t)t * p.ko_st + (hg + j * HG) * p.ko_sh + 8 * ch;
    *reinterpret_cast<u32x4*>(op) = pack8(y1);
    *reinterpret_cast<u32x4*>(op + HALF) = pack8(y2);
  }
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
static int launch_mfma(PrefillParams p, hipStream_t s) {
  const int64_t nwg = (int64_t)p.nqb * p.H * p.B;
  if (nwg > 0x7fffffff) {
    set_error("prefill: too many workgroups (%lld)", (long long)nwg);
    return DAISY_ERR_INVALID_ARGUMENT;
  }
  if (p.cos != nullptr) {
    // Pre-pass: rotate K once into k_out, then attend over k_out.
    const int hpt = p.H % 2 == 0 ? 2 : 1;
    const int64_t total = (int64_t)p.B * p.T * (p.H / hpt) * (D / 16);
    if (hpt == 2) hipLaunchKernelGGL((rope_k_kernel<D, 2>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((rope_k_kernel<D, 1>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, p);
    DAISY_CHECK_LAUNCH("rope_k_kernel");
    p.k = p.k_out; p.k_sb = p.ko_sb; p.k_st = p.ko_st; p.k_sh = p.ko_sh;
  }
  hipLaunchKernelGGL((prefill_tile_kernel<D>), dim3((unsigned)nwg), dim3(kPrefillThreads), 0, s, p);
  DAISY_CHECK_LAUNCH("prefill_tile_kernel");
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
  p.period = (window > 0 && window < T) ? (kBM - 1) / kTBN + 1 + (window - 1 + kTBN - 1) / kTBN : 0;
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
  DAISY_CHECK_ARG(flags == 0, "prefill: flags must be 0 (got %d)", flags);

  if (D == 64 || D == 128) {
    auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    DAISY_CHECK_ARG(al16(q) && al16(k) && al16(v) && al16(o) && al16(k_out) && al16(cos) && al16(sin),
                    "prefill: tensors must be 16-byte aligned");
    for (int i = 0; i < 3; ++i) {
      DAISY_CHECK_ARG(q_strides[i] % 8 == 0 && k_strides[i] % 8 == 0 && v_strides[i] % 8 == 0 && o_strides[i] % 8 == 0 &&
                          (!k_out || k_out_strides[i] % 8 == 0),
                      "prefill: strides must be multiples of 8 elements");
    }
    // The keys are rotated once, into k_out, and attended from there: without that buffer every query
    // block would have to rotate every key tile again (measured 3.7 times slower), so it is required.
    DAISY_CHECK_ARG(cos == nullptr || k_out != nullptr,
                    "prefill: cos/sin with head_dim %d need k_out (the rotated keys are written there and attended from there)", D);
    return D == 128 ? launch_mfma<128>(p, s) : launch_mfma<64>(p, s);
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
