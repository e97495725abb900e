// Kernel 3: chunked Kimi Delta Attention forward and its log-decay gate (gfx950).
#include "common.h"
#include <type_traits>

namespace daisy {

// out = -exp(A_log[h]) * softplus(g + bias[h, d]).  VEC = 8: a thread takes 8 consecutive channels
// (Dk a multiple of 8), 16-byte accesses; VEC = 1: one element per thread, any Dk.
template <bool BF16, int VEC>
__global__ __launch_bounds__(256) void kda_gate_kernel(const void* g, const float* A_log, const float* bias, void* out,
                                                       int64_t total, int H, int Dk, float sp_beta, float threshold) {
  const uint32_t vi = blockIdx.x * blockDim.x + threadIdx.x;   // 32-bit index arithmetic (64-bit division is slow)
  const int64_t i = (int64_t)vi * VEC;
  if (i >= total) return;
  const uint32_t per_row = (uint32_t)(H * Dk) / VEC, in_row = vi % per_row;
  const int h = (int)(in_row / (uint32_t)(Dk / VEC));
  const int d = (int)(in_row % (uint32_t)(Dk / VEC)) * VEC;
  const float scale = -expf(A_log[h]);
  float x[VEC], y[VEC];
  if (VEC == 8) {
    if (BF16) unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>((const uint16_t*)g + i)), x);
    else {
      const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>((const float*)g + i));
      const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>((const float*)g + i + 4));
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] = a[e]; x[4 + e] = b[e]; }
    }
  } else {
    x[0] = BF16 ? bf16lo_to_f32(((const uint16_t*)g)[i]) : ((const float*)g)[i];
  }
  float bv[VEC];
  if (bias == nullptr) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) bv[e] = 0.f;
  } else if (VEC == 8) {
    const f32x4 b0 = *reinterpret_cast<const f32x4*>(bias + h * Dk + d), b1 = *reinterpret_cast<const f32x4*>(bias + h * Dk + d + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { bv[e] = b0[e]; bv[(4 + e) % VEC] = b1[e]; }
  } else {
    bv[0] = bias[h * Dk + d];
  }
  const float inv_beta = 1.f / sp_beta;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    // softplus(bx) = max(bx, 0) + log1p(exp(-|bx|)); log1p by its series below 1/64 (error < 1e-6
    // of the value), by the hardware logarithm above (1 + t is exact enough there).
    const float v = x[e] + bv[e];
    const float bx = v * sp_beta;
    const float t = __expf(-fabsf(bx));
    const float l = (t < 0.015625f) ? t * (1.f - t * (0.5f - 0.33333334f * t)) : __logf(1.f + t);
    const float sp = (bx > threshold) ? v : (fmaxf(bx, 0.f) + l) * inv_beta;
    y[e] = scale * sp;
  }
  if (VEC == 8) {
    if (BF16) *reinterpret_cast<u32x4*>((uint16_t*)out + i) = pack8(y);
    else {
      *reinterpret_cast<f32x4*>((float*)out + i) = f32x4{y[0], y[1], y[2], y[3]};
      *reinterpret_cast<f32x4*>((float*)out + i + 4) = f32x4{y[4], y[5], y[6], y[7]};
    }
  } else {
    if (BF16) ((uint16_t*)out)[i] = (uint16_t)(pack_bf16x2(y[0], 0.f) & 0xffffu);
    else ((float*)out)[i] = y[0];
  }
}


// ===========================================================================
// Chunked forward.  Per (batch, head), chunk of C = 64 positions.  The kernels work on 128 key
// channels and 128 value columns; a smaller Dk (a multiple of 8) is served by reading the missing
// channels as zeros (zero channels of q, k and g change nothing: they add nothing to any dot product
// or norm, and their state rows stay zero), and value columns are independent of each other, so any
// Dv (a multiple of 8) is served in passes of up to 128 columns, a short last pass reading zeros.
//
// With G_i the inclusive running sum of the log-decay g inside the chunk (per
// channel), S0 the state at the chunk start, and (per channel products written
// with (.)):
//   A_ij = beta_i sum_d k_id k_jd exp(G_id - G_jd)     (j <  i)
//   P_ij =        sum_d q_id k_jd exp(G_id - G_jd)     (j <= i)
//   (I + A) [W | U0] = diag(beta) [exp(G) (.) K | V]
//   U  = U0 - W S0
//   O  = scale ((exp(G) (.) Q) S0 + P U)
//   S' = diag(exp(G_last)) S0 + (exp(G_last - G) (.) K)^T U
//
// kda_prep_kernel (one workgroup per chunk, all chunks in parallel) produces
// everything that does not depend on S0 into the workspace:
//   Wn  = -W                        bf16 [64][128]   contraction index (channel) permuted
//   Qg  = scale exp(G) (.) Q        bf16 [64][128]   channel permuted
//   Pm  = scale tril(P)             bf16 [64][64]    column (position) permuted
//   KtH + KtL = (exp(G_last - G) (.) K)^T split into two bf16 terms, [128][64], position permuted
//   U0T = U0^T                      fp32 [128][64]
//   dec = exp(G_last)               fp32 [128]
// kda_state_kernel (one workgroup per (batch, head, 32 value columns): two computing
// wavefronts per tile of 16 columns, four data-moving wavefronts that fill the
// double-buffered LDS stages with the chunk data) then walks the chunks in order
// with the fp32 state in registers; every product in it is a
// v_mfma_f32_16x16x32_bf16 whose B operand is an accumulator (S0 or U)
// converted to bf16 in place: in the 16x16 accumulator layout lane l holds
// column l%16 and rows 4*(l/16)+r of each tile, so two stacked tiles give the
// lane 8 contraction indices 16*t + 4*(l/16) + r (t = 0,1; r = 0..3).  The A
// operands are stored with their contraction index permuted inside every
// aligned group of 32 (perm32) so that those 8 indices are 8 consecutive
// elements, one 16-byte load.
//
// Numerics: the 16x16 blocks of A and P run on MFMA with both operands
// referenced to the row before the block (every exponent <= 0 off the diagonal);
// a diagonal block whose total decay exceeds exp(-80) is instead accumulated in
// fp32 pair by pair with exp(G_i - G_j), j < i (no exponent is ever positive, so strong
// decays cannot overflow).  The triangular solve works on 16-row blocks: fp32
// inverses of the diagonal blocks, everything else as products of two-term bf16
// splits (three MFMAs each, relative error ~2^-17).  The state update uses the
// same two-term split of both operands, which keeps the state error near fp32.
// ===========================================================================
constexpr int KC = 64;    // chunk length
constexpr int KD = 128;   // Dk = Dv
constexpr int KVS = 16;   // value columns per state wavefront
constexpr size_t kChunkBytes = (size_t)KC * KD * 2 * 2 + KC * KC * 2 + (size_t)KD * KC * 2 * 2 + (size_t)KD * KC * 4 + KD * 4;

struct KdaParams {
  const uint16_t* q; const uint16_t* k; const uint16_t* v;
  const void* g; int g_bf16; const float* beta;
  const float* s0; uint16_t* o; float* s_out;
  int B, T, H, NC; float scale; int l2norm; float l2eps;
  int Dk, Dv;     // the tensors' own widths: Dk <= 128 key channels, Dv value columns
  int v0, nv;     // this pass covers value columns v0 .. v0 + nv - 1 (nv <= 128)
  uint16_t* Wn; uint16_t* Qg; uint16_t* Pm; uint16_t* KtH; uint16_t* KtL; float* U0T; float* dec;
  // Sequences packed along the token axis of a batch of one (B == 1, T = all tokens): n_seq > 0,
  // bounds [n_seq + 1] = sanitised running lengths, seq_chunk0 [n_seq + 1] = first chunk slot of
  // every sequence, chunk_seq [NC] = sequence of every chunk slot; all three are written on the
  // device by kda_chunk_table_kernel, NC is the host's upper bound T / 64 + n_seq on the slots.
  int n_seq; const int32_t* bounds; const int32_t* seq_chunk0; const int32_t* chunk_seq;
  int nc_total;   // chunk slots per head in the workspace: B * NC, or NC for a packed batch
};

// Where a sequence lives: token rows [tok0, tok_end) of the flattened [B * T] token axis and
// chunk slots [c0, c0 + nc) of the workspace.  A batch element is a sequence of its own.
struct SeqSpan { int tok0, tok_end, c0, nc; };
__device__ __forceinline__ SeqSpan seq_span(const KdaParams& p, int seq) {
  SeqSpan s;
  if (p.n_seq > 0) {
    s.tok0 = p.bounds[seq]; s.tok_end = p.bounds[seq + 1];
    s.c0 = p.seq_chunk0[seq]; s.nc = p.seq_chunk0[seq + 1] - s.c0;
  } else {
    s.tok0 = seq * p.T; s.tok_end = s.tok0 + p.T;
    s.c0 = seq * p.NC; s.nc = p.NC;
  }
  return s;
}

// Chunk slots of packed sequences, built on the device so that the host never reads the bounds.
// bounds = cu_seqlens forced to start at 0, to stay within 0..T and not to decrease (whatever the
// caller passed, no kernel then leaves the tensors); seq_chunk0 = running sum of ceil(len / 64);
// chunk_seq = the sequence of every slot.  One workgroup; thread i takes a run of sequences.
__global__ __launch_bounds__(256) void kda_chunk_table_kernel(const int32_t* cu, int n_seq, int T, int nc_max,
                                                              int32_t* bounds, int32_t* seq_chunk0, int32_t* chunk_seq) {
  __shared__ int part[256];
  const int tid = threadIdx.x;
  const int per = (n_seq + 1 + 255) / 256;
  const int a = min(tid * per, n_seq + 1), b = min(a + per, n_seq + 1);
  int hi = 0;
  for (int i = a; i < b; ++i) hi = max(hi, min(max(cu[i], 0), T));
  part[tid] = hi;
  __syncthreads();
  hi = 0;
  for (int w = 0; w < tid; ++w) hi = max(hi, part[w]);
  for (int i = a; i < b; ++i) {
    hi = max(hi, min(max(cu[i], 0), T));
    bounds[i] = (i == 0) ? 0 : hi;
  }
  __threadfence_block();
  __syncthreads();
  const int per_s = (n_seq + 255) / 256;
  const int sa = min(tid * per_s, n_seq), sb = min(sa + per_s, n_seq);
  int mine = 0;
  for (int i = sa; i < sb; ++i) mine += (bounds[i + 1] - bounds[i] + KC - 1) / KC;
  __syncthreads();
  part[tid] = mine;
  __syncthreads();
  int run = 0;
  for (int w = 0; w < tid; ++w) run += part[w];
  for (int i = sa; i < sb; ++i) {
    const int nc = (bounds[i + 1] - bounds[i] + KC - 1) / KC;
    seq_chunk0[i] = min(run, nc_max);
    for (int c = 0; c < nc; ++c)
      if (run + c < nc_max) chunk_seq[run + c] = i;
    run += nc;
  }
  if (tid == 255) seq_chunk0[n_seq] = min(run, nc_max);   // the last thread's run ends at the total
}

// Stored position of contraction index x inside its aligned group of 32: bits (4,3,2) -> (3,2,4).
__host__ __device__ constexpr int perm32(int x) { return (x & ~0x1c) | ((x & 0x0c) << 1) | ((x & 0x10) >> 2); }
__host__ __device__ constexpr int perm32_inv(int p) { return (p & ~0x1c) | ((p & 0x18) >> 1) | ((p & 0x04) << 2); }

__device__ __forceinline__ f32x4 lds_f4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }

// Off-diagonal 16x16 blocks of A in LDS: block (I, J), J < I, has index I(I-1)/2 + J.
__host__ __device__ constexpr int off_block(int I, int J) { return I * (I - 1) / 2 + J; }

// A float as two bf16 terms (value = hi + lo up to 2^-17 relative).
__device__ __forceinline__ void split_bf16(float x, float& hi, float& lo) { hi = round_bf16(x); lo = x - hi; }

__global__ __launch_bounds__(256, 2) void kda_prep_kernel(KdaParams p) {
  __shared__ __attribute__((aligned(16))) float G[KC][KD + 4];       // inclusive running log-decay (rows 4 banks apart: 16 rows read side by side do not collide); later staging for Wn
  __shared__ __attribute__((aligned(16))) uint16_t Kr[KC][KD + 8];   // k as given (bf16)
  __shared__ __attribute__((aligned(16))) uint16_t QV[KC][KD + 8];   // q as given; v as given once A and P are done
  __shared__ __attribute__((aligned(16))) float Ad[4][16][16];       // diagonal blocks of A, [block][column j][row i]; later T = (I + A_II)^-1 as bf16 hi | lo
  __shared__ __attribute__((aligned(16))) uint16_t AoH[6][16][16];   // -A, off-diagonal blocks (off_block), [row][column], bf16 high term
  __shared__ __attribute__((aligned(16))) uint16_t AoL[6][16][16];   //   ... low term
  __shared__ float rk[KC], rq[KC], bt[KC];                           // 1/|k|, 1/|q|, beta (0 for padded rows)
  __shared__ int steep[4];                                           // per 16-row block: total decay beyond exp(-80); 2 when some 4 rows of it alone go beyond
  auto& Qr = QV;
  auto& Vr = QV;

  // Chunk slot gc of the workspace; token rows t0 .. t_end - 1 of the flattened token axis are this
  // chunk's share of its sequence (t_end = end of the sequence: the last chunk may be short).
  const int h = blockIdx.y;
  const int gc = blockIdx.z * p.NC + blockIdx.x;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  int t0, t_end;
  if (p.n_seq > 0) {
    if (gc >= p.seq_chunk0[p.n_seq]) return;      // a surplus slot (the grid covers the upper bound)
    const SeqSpan sp = seq_span(p, p.chunk_seq[gc]);
    t0 = sp.tok0 + (gc - sp.c0) * KC;
    t_end = sp.tok_end;
  } else {
    t0 = blockIdx.z * p.T + blockIdx.x * KC;
    t_end = (blockIdx.z + 1) * p.T;
  }
  const int n_live = t_end - t0;                  // live rows of the chunk when < 64
  const int64_t ci = (int64_t)h * p.nc_total + gc;
  // Addresses: a wavefront-uniform 64-bit base per array (the chunk's first token row of this head, or
  // the chunk's slot in the workspace) plus a 32-bit offset per lane.  Written out once here: as one
  // 64-bit expression per access the row products were rebuilt per lane and load (seven vector
  // instructions each, three of them at a quarter of the rate).
  const uint32_t row_stride = (uint32_t)p.H * (uint32_t)p.Dk;     // elements between token rows of one head (q, k, g)
  const uint32_t row_stride_v = (uint32_t)p.H * (uint32_t)p.Dv;   //   ... of v
  const int64_t tok_base = ((int64_t)t0 * p.H + h) * p.Dk;        // first element of the chunk's first row
  const uint16_t* const q_c = p.q + tok_base;
  const uint16_t* const k_c = p.k + tok_base;
  const uint16_t* const v_c = p.v + ((int64_t)t0 * p.H + h) * p.Dv + p.v0;
  const float* const beta_c = p.beta + ((int64_t)t0 * p.H + h);
  uint16_t* const qg_c = p.Qg + ci * KC * KD;
  uint16_t* const pm_c = p.Pm + ci * KC * KC;
  float* const u0_c = p.U0T + ci * KD * KC;

  // ---- phase 0a: G = cumsum(g) -----------------------------------------------
  // Every global load of the chunk (g here, then q, k, v and beta of phase 0b) goes out before
  // the first result is used, so that the memory latency is paid once.  Inputs are read once and
  // the workspace is written once: both as streaming (non-temporal) accesses.
  if (tid < 4) steep[tid] = 0;
  __syncthreads();
  const int cc = tid & 15, r4 = tid >> 4;
  u32x4 qraw[4], vraw[4], kraw[4];
  float btv[4];
  {
    const int d = tid & 127, half = __builtin_amdgcn_readfirstlane(tid >> 7);   // the row of a g load is wavefront-uniform
    const bool d_live = d < p.Dk;                 // channels beyond Dk read as zero (their loads re-read the last channel)
    const int dl = min(d, p.Dk - 1);
    float gv[32];
    // Rows past the end re-read the last row (always valid) and are zeroed afterwards, so that
    // the loads carry no branches and all go out together; the dtype is decided once, outside
    // the loops, for the same reason.  bf16 g: the two channels of a pair read the same dword
    // (no sub-dword loads) and take their half.
    uint32_t graw[32];
    if (p.g_bf16) {
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        const uint32_t* row = reinterpret_cast<const uint32_t*>(p.g) + ((tok_base + (uint32_t)min(32 * half + i, n_live - 1) * row_stride) >> 1);
        graw[i] = __builtin_nontemporal_load(row + (uint32_t)(dl >> 1));
      }
    } else {
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        const uint32_t* row = reinterpret_cast<const uint32_t*>(p.g) + (tok_base + (uint32_t)min(32 * half + i, n_live - 1) * row_stride);
        graw[i] = __builtin_nontemporal_load(row + (uint32_t)dl);
      }
    }
    const bool g16 = p.g_bf16 != 0, odd = (d & 1) != 0;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const float x = g16 ? (odd ? bf16hi_to_f32(graw[i]) : bf16lo_to_f32(graw[i])) : __uint_as_float(graw[i]);
      gv[i] = (32 * half + i < n_live && d_live) ? x : 0.f;
    }
    const int ccl = min(cc, p.Dk / 8 - 1), ccv = min(cc, p.nv / 8 - 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = r4 + 16 * i;
      const int rc = min(r, n_live - 1);
      const uint32_t off = (uint32_t)rc * row_stride + 8u * ccl;
      kraw[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(k_c + off));
      vraw[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(v_c + (uint32_t)rc * row_stride_v + 8u * ccv));
      qraw[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q_c + off));
      btv[i] = beta_c[(uint32_t)rc * (uint32_t)p.H];
    }
    __builtin_amdgcn_sched_barrier(0);
    // G holds the running sum in units of log 2 (g * log2(e)): every exponential below is a bare
    // v_exp_f32.
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      acc += gv[i] * kLog2e;
      G[32 * half + i][d] = acc;
    }
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      float tot = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) tot += gv[16 * blk + i];
      if (tot < -80.f) atomicMax(&steep[2 * half + blk], 1);
      // ... and whether four consecutive rows alone decay that far (then no reference row per
      // group of four keeps the exponents of the matrix-core path in range)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const float t4 = gv[16 * blk + 4 * g4] + gv[16 * blk + 4 * g4 + 1] + gv[16 * blk + 4 * g4 + 2] + gv[16 * blk + 4 * g4 + 3];
        if (t4 < -80.f) atomicMax(&steep[2 * half + blk], 2);
      }
    }
    __syncthreads();
    if (half == 1) {
      const float add = G[31][d];
#pragma unroll
      for (int i = 0; i < 32; ++i) G[32 + i][d] += add;
    }
  }

  // ---- phase 0b: raw q, k to LDS, row norms, beta ---------------------------
  float rqv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r4 + 16 * i;
    const bool live = r < n_live;
    const u32x4 zero4 = {0, 0, 0, 0};
    if (!live || 8 * cc >= p.Dk) { kraw[i] = zero4; qraw[i] = zero4; }
    if (!live || 8 * cc >= p.nv) vraw[i] = zero4;
    float kf[8], qf[8];
    unpack8(kraw[i], kf);
    unpack8(qraw[i], qf);
    float sk = 0.f, sq = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { sk = fmaf(kf[e], kf[e], sk); sq = fmaf(qf[e], qf[e], sq); }
    sk = group_sum<16>(sk);
    sq = group_sum<16>(sq);
    const float nk = p.l2norm ? rsqrtf(sk + p.l2eps) : 1.f;
    rqv[i] = p.l2norm ? rsqrtf(sq + p.l2eps) : 1.f;
    if (cc == 0) {
      rk[r] = nk;
      rq[r] = rqv[i];
      bt[r] = live ? btv[i] : 0.f;
    }
    *reinterpret_cast<u32x4*>(&Kr[r][8 * cc]) = kraw[i];
    *reinterpret_cast<u32x4*>(&Qr[r][8 * cc]) = qraw[i];
  }
  __syncthreads();

  // ---- phase 1: Qg = scale exp(G) q/|q| (channel permuted), dec = exp(G_last) ----
  {
    const int pos0 = ((cc >> 2) << 5) | ((cc & 1) << 4) | (((cc >> 1) & 1) << 2);  // perm32(8*cc)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = r4 + 16 * i;
      float qf[8], o8[8];
      unpack8(qraw[i], qf);
      const f32x4 g0 = lds_f4(&G[r][8 * cc]), g1 = lds_f4(&G[r][8 * cc + 4]);
      const float sc = p.scale * rqv[i];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        o8[e] = sc * __builtin_amdgcn_exp2f(g0[e]) * qf[e];
        o8[4 + e] = sc * __builtin_amdgcn_exp2f(g1[e]) * qf[4 + e];
      }
      const u32x4 pk = pack8(o8);
      uint16_t* dst = qg_c + (uint32_t)(r * KD + pos0);
      u32x2 lo2 = {pk.x, pk.y}, hi2 = {pk.z, pk.w};
      __builtin_nontemporal_store(lo2, reinterpret_cast<u32x2*>(dst));        // channels 8cc+0..3
      __builtin_nontemporal_store(hi2, reinterpret_cast<u32x2*>(dst + 8));    // channels 8cc+4..7
    }
    if (r4 == 0) {
      const f32x4 g0 = lds_f4(&G[KC - 1][8 * cc]), g1 = lds_f4(&G[KC - 1][8 * cc + 4]);
      f32x4 d0, d1;
#pragma unroll
      for (int e = 0; e < 4; ++e) { d0[e] = __builtin_amdgcn_exp2f(g0[e]); d1[e] = __builtin_amdgcn_exp2f(g1[e]); }
      float* dd = p.dec + ci * KD + 8 * cc;
      *reinterpret_cast<f32x4*>(dd) = d0;
      *reinterpret_cast<f32x4*>(dd + 4) = d1;
    }
  }

  // ---- phase 2a: 16x16 blocks of A and P on MFMA --------------------------------
  // Block (I, J), J <= I: both operands are referenced to the row before block I, so the row
  // factor exp(G_i - G_ref) is <= 1 and, for J < I, so is the column factor exp(G_ref - G_j).
  // For a diagonal block (J == I) the column factor grows to exp(total decay of the block); the
  // block takes this path only when that total stays below 80 (flag `steep` otherwise).
  // The row operands (k_i f_i, q_i f_i with f_i = exp(G_i - G_ref)) of a block row are made once
  // and serve every block of the row.
  bf16x8 va[4], vq[4];
  auto row_operands = [&](int I) {
    const int li = lane & 15, q4 = lane >> 4;
    const int ref = 16 * I - 1;   // -1 for the first block: G_ref = 0
    const int ri = 16 * I + li;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int d0 = 32 * m + 8 * q4;
      float ki[8], qi[8], ak[8], aq[8];
      unpack8(*reinterpret_cast<const u32x4*>(&Kr[ri][d0]), ki);
      unpack8(*reinterpret_cast<const u32x4*>(&Qr[ri][d0]), qi);
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        const f32x4 gi = lds_f4(&G[ri][d0 + 4 * hf]);
        const f32x4 gr = (ref >= 0) ? lds_f4(&G[max(ref, 0)][d0 + 4 * hf]) : zero;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float fi = __builtin_amdgcn_exp2f(gi[e] - gr[e]);
          ak[4 * hf + e] = ki[4 * hf + e] * fi;
          aq[4 * hf + e] = qi[4 * hf + e] * fi;
        }
      }
      va[m] = __builtin_bit_cast(bf16x8, pack8(ak));
      vq[m] = __builtin_bit_cast(bf16x8, pack8(aq));
    }
  };
  auto mfma_block = [&](int I, int J) {
    const int li = lane & 15, q4 = lane >> 4;
    const int ref = 16 * I - 1;
    const int rj = 16 * J + li;
    f32x4 accA = {0.f, 0.f, 0.f, 0.f}, accP = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int d0 = 32 * m + 8 * q4;
      float kj[8], bk[8];
      unpack8(*reinterpret_cast<const u32x4*>(&Kr[rj][d0]), kj);
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        const f32x4 gj = lds_f4(&G[rj][d0 + 4 * hf]);
        const f32x4 gr = (ref >= 0) ? lds_f4(&G[max(ref, 0)][d0 + 4 * hf]) : zero;
#pragma unroll
        for (int e = 0; e < 4; ++e) bk[4 * hf + e] = kj[4 * hf + e] * __builtin_amdgcn_exp2f(gr[e] - gj[e]);
      }
      const bf16x8 vb = __builtin_bit_cast(bf16x8, pack8(bk));
      accA = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[m], vb, accA, 0, 0, 0);
      // P comes out transposed (operands swapped: both operand layouts hold 8 contraction indices of
      // one row / column per lane): a lane then owns four consecutive columns of one row of P, one
      // 8-byte store instead of four 2-byte ones.
      accP = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vb, vq[m], accP, 0, 0, 0);
    }
    // accA: lane holds column j = 16J + li, rows i = 16I + 4*q4 + r
    const int j = 16 * J + li;
    const float rkj = rk[j];
    f32x4 av;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * I + 4 * q4 + r;
      av[r] = bt[i] * rk[i] * rkj * accA[r];
    }
    {
      // accP: lane holds row i = 16I + li, columns j = 16J + 4*q4 + r (stored positions perm32(j): the
      // four are consecutive, perm32 keeps the low two bits)
      const int ip = 16 * I + li, jp = 16 * J + 4 * q4;
      const f32x4 rk4 = lds_f4(&rk[jp]);
      const float qs = p.scale * rq[ip];
      float pv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) pv[r] = (jp + r <= ip) ? qs * rk4[r] * accP[r] : 0.f;
      const u32x2 w = {pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3])};
      *reinterpret_cast<u32x2*>(pm_c + (uint32_t)(ip * KC + perm32(jp))) = w;
    }
    if (I == J) {
      *reinterpret_cast<f32x4*>(&Ad[I][li][4 * q4]) = av;   // entries with i <= j are never read
    } else {
      const int ob = off_block(I, J);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float hi, lo;
        split_bf16(-av[r], hi, lo);
        AoH[ob][4 * q4 + r][li] = (uint16_t)(pack_bf16x2(hi, 0.f) & 0xffffu);
        AoL[ob][4 * q4 + r][li] = (uint16_t)(pack_bf16x2(lo, 0.f) & 0xffffu);
      }
    }
  };
  // Blocks by wavefront, normally: 0 -> (0,0), (3,3); 1 -> (1,0), (1,1); 2 -> (2,0), (2,1), (2,2);
  // 3 -> (3,0), (3,1), (3,2).  A diagonal block whose decay is too steep for the MFMA path (some
  // channel beyond exp(-80) across the block: the column factors could overflow) is accumulated
  // in fp32 pair by pair with exp(G_i - G_j), j < i, where no exponent is ever positive.
  auto steep_diagonal = [&](int I) {
    const int il = lane >> 2, dq = lane & 3;
    const int ri = 16 * I + il;
    float a[16], pp[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) { a[j] = 0.f; pp[j] = 0.f; }
#pragma unroll 1
    for (int dc = 0; dc < 4; ++dc) {
      const int d0 = 32 * dq + 8 * dc;
      float ki[8], qi[8];
      unpack8(*reinterpret_cast<const u32x4*>(&Kr[ri][d0]), ki);
      unpack8(*reinterpret_cast<const u32x4*>(&Qr[ri][d0]), qi);
      const f32x4 gi0 = lds_f4(&G[ri][d0]), gi1 = lds_f4(&G[ri][d0 + 4]);
#pragma unroll
      for (int j = 15; j >= 0; --j) {
        const int rj = 16 * I + j;
        float kj[8];
        unpack8(*reinterpret_cast<const u32x4*>(&Kr[rj][d0]), kj);
        // exp(G_i - G_j) for j < i: the exponent is a sum of log-decays, never positive; rows at or
        // above the diagonal take the factor 1 (only j == i is used, by P).
        const f32x4 gj0 = lds_f4(&G[rj][d0]), gj1 = lds_f4(&G[rj][d0 + 4]);
        const bool below = j < il;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float diff = (e < 4) ? gi0[e & 3] - gj0[e & 3] : gi1[e & 3] - gj1[e & 3];
          const float t = kj[e] * (below ? __builtin_amdgcn_exp2f(diff) : 1.f);
          a[j] = fmaf(ki[e], t, a[j]);
          pp[j] = fmaf(qi[e], t, pp[j]);
        }
      }
    }
    const float bi = bt[ri] * rk[ri], qs = p.scale * rq[ri];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      float av = dpp_add<0x4E>(dpp_add<0xB1>(a[j]));    // sum over the 4 channel quarters
      float pv = dpp_add<0x4E>(dpp_add<0xB1>(pp[j]));
      if ((j & 3) == dq) {
        const int rj = 16 * I + j;
        const float rkj = rk[rj];
        if (j < il) Ad[I][j][il] = bi * rkj * av;
        pv = (j <= il) ? qs * rkj * pv : 0.f;
        pm_c[(uint32_t)(ri * KC + perm32(rj))] = (uint16_t)(pack_bf16x2(pv, 0.f) & 0xffffu);
      }
    }
  };
  // A steep diagonal block on the matrix cores after all: with one reference row per group of four
  // rows (the row before the group) every row factor exp(G_i - G_ref(i)) is <= 1, and the column
  // factors exp(G_ref - G_j) are <= 1 for columns of earlier groups and at most the decay of four
  // rows inside the group.  Pass r multiplies all rows by the columns scaled for the reference of
  // group r; the accumulator layout gives rows 4r..4r+3 to the lanes with q4 == r, which keep
  // that pass's result.  Four passes, a fifth of the exponentials of the pairwise path.
  auto steep_diagonal_mfma = [&](int I) {
    const int li = lane & 15, q4 = lane >> 4;
    const int ri = 16 * I + li;
    // The diagonal block is the last of its segment: the row operands of the block row are not needed
    // again and their registers take the ones made here.
    bf16x8 (&sa)[4] = va;
    bf16x8 (&sq)[4] = vq;
    {
      const int ref = 16 * I + (li & ~3) - 1;   // -1: the chunk's first rows, G_ref = 0
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int d0 = 32 * m + 8 * q4;
        float ki[8], qi[8], ak[8], aq[8];
        unpack8(*reinterpret_cast<const u32x4*>(&Kr[ri][d0]), ki);
        unpack8(*reinterpret_cast<const u32x4*>(&Qr[ri][d0]), qi);
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
          const f32x4 gi = lds_f4(&G[ri][d0 + 4 * hf]);
          const f32x4 gr = (ref >= 0) ? lds_f4(&G[max(ref, 0)][d0 + 4 * hf]) : zero;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float fi = __builtin_amdgcn_exp2f(gi[e] - gr[e]);
            ak[4 * hf + e] = ki[4 * hf + e] * fi;
            aq[4 * hf + e] = qi[4 * hf + e] * fi;
          }
        }
        sa[m] = __builtin_bit_cast(bf16x8, pack8(ak));
        sq[m] = __builtin_bit_cast(bf16x8, pack8(aq));
      }
    }
    f32x4 accA = {0.f, 0.f, 0.f, 0.f}, accP = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
    for (int r = 0; r < 4; ++r) {
      const int ref = 16 * I + 4 * r - 1;
      const bool live = (li >> 2) <= r;     // later columns are above the diagonal for every row of the group
      f32x4 pa = {0.f, 0.f, 0.f, 0.f}, pp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int d0 = 32 * m + 8 * q4;
        float kj[8], bk[8];
        unpack8(*reinterpret_cast<const u32x4*>(&Kr[ri][d0]), kj);
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
          const f32x4 gj = lds_f4(&G[ri][d0 + 4 * hf]);
          const f32x4 gr = (ref >= 0) ? lds_f4(&G[max(ref, 0)][d0 + 4 * hf]) : zero;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            bk[4 * hf + e] = live ? kj[4 * hf + e] * __builtin_amdgcn_exp2f(fminf(gr[e] - gj[e], 120.f)) : 0.f;
        }
        const bf16x8 vb = __builtin_bit_cast(bf16x8, pack8(bk));
        pa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sa[m], vb, pa, 0, 0, 0);
        pp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sq[m], vb, pp, 0, 0, 0);
      }
      if (q4 == r) { accA = pa; accP = pp; }
    }
    // accumulator: lane holds column j = 16I + li, rows i = 16I + 4*q4 + r
    const int j = 16 * I + li;
    const float rkj = rk[j];
    f32x4 av;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * I + 4 * q4 + r;
      av[r] = bt[i] * rk[i] * rkj * accA[r];
      const float pv = (j <= i) ? p.scale * rq[i] * rkj * accP[r] : 0.f;
      pm_c[(uint32_t)(i * KC + perm32(j))] = (uint16_t)(pack_bf16x2(pv, 0.f) & 0xffffu);
    }
    *reinterpret_cast<f32x4*>(&Ad[I][li][4 * q4]) = av;   // entries with i <= j are never read
  };
  {
    // Segments (block row I, columns jlo..jhi) per wavefront, 4 bits each, two per wavefront
    // (0xf.. = none).  A steep diagonal block costs about as much as five others, so when there
    // is one the blocks are dealt differently: 0 -> (0,0), (3,0..1); 1 -> (1,1), (3,2);
    // 2 -> (2,0..2); 3 -> (3,3), (1,0).
    const bool any_steep = (steep[0] | steep[1] | steep[2] | steep[3]) != 0;
    constexpr uint32_t kPlain[4] = {0x333000u, 0xfff101u, 0xfff202u, 0xfff203u};   // (jhi, jlo, I) second | first
    constexpr uint32_t kSteep[4] = {0x103000u, 0x223111u, 0xfff202u, 0x001333u};
    uint32_t plan = any_steep ? kSteep[0] : kPlain[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) if (wave == w) plan = any_steep ? kSteep[w] : kPlain[w];
    for (int sg = 0; sg < 2; ++sg, plan >>= 12) {
      const int I = plan & 15, jlo = (plan >> 4) & 15, jhi = (plan >> 8) & 15;
      if (I == 15) break;
      row_operands(I);
      for (int J = jlo; J <= jhi; ++J) {
        if (J == I && steep[I] == 2) steep_diagonal(I);
        else if (J == I && steep[I] == 1) steep_diagonal_mfma(I);
        else mfma_block(I, J);
      }
    }
    // The state kernel reads P in 16x32 pieces; blocks (0,1) and (2,3) lie above the diagonal.
    if (wave == 1) {
      const int li = lane & 15, q4 = lane >> 4;
#pragma unroll
      for (int I = 0; I < 4; I += 2)
#pragma unroll
        for (int r = 0; r < 4; ++r) pm_c[(uint32_t)((16 * I + 4 * q4 + r) * KC + perm32(16 * (I + 1) + li))] = 0;
    }
  }
  __syncthreads();

  // Q is no longer needed: V takes its place in LDS (right-hand side of the solve).
#pragma unroll
  for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(&Vr[r4 + 16 * i][8 * cc]) = vraw[i];

  __syncthreads();   // V is in place

  // ---- phase 4: (I + A) X = diag(beta) [exp(G) K | V] by blocks of 16 rows on MFMA ----
  //     X_I = T_I (B_I - sum_{J<I} A_IJ X_J),   T_I = (I + A_II)^-1.
  // The 256 right-hand-side columns form 16 tiles of 16; wavefront w solves tiles w, w+4 (W part)
  // and w+8, w+12 (U part).  In the 16x16x32 MFMA a lane's accumulator holds rows 4q..4q+3 of a
  // block for one column; the same four values, split into two bf16 terms, are that lane's
  // share of the next product's right operand when contraction slot (q, e) stands for row
  // 4q+e of block J (e < 4) and of block J+1 (e >= 4) -- so X never leaves the registers.  The left
  // operands (T and -A, two bf16 terms each) come from LDS in that slot order; every product is
  // three MFMAs (hi*hi, hi*lo, lo*hi).
  {
    const int li = lane & 15, q4 = lane >> 4;
    // 4a: T of diagonal block `wave`, one column per lane (lanes 16.. repeat the work of lane & 15).
    {
      float tc[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) tc[i] = (i == li) ? 1.f : 0.f;
#pragma unroll
      for (int j = 0; j < 15; ++j) {
        f32x4 ar[4];
#pragma unroll
        for (int i4 = (j + 1) / 4; i4 < 4; ++i4) ar[i4] = lds_f4(&Ad[wave][j][4 * i4]);
        const float xj = tc[j];
#pragma unroll
        for (int i = j + 1; i < 16; ++i) tc[i] = fmaf(-ar[i >> 2][i & 3], xj, tc[i]);
      }
      // The wavefront has read all of its block before any lane writes: T replaces A_II in place.
      uint16_t* Th = reinterpret_cast<uint16_t*>(&Ad[wave][0][0]);   // [16][16] high terms, then [16][16] low terms
      if (lane < 16) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float hi, lo;
          split_bf16(tc[i], hi, lo);
          Th[i * 16 + li] = (uint16_t)(pack_bf16x2(hi, 0.f) & 0xffffu);
          Th[256 + i * 16 + li] = (uint16_t)(pack_bf16x2(lo, 0.f) & 0xffffu);
        }
      }
    }
    // 4b: right-hand sides in accumulator layout: C[tile][block][r] = B[16*block + 4*q4 + r][column].
    f32x4 C[4][4];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      const int col = 16 * (wave + 4 * (tt & 1)) + li;
#pragma unroll
      for (int I = 0; I < 4; ++I) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = 16 * I + 4 * q4 + r;
          C[tt][I][r] = (tt < 2) ? bt[i] * rk[i] * __builtin_amdgcn_exp2f(G[i][col]) * bf16lo_to_f32(Kr[i][col])
                                 : bt[i] * bf16lo_to_f32(Vr[i][col]);
        }
      }
    }
    // ---- phase 3 (placed here, where few registers are live): (exp(G_last - G) k/|k|)^T as two
    // bf16 terms, position permuted.  Thread (d, gh) makes four 16-byte pieces of row d; stored
    // from here they would hit 64 different lines per instruction, so they go through LDS (the
    // space of G and of K, both dead after the barrier) and leave as whole rows.
    u32x4 kth[4], ktl[4];
    const int kd = tid & 127, kgh = tid >> 7;
    {
      const float glast = G[KC - 1][kd];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int g8 = 4 * kgh + i;   // group of 8 stored positions
        float hi[8], lo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int pos = perm32_inv(8 * g8 + e);
          const float val = __builtin_amdgcn_exp2f(glast - G[pos][kd]) * bf16lo_to_f32(Kr[pos][kd]) * rk[pos];
          hi[e] = round_bf16(val);
          lo[e] = val - hi[e];
        }
        kth[i] = pack8(hi);
        ktl[i] = pack8(lo);
      }
    }
    __syncthreads();   // G, K and V have been read by everyone (their space becomes staging); T is in place
    char* KtHst = reinterpret_cast<char*>(&G[0][0]) + KC * KD * 2;   // [128][64] bf16 behind the Wn tile
    char* KtLst = reinterpret_cast<char*>(&Kr[0][0]);                // [128][64] bf16
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int off = kd * 128 + 16 * ((4 * kgh + i) ^ (kd & 7));    // pieces of a row swizzled against bank conflicts
      *reinterpret_cast<u32x4*>(KtHst + off) = kth[i];
      *reinterpret_cast<u32x4*>(KtLst + off) = ktl[i];
    }
    // 4c: left operands.  Slot (q4, e): e < 4 -> column 4*q4+e of the first block, e >= 4 -> of the second.
    auto lds_half = [&](const uint16_t* row) -> u32x2 { return *reinterpret_cast<const u32x2*>(row + 4 * q4); };
    auto frag = [&](u32x2 a, u32x2 b) -> bf16x8 { u32x4 w = {a.x, a.y, b.x, b.y}; return __builtin_bit_cast(bf16x8, w); };
    const u32x2 none = {0u, 0u};
    bf16x8 Tf[4][2], Af[4][2];   // Af: (1,0) | (2,0)(2,1) | (3,0)(3,1) | (3,2)
#pragma unroll
    for (int I = 0; I < 4; ++I) {
      const uint16_t* Th = reinterpret_cast<const uint16_t*>(&Ad[I][0][0]);
      Tf[I][0] = frag(lds_half(Th + li * 16), none);
      Tf[I][1] = frag(lds_half(Th + 256 + li * 16), none);
    }
    Af[0][0] = frag(lds_half(&AoH[off_block(1, 0)][li][0]), none);
    Af[0][1] = frag(lds_half(&AoL[off_block(1, 0)][li][0]), none);
    Af[1][0] = frag(lds_half(&AoH[off_block(2, 0)][li][0]), lds_half(&AoH[off_block(2, 1)][li][0]));
    Af[1][1] = frag(lds_half(&AoL[off_block(2, 0)][li][0]), lds_half(&AoL[off_block(2, 1)][li][0]));
    Af[2][0] = frag(lds_half(&AoH[off_block(3, 0)][li][0]), lds_half(&AoH[off_block(3, 1)][li][0]));
    Af[2][1] = frag(lds_half(&AoL[off_block(3, 0)][li][0]), lds_half(&AoL[off_block(3, 1)][li][0]));
    Af[3][0] = frag(lds_half(&AoH[off_block(3, 2)][li][0]), none);
    Af[3][1] = frag(lds_half(&AoL[off_block(3, 2)][li][0]), none);

    // Two bf16 terms of an accumulator as halves of a right operand.
    auto split_acc = [&](const f32x4& x, u32x2& hi, u32x2& lo) {
      float h[4], l[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) split_bf16(x[e], h[e], l[e]);
      hi.x = pack_bf16x2(h[0], h[1]); hi.y = pack_bf16x2(h[2], h[3]);
      lo.x = pack_bf16x2(l[0], l[1]); lo.y = pack_bf16x2(l[2], l[3]);
    };
    // acc += L * R with L = Lf[0] + Lf[1], R = (hi | lo)
    auto mul3 = [&](const bf16x8 (&Lf)[2], bf16x8 Rh, bf16x8 Rl, f32x4 acc) -> f32x4 {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Lf[1], Rh, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Lf[0], Rl, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Lf[0], Rh, acc, 0, 0, 0);
      return acc;
    };
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    uint16_t* Wst = reinterpret_cast<uint16_t*>(&G[0][0]);   // [64][128] bf16 staging
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      f32x4 X[4];
      u32x2 xh[4], xl[4], ch, cl;
      split_acc(C[tt][0], ch, cl);
      X[0] = mul3(Tf[0], frag(ch, none), frag(cl, none), zero4);
      split_acc(X[0], xh[0], xl[0]);
      C[tt][1] = mul3(Af[0], frag(xh[0], none), frag(xl[0], none), C[tt][1]);
      split_acc(C[tt][1], ch, cl);
      X[1] = mul3(Tf[1], frag(ch, none), frag(cl, none), zero4);
      split_acc(X[1], xh[1], xl[1]);
      C[tt][2] = mul3(Af[1], frag(xh[0], xh[1]), frag(xl[0], xl[1]), C[tt][2]);
      C[tt][3] = mul3(Af[2], frag(xh[0], xh[1]), frag(xl[0], xl[1]), C[tt][3]);
      split_acc(C[tt][2], ch, cl);
      X[2] = mul3(Tf[2], frag(ch, none), frag(cl, none), zero4);
      split_acc(X[2], xh[2], xl[2]);
      C[tt][3] = mul3(Af[3], frag(xh[2], none), frag(xl[2], none), C[tt][3]);
      split_acc(C[tt][3], ch, cl);
      X[3] = mul3(Tf[3], frag(ch, none), frag(cl, none), zero4);

      const int col = 16 * (wave + 4 * (tt & 1)) + li;
      if (tt < 2) {
        const int pc = perm32(col);
#pragma unroll
        for (int I = 0; I < 4; ++I)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            Wst[(16 * I + 4 * q4 + r) * KD + pc] = (uint16_t)(pack_bf16x2(-X[I][r], 0.f) & 0xffffu);
      } else {
        float* dst = u0_c + (uint32_t)(col * KC + 4 * q4);
#pragma unroll
        for (int I = 0; I < 4; ++I) __builtin_nontemporal_store(X[I], reinterpret_cast<f32x4*>(dst + 16 * I));
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ch = tid + 256 * i;   // 16-byte chunk of the [64][128] bf16 tile
      __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(Wst + 8 * ch), reinterpret_cast<u32x4*>(p.Wn + ci * KC * KD + 8 * ch));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ch = tid + 256 * i;   // 16-byte chunk of a [128][64] bf16 tile
      const int off = (ch >> 3) * 128 + 16 * ((ch & 7) ^ ((ch >> 3) & 7));
      __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(KtHst + off), reinterpret_cast<u32x4*>(p.KtH + ci * KD * KC + 8 * ch));
      __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(KtLst + off), reinterpret_cast<u32x4*>(p.KtL + ci * KD * KC + 8 * ch));
    }
  }
}

__device__ __forceinline__ bf16x8 pack_acc2(const f32x4& t0, const f32x4& t1) {
  u32x4 r;
  r.x = pack_bf16x2(t0[0], t0[1]); r.y = pack_bf16x2(t0[2], t0[3]);
  r.z = pack_bf16x2(t1[0], t1[1]); r.w = pack_bf16x2(t1[2], t1[3]);
  return __builtin_bit_cast(bf16x8, r);
}

// LDS stage of the state kernel: everything of one chunk that does not depend on the value
// column, copied with asynchronous global->LDS copies while the previous chunk is computed.
// Rows are stored with their 16-byte chunks XOR-swizzled (chunk c of row r at position
// c ^ f(r)) so that the 16-byte operand reads of 16 consecutive rows fall into 16 different
// slots of the 256-byte bank window: f(r) = r & 15 for 256-byte rows, (r >> 1) & 7 for 128-byte
// rows (two rows per window).
constexpr int KCT = 2;                        // tiles of 16 value columns per workgroup
constexpr int KSW = 2 * KCT;                  // computing wavefronts per workgroup: two per column tile
constexpr int KPW = 4;                        // data-moving wavefronts per workgroup
constexpr int kStageWn = 0;                   // [64][128] bf16
constexpr int kStageQg = 16384;               // [64][128] bf16
constexpr int kStageKtH = 32768;              // [128][64] bf16
constexpr int kStageKtL = 49152;              // [128][64] bf16
constexpr int kStageDec = 65536;               // [128] fp32: the chunk's total decay per key channel
constexpr int kStageBytes = 65536 + 1024;

typedef __attribute__((address_space(3))) const char* lds_cptr;
__device__ __forceinline__ bf16x8 lds_bf16x8(lds_cptr p) {
  return __builtin_bit_cast(bf16x8, *(const u32x4 __attribute__((address_space(3)))*)p);
}

// The chunk-to-chunk chain sets the time of this kernel.  Two measures shorten a link:
//  * the work of one tile of 16 value columns is shared by two wavefronts: wavefront `hf` keeps
//    the state rows (key channels) [64 hf, 64 hf + 64) and produces the output rows (positions)
//    [32 hf, 32 hf + 32) of the chunk.  Both need all of U = U0 - W S0, whose contraction runs
//    over every key channel: each computes it in full (16 MFMAs, duplicated) from its own half of
//    the state and a bf16 copy of the partner's half, handed over through LDS at the barrier
//    that ends a chunk -- no barrier inside a chunk;
//  * a fifth wavefront does nothing but move data: it issues the global->LDS copies of the next
//    chunk (a CU takes in only ~30 bytes per cycle, so issuing 64 KB blocks a wavefront for
//    longer than the arithmetic of a chunk lasts) and stores the previous chunk's output rows,
//    which the computing wavefronts leave in LDS, as whole 64-byte row pieces.
__global__ __launch_bounds__(64 * (KSW + KPW), 1) void kda_state_kernel(KdaParams p) {
  __shared__ __attribute__((aligned(1024))) char stage[2][kStageBytes];
  __shared__ __attribute__((aligned(16))) u32x4 xch[2][KSW][2][64];           // [chunk parity][wavefront][k-group][lane]
  __shared__ __attribute__((aligned(16))) uint16_t ost[2][KC][KVS * KCT];      // [chunk parity][position][value column]

  // Keep the column groups of one (batch, head) on one XCD: they read the same chunk data.
  int vid = blockIdx.x;
  if ((gridDim.x & 7) == 0) vid = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int NGRP = (p.nv + KVS * KCT - 1) / (KVS * KCT);   // groups of 32 value columns in this pass
  const int grp = vid % NGRP, bh = vid / NGRP;
  const int h = bh % p.H, b = bh / p.H;     // b: batch element, or sequence of a packed batch
  const SeqSpan sp = seq_span(p, b);
  const int nc = sp.nc;                      // chunks of this sequence (0 for an empty one)
  const int64_t ci0 = (int64_t)h * p.nc_total + sp.c0;
  const int lane = threadIdx.x & 63, ln = lane & 15, q4 = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  if (wave >= KSW) {
    const int pw = wave - KSW;
    // ================= data-moving wavefront =================
    const uint32_t stage_lds = lds_address(&stage[0][0]);
    // 256-byte rows: a wavefront copy moves 4 rows; lane i lands at row i/16, position i%16.
    // 128-byte rows: 8 rows per copy; lane i lands at row i/8, position i%8.
    int src256[4], src128[2];   // source byte offsets inside a group of 16 rows, by (copy index & 3) / (& 1)
#pragma unroll
    for (int v = 0; v < 4; ++v) src256[v] = (4 * v + (lane >> 4)) * 256 + 16 * ((lane & 15) ^ ((4 * v + (lane >> 4)) & 15));
#pragma unroll
    for (int v = 0; v < 2; ++v) src128[v] = (8 * v + (lane >> 3)) * 128 + 16 * ((lane & 7) ^ ((4 * v + (lane >> 4)) & 7));
    auto issue_copies = [&](int n, int st) {
      const int64_t ci = ci0 + n;
      const uint32_t dst = stage_lds + st * kStageBytes;
      const uint16_t* wn = p.Wn + ci * KC * KD;
      const uint16_t* qg = p.Qg + ci * KC * KD;
      const uint16_t* kh = p.KtH + ci * KD * KC;
      const uint16_t* kl = p.KtL + ci * KD * KC;
#pragma unroll
      for (int j = pw; j < 16; j += KPW) {
        copy16_to_lds_async(wn + (j >> 2) * 2048, src256[j & 3], dst + kStageWn + j * 1024);
        copy16_to_lds_async(qg + (j >> 2) * 2048, src256[j & 3], dst + kStageQg + j * 1024);
      }
#pragma unroll
      for (int j = pw; j < 16; j += KPW) {
        copy16_to_lds_async(kh + (j >> 1) * 1024, src128[j & 1], dst + kStageKtH + j * 1024);
        copy16_to_lds_async(kl + (j >> 1) * 1024, src128[j & 1], dst + kStageKtL + j * 1024);
      }
      // the 512 bytes of the chunk's decay ride along (half a copy): fetched by the computing wavefronts
      // themselves they were four more vector-memory instructions per wavefront and chunk, and the number
      // of such instructions a CU issues per chunk is what the chunk time follows
      if (pw == 0 && lane < 32) copy16_to_lds_async(reinterpret_cast<const uint16_t*>(p.dec + ci * KD), lane * 16, dst + kStageDec);
    };
    // The four workgroups of a (batch, head) copy the same 64 KB per chunk at about the same
    // time and would all wait out the full HBM latency.  Each touches a quarter of a later chunk
    // (this wavefront 4 KB of it, one dword per 64 bytes) so that the copies find their lines in
    // L2.  The touching load is the youngest of an iteration: vmcnt(1) then means that every copy
    // has landed (loads return in order) while the touch stays in flight.  Its target register
    // is tied up for the whole loop.
    uint32_t touched = 0;
    constexpr int kAhead = 3;
    auto touch_ahead = [&](int n) {
      const int64_t ci = ci0 + n;
      const uint16_t* base = (grp == 0) ? p.Wn + ci * KC * KD : (grp == 1) ? p.Qg + ci * KC * KD
                           : (grp == 2) ? p.KtH + ci * KD * KC : p.KtL + ci * KD * KC;
      asm volatile("global_load_dword %0, %1, %2" : "+v"(touched) : "v"(pw * 4096 + lane * 64), "s"(base) : "memory");
    };
    // Output rows of chunk n: 64 rows x 64 bytes, 16 bytes per lane and pass.
    auto store_o = [&](int n) {
#pragma unroll
      for (int k = pw; k < 4; k += KPW) {
        const int idx = 64 * k + lane, row = idx >> 2, piece = idx & 3;
        const u32x4 v = *reinterpret_cast<const u32x4*>(&ost[n & 1][row][8 * piece]);
        const int tok = sp.tok0 + n * KC + row;
        if (tok < sp.tok_end && KVS * KCT * grp + 8 * piece < p.nv)
          *reinterpret_cast<u32x4*>(p.o + ((int64_t)tok * p.H + h) * p.Dv + p.v0 + KVS * KCT * grp + 8 * piece) = v;
      }
    };
    if (nc > 0) issue_copies(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    asm volatile("" ::: "memory");
    __syncthreads();
    for (int n = 0; n < nc; ++n) {
      if (n > 0) store_o(n - 1);
      if (n + 1 < nc) issue_copies(n + 1, (n + 1) & 1);
      if (NGRP == 4 && n + kAhead < nc) {
        touch_ahead(n + kAhead);
        __builtin_amdgcn_s_waitcnt(0x0F71);   // vmcnt(1)
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
      asm volatile("" ::: "memory");
      __syncthreads();
    }
    if (nc > 0) store_o(nc - 1);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" :: "v"(touched));
    return;
  }

  // ================= computing wavefronts =================
  const int ct = wave >> 1, hf = wave & 1;
  const int vcol = KVS * (KCT * grp + ct) + ln;

  // ---- per-lane LDS read offsets (bytes, inside a stage) ------------------------------------
  // A operand of a 16x16x32 MFMA: lane (row ln, k-group q4) reads chunk 4m + q4 of its row.
  // Groups of 32 key channels are taken own half first: local group mm is channel group
  // 2 hf + mm for mm < 2 and 2 (1 - hf) + mm - 2 after that.
  int rdk[4], rd128[2];
#pragma unroll
  for (int mm = 0; mm < 4; ++mm) {
    const int m = (mm < 2) ? 2 * hf + mm : 2 * (1 - hf) + (mm - 2);
    rdk[mm] = ln * 256 + 16 * ((4 * m + q4) ^ ln);
  }
#pragma unroll
  for (int m = 0; m < 2; ++m) rd128[m] = ln * 128 + 16 * ((4 * m + q4) ^ ((ln >> 1) & 7));
  lds_cptr stage0 = (lds_cptr)&stage[0][0];

  // State tile i: rows (key channels) 16*(4 hf + i) + 4*q4 + r, column vcol of this pass; rows beyond Dk and
  // columns beyond Dv do not exist in the caller's [Dk, Dv] state: they are zero and stay zero.
  const bool col_live = vcol < p.nv;
  f32x4 S[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 16 * (4 * hf + i) + 4 * q4 + r;
      S[i][r] = (p.s0 && col_live && row < p.Dk) ? p.s0[((int64_t)bh * p.Dk + row) * p.Dv + p.v0 + vcol] : 0.f;
    }
  }

  // What depends on the value column comes straight from global memory, one chunk ahead: U0
  // (accumulator initial value of U) and this wavefront's rows of P as left operand.
  auto load_direct = [&](int n, f32x4* u0, bf16x8 (*pa)[2]) {
    const int64_t ci = ci0 + n;
    const float* src = p.U0T + (ci * KD + vcol) * KC + 4 * q4;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) u0[mt] = *reinterpret_cast<const f32x4*>(src + 16 * mt);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int m = 0; m < 2; ++m)
        pa[i][m] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(p.Pm + (ci * KC + 16 * (2 * hf + i) + ln) * KC + 32 * m + 8 * q4));
  };
  // Two sets, used in turn by even and odd chunks (the chunk loop is unrolled by two so that no
  // register copy, which would have to wait for the loads, sits between them and their use).
  f32x4 u0[2][4];
  bf16x8 pa[2][2][2];
  bf16x8 Sb[4];   // the state as right operand, by local channel group
  Sb[0] = pack_acc2(S[0], S[1]);
  Sb[1] = pack_acc2(S[2], S[3]);
  xch[0][wave][0][lane] = __builtin_bit_cast(u32x4, Sb[0]);
  xch[0][wave][1][lane] = __builtin_bit_cast(u32x4, Sb[1]);
  if (nc > 0) load_direct(0, u0[0], pa[0]);
  __syncthreads();

  auto chunk_step = [&](int n, auto parity) {
    constexpr int st = decltype(parity)::value;
    f32x4 (&u0c)[4] = u0[st];
    f32x4 dcc[4];
    bf16x8 (&pac)[2][2] = pa[st];
    // The direct loads of the next chunk go out first thing, ahead of the burst of copies of the
    // data-moving wavefronts (the memory pipeline of a CU is one queue: behind that burst they
    // would block this wavefront for thousands of cycles), and are waited for at the end of the
    // chunk, so that no wait for them can end up behind newer loads.
    if (n + 1 < nc) load_direct(n + 1, u0[st ^ 1], pa[st ^ 1]);
    __builtin_amdgcn_sched_barrier(0);
    lds_cptr sb = stage0 + st * kStageBytes;

    // LDS operands are read in two batches ahead of the MFMAs that use them instead of each next
    // to its MFMA, where every MFMA waited for a full LDS latency.
    Sb[2] = __builtin_bit_cast(bf16x8, xch[st][wave ^ 1][0][lane]);
    Sb[3] = __builtin_bit_cast(bf16x8, xch[st][wave ^ 1][1][lane]);
    bf16x8 wa[4][4], qa[2][4], kh[4][2], kl[4][2];
#pragma unroll
    for (int mm = 0; mm < 4; ++mm) {
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) wa[mt][mm] = lds_bf16x8(sb + kStageWn + 4096 * mt + rdk[mm]);
#pragma unroll
      for (int i = 0; i < 2; ++i) qa[i][mm] = lds_bf16x8(sb + kStageQg + 4096 * (2 * hf + i) + rdk[mm]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) dcc[i] = *(const f32x4 __attribute__((address_space(3)))*)(sb + kStageDec + 4 * (16 * (4 * hf + i) + 4 * q4));
    __builtin_amdgcn_sched_barrier(0);

    // U = U0 + (-W) S0 (all four row tiles) and O = Qg S0 (this wavefront's two row tiles).
    // Row tile mt: positions 16*mt + 4*q4 + r, column vcol.
    f32x4 U[4], O[2];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) U[mt] = u0c[mt];
#pragma unroll
    for (int i = 0; i < 2; ++i) O[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mm = 0; mm < 4; ++mm) {
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) U[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[mt][mm], Sb[mm], U[mt], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 2; ++i) O[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[i][mm], Sb[mm], O[i], 0, 0, 0);
    }
    // The operands of the state update are read while those MFMAs run.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int m = 0; m < 2; ++m) {
        kh[i][m] = lds_bf16x8(sb + kStageKtH + 2048 * (4 * hf + i) + rd128[m]);
        kl[i][m] = lds_bf16x8(sb + kStageKtL + 2048 * (4 * hf + i) + rd128[m]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    bf16x8 Uh[2], Ul[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      Uh[m] = pack_acc2(U[2 * m], U[2 * m + 1]);
      f32x4 l0, l1;
      const u32x4 hb = __builtin_bit_cast(u32x4, Uh[m]);
      l0[0] = U[2 * m][0] - bf16lo_to_f32(hb.x); l0[1] = U[2 * m][1] - bf16hi_to_f32(hb.x);
      l0[2] = U[2 * m][2] - bf16lo_to_f32(hb.y); l0[3] = U[2 * m][3] - bf16hi_to_f32(hb.y);
      l1[0] = U[2 * m + 1][0] - bf16lo_to_f32(hb.z); l1[1] = U[2 * m + 1][1] - bf16hi_to_f32(hb.z);
      l1[2] = U[2 * m + 1][2] - bf16lo_to_f32(hb.w); l1[3] = U[2 * m + 1][3] - bf16hi_to_f32(hb.w);
      Ul[m] = pack_acc2(l0, l1);
    }

    // S = exp(G_last) (.) S + Kt^T U, with both operands split into two bf16 terms.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 4; ++r) S[i][r] *= dcc[i][r];
    }
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        S[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kh[i][m], Uh[m], S[i], 0, 0, 0);
        S[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kh[i][m], Ul[m], S[i], 0, 0, 0);
        S[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kl[i][m], Uh[m], S[i], 0, 0, 0);
      }
    }
    // O += Pm U (scale already folded into Qg and Pm).  Positions 32..63 of U only reach the
    // output rows of the second half (P is zero above the diagonal).
#pragma unroll
    for (int i = 0; i < 2; ++i) O[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pac[i][0], Uh[0], O[i], 0, 0, 0);
    if (hf) {
#pragma unroll
      for (int i = 0; i < 2; ++i) O[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pac[i][1], Uh[1], O[i], 0, 0, 0);
    }
    // The new state goes to the partner as soon as it exists.
    Sb[0] = pack_acc2(S[0], S[1]);
    Sb[1] = pack_acc2(S[2], S[3]);
    xch[st ^ 1][wave][0][lane] = __builtin_bit_cast(u32x4, Sb[0]);
    xch[st ^ 1][wave][1][lane] = __builtin_bit_cast(u32x4, Sb[1]);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        ost[st][16 * (2 * hf + i) + 4 * q4 + r][KVS * ct + ln] = (uint16_t)(pack_bf16x2(O[i][r], 0.f) & 0xffffu);
    }

    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the direct loads of the next chunk
    __syncthreads();
  };
  for (int n = 0; n < nc; n += 2) {
    chunk_step(n, std::integral_constant<int, 0>{});
    if (n + 1 < nc) chunk_step(n + 1, std::integral_constant<int, 1>{});
  }
  if (p.s_out != nullptr && col_live) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = 16 * (4 * hf + i) + 4 * q4 + r;
        if (row < p.Dk) p.s_out[((int64_t)bh * p.Dk + row) * p.Dv + p.v0 + vcol] = S[i][r];
      }
  }
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
  const bool vec = Dk % 8 == 0 && (reinterpret_cast<uintptr_t>(g) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  const int64_t nblk = ((vec ? total / 8 : total) + 255) / 256;
  DAISY_CHECK_ARG(nblk <= 0x7fffffff, "kda_gate: too many elements");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)nblk), block(256);
  if (vec && io_is_bf16) hipLaunchKernelGGL((kda_gate_kernel<true, 8>), grid, block, 0, s, g, A_log, bias, out, total, H, Dk, softplus_beta, threshold);
  else if (vec) hipLaunchKernelGGL((kda_gate_kernel<false, 8>), grid, block, 0, s, g, A_log, bias, out, total, H, Dk, softplus_beta, threshold);
  else if (io_is_bf16) hipLaunchKernelGGL((kda_gate_kernel<true, 1>), grid, block, 0, s, g, A_log, bias, out, total, H, Dk, softplus_beta, threshold);
  else hipLaunchKernelGGL((kda_gate_kernel<false, 1>), grid, block, 0, s, g, A_log, bias, out, total, H, Dk, softplus_beta, threshold);
  DAISY_CHECK_LAUNCH("kda_gate_kernel");
  return DAISY_OK;
}


// Chunk slots of the workspace: B * ceil(T / 64), or for n_seq packed sequences of T tokens in all
// the upper bound T / 64 + n_seq on sum(ceil(len / 64)).
static size_t kda_chunk_slots(int B, int T, int n_seq) {
  return n_seq > 0 ? (size_t)T / KC + (size_t)n_seq : (size_t)B * ((size_t)(T + KC - 1) / KC);
}
static size_t kda_table_bytes(int T, int n_seq) {
  if (n_seq <= 0) return 0;
  const size_t ints = 2 * ((size_t)n_seq + 1) + kda_chunk_slots(1, T, n_seq);
  return (ints * sizeof(int32_t) + 255) & ~(size_t)255;
}

// Head widths the kernels serve: Dk a multiple of 8 up to 128, Dv any multiple of 8.
static bool kda_dims_ok(int Dk, int Dv) { return Dk >= 8 && Dk <= KD && Dk % 8 == 0 && Dv >= 8 && Dv % 8 == 0; }

extern "C" size_t daisy_kda_workspace_bytes(int B, int T, int H, int Dk, int Dv, int chunk) {
  if (B <= 0 || T <= 0 || H <= 0 || !kda_dims_ok(Dk, Dv) || chunk != KC) return 0;
  return kda_chunk_slots(B, T, 0) * H * kChunkBytes;
}

extern "C" size_t daisy_kda_varlen_workspace_bytes(int T, int n_seq, int H, int Dk, int Dv, int chunk) {
  if (T <= 0 || n_seq <= 0 || H <= 0 || !kda_dims_ok(Dk, Dv) || chunk != KC) return 0;
  return kda_chunk_slots(1, T, n_seq) * H * kChunkBytes + kda_table_bytes(T, n_seq);
}

// Shared by the batched and the packed entry point (n_seq == 0: batched).
static int kda_chunk_launch(const void* q, const void* k, const void* v,
                            const void* g, int g_is_bf16, const float* beta,
                            const int32_t* cu_seqlens, int n_seq,
                            const float* initial_state, void* o, float* final_state,
                            int B, int T, int H, int Dk, int Dv, int chunk,
                            float scale, int l2norm_qk, float l2_eps,
                            void* workspace, size_t workspace_bytes, void* stream) {
  DAISY_CHECK_SUPPORTED(kda_dims_ok(Dk, Dv), "kda: Dk=%d, Dv=%d not supported (Dk: a multiple of 8 up to %d; Dv: a multiple of 8)", Dk, Dv, KD);
  DAISY_CHECK_SUPPORTED(chunk == KC, "kda: chunk=%d not supported (must be %d)", chunk, KC);
  DAISY_CHECK_ARG(q && k && v && g && beta && o, "kda: q, k, v, g, beta and o must be non-NULL");
  DAISY_CHECK_ARG(B > 0 && T > 0 && H > 0, "kda: B=%d, T=%d, H=%d must be positive", B, T, H);
  DAISY_CHECK_ARG(B <= 65535 && H <= 65535, "kda: B and H must each be <= 65535");
  DAISY_CHECK_ARG((int64_t)B * T <= 0x7fffffff, "kda: B*T too large");
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(al16(q) && al16(k) && al16(v) && al16(g) && al16(o) && al16(workspace),
                  "kda: tensors and workspace must be 16-byte aligned");
  const size_t slots = kda_chunk_slots(B, T, n_seq);
  const size_t need = slots * H * kChunkBytes + kda_table_bytes(T, n_seq);
  if (!workspace || workspace_bytes < need) {
    set_error("kda: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    return DAISY_ERR_WORKSPACE;
  }
  DAISY_CHECK_ARG(slots <= 0x7fffffff && (int64_t)(n_seq > 0 ? n_seq : B) * H * (KD / (KVS * KCT)) <= 0x7fffffff,
                  "kda: too many chunks or sequences");
  KdaParams p;
  p.q = (const uint16_t*)q; p.k = (const uint16_t*)k; p.v = (const uint16_t*)v;
  p.g = g; p.g_bf16 = g_is_bf16; p.beta = beta;
  p.s0 = initial_state; p.o = (uint16_t*)o; p.s_out = final_state;
  p.B = B; p.T = T; p.H = H;
  p.NC = n_seq > 0 ? (int)slots : (T + KC - 1) / KC;
  p.nc_total = (int)slots;
  p.scale = scale; p.l2norm = l2norm_qk; p.l2eps = l2_eps;
  const size_t chunks = slots * H;
  char* w = (char*)workspace;
  p.Wn = (uint16_t*)w;  w += chunks * KC * KD * 2;
  p.Qg = (uint16_t*)w;  w += chunks * KC * KD * 2;
  p.KtH = (uint16_t*)w; w += chunks * KD * KC * 2;
  p.KtL = (uint16_t*)w; w += chunks * KD * KC * 2;
  p.U0T = (float*)w;    w += chunks * KD * KC * 4;
  p.Pm = (uint16_t*)w;  w += chunks * KC * KC * 2;
  p.dec = (float*)w;    w += chunks * KD * 4;
  p.n_seq = n_seq; p.bounds = p.seq_chunk0 = p.chunk_seq = nullptr;
  hipStream_t s = (hipStream_t)stream;
  if (n_seq > 0) {
    int32_t* tab = (int32_t*)w;
    int32_t* bounds = tab; int32_t* seq_chunk0 = tab + n_seq + 1; int32_t* chunk_seq = tab + 2 * (n_seq + 1);
    hipLaunchKernelGGL(kda_chunk_table_kernel, dim3(1), dim3(256), 0, s, cu_seqlens, n_seq, T, (int)slots, bounds, seq_chunk0, chunk_seq);
    DAISY_CHECK_LAUNCH("kda_chunk_table_kernel");
    p.bounds = bounds; p.seq_chunk0 = seq_chunk0; p.chunk_seq = chunk_seq;
  }
  const int n_streams = n_seq > 0 ? n_seq : B;    // independent recurrences per head
  p.Dk = Dk; p.Dv = Dv;
  // Value columns are independent: passes of up to 128 columns, each through the same workspace (the
  // launches of one stream run in order).
  for (int v0 = 0; v0 < Dv; v0 += KD) {
    p.v0 = v0; p.nv = Dv - v0 < KD ? Dv - v0 : KD;
    const int groups = (p.nv + KVS * KCT - 1) / (KVS * KCT);
    hipLaunchKernelGGL(kda_prep_kernel, dim3(p.NC, H, n_seq > 0 ? 1 : B), dim3(256), 0, s, p);
    DAISY_CHECK_LAUNCH("kda_prep_kernel");
    hipLaunchKernelGGL(kda_state_kernel, dim3((unsigned)(n_streams * H * groups)), dim3(64 * (KSW + KPW)), 0, s, p);
    DAISY_CHECK_LAUNCH("kda_state_kernel");
  }
  return DAISY_OK;
}

extern "C" int daisy_kda_chunk_fwd(const void* q, const void* k, const void* v,
                                   const void* g, int g_is_bf16, const float* beta,
                                   const float* initial_state, void* o, float* final_state,
                                   int B, int T, int H, int Dk, int Dv, int chunk,
                                   float scale, int l2norm_qk, float l2_eps,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  return kda_chunk_launch(q, k, v, g, g_is_bf16, beta, nullptr, 0, initial_state, o, final_state, B, T, H, Dk, Dv, chunk,
                          scale, l2norm_qk, l2_eps, workspace, workspace_bytes, stream);
}

extern "C" int daisy_kda_chunk_varlen_fwd(const void* q, const void* k, const void* v,
                                          const void* g, int g_is_bf16, const float* beta,
                                          const int32_t* cu_seqlens, int n_seq,
                                          const float* initial_state, void* o, float* final_state,
                                          int T, int H, int Dk, int Dv, int chunk,
                                          float scale, int l2norm_qk, float l2_eps,
                                          void* workspace, size_t workspace_bytes, void* stream) {
  DAISY_CHECK_ARG(cu_seqlens != nullptr && n_seq >= 1, "kda_varlen: cu_seqlens and n_seq >= 1 are required");
  return kda_chunk_launch(q, k, v, g, g_is_bf16, beta, cu_seqlens, n_seq, initial_state, o, final_state, 1, T, H, Dk, Dv,
                          chunk, scale, l2norm_qk, l2_eps, workspace, workspace_bytes, stream);
}
