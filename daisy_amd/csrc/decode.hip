// Kernel 2: split-K single-token decode over a bf16 KV cache (gfx950).
//
// One workgroup (4 wavefronts) streams a contiguous range of cache rows of one
// (batch, head).  A row of D bf16 is covered by D/8 lanes with one 16-byte
// load each, so a wavefront load instruction fetches 64*16 = 1 KiB of
// consecutive cache bytes.  Every group of D/8 lanes keeps its own online
// softmax state (max, sum, 8 output channels); the groups of a wavefront are
// merged with cross-lane moves, the wavefronts of a workgroup through LDS, and
// the splits of a (batch, head) -- when there are several -- by a second tiny
// kernel over fp32 partials in the caller's workspace.
//
// HBM traffic per step is the K and V rows once: B*H*n_rows*D*2*2 bytes.
//
// Variants of the same kernel (template flags): PREP takes the new token's rows straight from the
// QKV projection and does the RMS norm, the rotation and the value-embedding mix itself, so that a
// decode step is one launch between the two projections; F16C reads and appends to a cache kept in
// fp16.  The step's position comes as a launch argument or from one int32 in device memory that
// the kernel reads when it runs: launch arguments then do not change from step to step and a
// recorded launch (HIP graph) can be replayed for every later token.
#include "common.h"

#include <mutex>

namespace daisy {

struct DecodeParams {
  const uint16_t* q; int64_t q_sb, q_sh;
  const uint16_t* k_new; int64_t kn_sb, kn_sh;
  const uint16_t* v_new; int64_t vn_sb, vn_sh;
  uint16_t* kc; int64_t kc_sb, kc_sh, kc_sr;
  uint16_t* vc; int64_t vc_sb, vc_sh, vc_sr;
  const float* cos_row; const float* sin_row;
  uint16_t* o; int64_t o_sb, o_sh;
  float* partials;  // [B, H, nsplit, D + 2] when nsplit > 1
  int B, H, n_rows, new_idx, write_back, nsplit, rows_per_split;
  float scale_log2e;
  // When set, the step's position t is read from device memory at run time (so that a recorded
  // launch can be replayed for later positions): the cache is a ring of ring_rows slots,
  // n_rows = min(t + 1, ring_rows) of them are live and the new row goes to slot t % ring_rows.
  const int32_t* pos_dev; int ring_rows;
  // For the kernel variant that prepares the rows itself (RMS norm of q, k_new, v_new, RoPE of q
  // and k_new at the step's position, value-embedding mix): the position when it is a launch
  // argument, the rotation tables, and the optional second value row with its gate.
  int pos_host; const float* cos_tab; const float* sin_tab; int table_rows; float eps;
  const uint16_t* ve; int64_t ve_sb, ve_sh; const float* gate;
  int32_t* status;   // optional: receives DAISY_STATUS_* bits the kernel raises (never cleared by it)
};

struct DecodeRange { int n_rows, new_idx, rows_per_split; };

__device__ __forceinline__ DecodeRange decode_range(const DecodeParams& p) {
  DecodeRange r{p.n_rows, p.new_idx, p.rows_per_split};
  if (p.pos_dev != nullptr) {
    const int t = max(p.pos_dev[0], 0);
    r.n_rows = min(t + 1, p.ring_rows);
    r.new_idx = t % p.ring_rows;
    r.rows_per_split = (r.n_rows + p.nsplit - 1) / p.nsplit;
  }
  return r;
}

constexpr int kDecodeThreads = 256;
constexpr int kDecodeWaves = kDecodeThreads / 64;
constexpr int kDecodeUnroll = 4;  // 16-byte loads per lane, tensor and register set (two sets)

// The new token's rows are fetched in two steps -- raw loads first, arithmetic later -- so that the
// kernel can put the first cache-row loads between the two: the rows and the rotation table take a
// memory round trip that the stream of cache rows then does not wait for.
struct RawRow { u32x4 own, par; };   // this lane's 8 channels and the 8 they are rotated with
struct TrigRow { float c[8], s[8]; };

template <int D>
__device__ __forceinline__ RawRow load_raw_row(const uint16_t* vec, int dl, bool with_partner) {
  constexpr int HALF = D / 2;
  RawRow r;
  r.own = *reinterpret_cast<const u32x4*>(vec + dl);
  r.par = with_partner ? *reinterpret_cast<const u32x4*>(vec + (dl < HALF ? dl + HALF : dl - HALF)) : r.own;
  return r;
}
template <int D>
__device__ __forceinline__ TrigRow load_trig_row(const float* cos_row, const float* sin_row, int dl) {
  constexpr int HALF = D / 2;
  const int tl = dl < HALF ? dl : dl - HALF;
  TrigRow t;
#pragma unroll
  for (int i = 0; i < 8; ++i) { t.c[i] = cos_row[tl + i]; t.s[i] = sin_row[tl + i]; }
  return t;
}

// This lane's 8 channels of a [D] bf16 vector rotated with the position's cos/sin row (pairs
// (i, i + D/2)) and rounded to bf16 like the reference does after RoPE, as floats.
template <int D>
__device__ __forceinline__ void rot_row(const RawRow& r, const TrigRow& t, int dl, float* out) {
  const bool lower = dl < D / 2;
  float pf[8];
  unpack8(r.own, out);
  unpack8(r.par, pf);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float y = lower ? rope_lo(out[i], pf[i], t.c[i], t.s[i]) : rope_hi(pf[i], out[i], t.c[i], t.s[i]);
    out[i] = round_bf16(y);
  }
}

// RMS norm of this lane's 8 channels of a [D] bf16 row (statistics over the row's D/8 lanes),
// rounded to bf16 like the norm's output tensor, then the rotation, rounded again: the arithmetic
// and the roundings of qkv_prep_kernel for one row.
template <int D>
__device__ __forceinline__ void norm_rot_row(const RawRow& r, const TrigRow& t, int dl, float eps, float* out) {
  constexpr int LPR = D / 8;
  const bool lower = dl < D / 2;
  float own[8], par[8];
  unpack8(r.own, own);
  unpack8(r.par, par);
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss += own[i] * own[i];
  ss = group_sum<LPR>(ss);
  const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float a = round_bf16(own[i] * rstd), b = round_bf16(par[i] * rstd);
    out[i] = round_bf16(lower ? rope_lo(a, b, t.c[i], t.s[i]) : rope_hi(b, a, t.c[i], t.s[i]));
  }
}

// RMS norm of a value row and, when a second row is given, gate * v + (1 - gate) * ve with every
// product and the sum rounded to bf16 (the roundings of a bf16 tensor library).
template <int D>
__device__ __forceinline__ void norm_mix_row(const u32x4& v_raw, bool with_ve, const u32x4& ve_raw, float g, float eps,
                                             float* out) {
  constexpr int LPR = D / 8;
  float own[8];
  unpack8(v_raw, own);
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss += own[i] * own[i];
  ss = group_sum<LPR>(ss);
  const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = round_bf16(own[i] * rstd);
  if (with_ve) {
    float e[8];
    unpack8(ve_raw, e);
    const float og = round_bf16(1.0f - g);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = round_bf16(round_bf16(g * out[i]) + round_bf16(og * e[i]));
  }
}

// Cache rows in fp16 (the reference's default cache dtype, inference/generate.py:62): eight
// values of a 16-byte piece to floats and back.  bf16 rows convert to fp16 without loss as long as
// they are in fp16's normal range, which normalised keys and values are.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void unpack8_f16(const u32x4& r, float* f) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f16x2 h = __builtin_bit_cast(f16x2, w[i]);
    f[2 * i] = (float)h[0];
    f[2 * i + 1] = (float)h[1];
  }
}
__device__ __forceinline__ u32x4 pack8_f16(const float* f) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f16x2 h = {(_Float16)f[2 * i], (_Float16)f[2 * i + 1]};
    w[i] = __builtin_bit_cast(uint32_t, h);
  }
  return u32x4{w[0], w[1], w[2], w[3]};
}
template <bool F16>
__device__ __forceinline__ void unpack8_cache(const u32x4& r, float* f) {
  if constexpr (F16) unpack8_f16(r, f); else unpack8(r, f);
}

struct SoftmaxState {
  float m, l;
  float acc[8];
};

// Merges `b` into `a` (both may be empty, i.e. m == -inf).
__device__ __forceinline__ void merge_state(SoftmaxState& a, const SoftmaxState& b) {
  const float m = fmaxf(a.m, b.m);
  const float mu = (m == -INFINITY) ? 0.f : m;
  const float sa = fast_exp2(a.m - mu), sb = fast_exp2(b.m - mu);
  a.l = a.l * sa + b.l * sb;
#pragma unroll
  for (int i = 0; i < 8; ++i) a.acc[i] = a.acc[i] * sa + b.acc[i] * sb;
  a.m = m;
}

// PREP: q, k_new and v_new are rows of the QKV projection output; the kernel normalises, rotates
// and mixes them itself (every workgroup of a (batch, head) redoes these few hundred flops).
// F16C: the cache rows are fp16 (the new rows are converted on their way in).
//
// Order of the memory instructions: the new token's rows and the table rows (raw), then the first two
// sets of cache rows, and only then the arithmetic on the new rows; inside the loop a register set is
// loaded again as soon as it has been used.  A wavefront so keeps 2 to 4 * kDecodeUnroll KiB of cache rows
// in flight from its first instructions to its last row: with a few hundred workgroups on the chip
// (one sequence, a dozen heads) the launch is a handful of memory round trips long, and every trip
// spent with nothing in flight shows.
template <int D, bool PREP, bool F16C = false>
__global__ __launch_bounds__(kDecodeThreads) void decode_kernel(DecodeParams p) {
  constexpr int LPR = D / 8;        // lanes per cache row
  constexpr int RPW = 64 / LPR;     // rows per wavefront load
  constexpr int U = kDecodeUnroll;
  constexpr int RB = RPW * U;       // rows of one register set
  constexpr int STRIDE = kDecodeWaves * RB;   // rows the four wavefronts cover with one set each

  const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int sub = lane / LPR;
  const int dl = (lane % LPR) * 8;

  const DecodeRange rg = decode_range(p);
  const int new_idx = rg.new_idx;
  const int r0 = split * rg.rows_per_split;
  const int r1 = min(r0 + rg.rows_per_split, rg.n_rows);
  // Only the split that holds the new token's slot needs the new key and value rows.
  const bool holds_new = new_idx >= r0 && new_idx < r0 + rg.rows_per_split;
  uint16_t* kbase = p.kc + b * p.kc_sb + h * p.kc_sh + dl;
  uint16_t* vbase = p.vc + b * p.vc_sb + h * p.vc_sh + dl;
  const uint16_t* q_row = p.q + b * p.q_sb + h * p.q_sh;
  const uint16_t* kn_row = p.k_new + b * p.kn_sb + h * p.kn_sh;
  const uint16_t* vn_row = p.v_new + b * p.vn_sb + h * p.vn_sh;

  // Raw rows of the new token.
  RawRow q_raw, kn_raw;
  TrigRow trig;
  u32x4 vn_raw, ve_raw = {0u, 0u, 0u, 0u};
  float gate = 0.f;
  bool past_tables = false, rotate = true;
  if constexpr (PREP) {
    const int t = p.pos_dev != nullptr ? max(p.pos_dev[0], 0) : p.pos_host;
    // A position past the rotation tables (possible only when it comes from device memory) reads the
    // last table row, to stay inside the allocation, and is reported: the status word gets its bit and
    // the outputs of the step are NaN, so that the step cannot pass for a valid one.
    past_tables = t >= p.table_rows;
    const int64_t trow = (int64_t)min(t, p.table_rows - 1) * (D / 2);
    trig = load_trig_row<D>(p.cos_tab + trow, p.sin_tab + trow, dl);
    q_raw = load_raw_row<D>(q_row, dl, true);
    kn_raw = load_raw_row<D>(holds_new ? kn_row : q_row, dl, true);
    vn_raw = *reinterpret_cast<const u32x4*>((holds_new ? vn_row : q_row) + dl);
    if (p.ve != nullptr) {
      ve_raw = *reinterpret_cast<const u32x4*>((holds_new ? p.ve + b * p.ve_sb + h * p.ve_sh : q_row) + dl);
      gate = p.gate[0];
    }
  } else {
    static_assert(!F16C, "fp16 cache rows come with the kernel-side preparation only");
    rotate = p.cos_row != nullptr;
    if (rotate) trig = load_trig_row<D>(p.cos_row, p.sin_row, dl);
    q_raw = load_raw_row<D>(q_row, dl, rotate);
    kn_raw = load_raw_row<D>(kn_row, dl, rotate);
    vn_raw = *reinterpret_cast<const u32x4*>(vn_row + dl);
  }

  // Lanes whose row is past the range, or is the new token's slot, load a row
  // that is always readable instead (and are masked / overwritten below).
  const int safe_row = (r0 != new_idx) ? r0 : r0 + 1;
  const uint16_t* k_safe = (safe_row < r1) ? kbase + (int64_t)safe_row * p.kc_sr : kn_row + dl;
  const uint16_t* v_safe = (safe_row < r1) ? vbase + (int64_t)safe_row * p.vc_sr : vn_row + dl;

  auto load_set = [&](int base, u32x4* kr, u32x4* vr) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int row = base + u * RPW + sub;
      const uint16_t* a = (row < r1 && row != new_idx) ? kbase + (int64_t)row * p.kc_sr : k_safe;
      kr[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int row = base + u * RPW + sub;
      const uint16_t* a = (row < r1 && row != new_idx) ? vbase + (int64_t)row * p.vc_sr : v_safe;
      vr[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a));
    }
  };

  // Two register sets; a set past the end of the range loads the safe row (one cache line) and is not used.
  u32x4 kA[U], vA[U], kB[U], vB[U];
  int base = r0 + wave * RB;
  __builtin_amdgcn_sched_barrier(0);
  load_set(base, kA, vA);
  load_set(base + STRIDE, kB, vB);
  __builtin_amdgcn_sched_barrier(0);

  float qf[8], knf[8];
  u32x4 vn_packed;
  if constexpr (PREP) {
    norm_rot_row<D>(q_raw, trig, dl, p.eps, qf);
    if (past_tables) {
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[i] = __builtin_nanf("");
      if (p.status != nullptr && tid == 0 && split == 0 && h == 0 && b == 0)
        __hip_atomic_fetch_or(p.status, DAISY_STATUS_POSITION_PAST_TABLES, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float vnf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { knf[i] = 0.f; vnf[i] = 0.f; }
    if (holds_new) {
      norm_rot_row<D>(kn_raw, trig, dl, p.eps, knf);
      norm_mix_row<D>(vn_raw, p.ve != nullptr, ve_raw, gate, p.eps, vnf);
    }
    vn_packed = F16C ? pack8_f16(vnf) : pack8(vnf);
  } else {
    if (rotate) {
      rot_row<D>(q_raw, trig, dl, qf);
      rot_row<D>(kn_raw, trig, dl, knf);
    } else {
      unpack8(q_raw.own, qf);
      unpack8(kn_raw.own, knf);
    }
    vn_packed = vn_raw;
  }
  const u32x4 kn_packed = F16C ? pack8_f16(knf) : pack8(knf);
#pragma unroll
  for (int i = 0; i < 8; ++i) qf[i] *= p.scale_log2e;

  SoftmaxState st;
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) st.acc[i] = 0.f;

  auto consume = [&](int base, u32x4* kr, u32x4* vr) {
    float s[U];
    float mblk = -INFINITY;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int row = base + u * RPW + sub;
      if (row == new_idx && row < r1) {
        kr[u] = kn_packed;
        vr[u] = vn_packed;
        if (p.write_back) {
          *reinterpret_cast<u32x4*>(kbase + (int64_t)row * p.kc_sr) = kn_packed;
          *reinterpret_cast<u32x4*>(vbase + (int64_t)row * p.vc_sr) = vn_packed;
        }
      }
      float kf[8];
      unpack8_cache<F16C>(kr[u], kf);
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) d = fmaf(qf[i], kf[i], d);
      d = group_sum<LPR>(d);
      s[u] = (row < r1) ? d : -INFINITY;
      mblk = fmaxf(mblk, s[u]);
    }

    const float mnew = fmaxf(st.m, mblk);
    const float mu = (mnew == -INFINITY) ? 0.f : mnew;
    const float alpha = fast_exp2(st.m - mu);
    st.m = mnew;
    st.l *= alpha;
#pragma unroll
    for (int i = 0; i < 8; ++i) st.acc[i] *= alpha;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float pu = fast_exp2(s[u] - mu);
      st.l += pu;
      float vf[8];
      unpack8_cache<F16C>(vr[u], vf);
#pragma unroll
      for (int i = 0; i < 8; ++i) st.acc[i] = fmaf(pu, vf[i], st.acc[i]);
    }
  };

  for (; base < r1; base += 2 * STRIDE) {
    consume(base, kA, vA);
    load_set(base + 2 * STRIDE, kA, vA);
    if (base + STRIDE < r1) consume(base + STRIDE, kB, vB);
    load_set(base + 3 * STRIDE, kB, vB);
  }

  // Merge the row groups of this wavefront (lanes that differ above bit log2(LPR)).
#pragma unroll
  for (int off = LPR; off < 64; off <<= 1) {
    SoftmaxState o;
    o.m = __shfl_xor(st.m, off);
    o.l = __shfl_xor(st.l, off);
#pragma unroll
    for (int i = 0; i < 8; ++i) o.acc[i] = __shfl_xor(st.acc[i], off);
    merge_state(st, o);
  }

  // Merge the wavefronts through LDS.
  __shared__ float sm_m[kDecodeWaves], sm_l[kDecodeWaves];
  __shared__ float sm_acc[kDecodeWaves][D];
  if (lane < LPR) {
    if (lane == 0) {
      sm_m[wave] = st.m;
      sm_l[wave] = st.l;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) sm_acc[wave][dl + i] = st.acc[i];
  }
  __syncthreads();
  if (wave == 0 && lane < LPR) {
#pragma unroll
    for (int w = 1; w < kDecodeWaves; ++w) {
      SoftmaxState o;
      o.m = sm_m[w];
      o.l = sm_l[w];
#pragma unroll
      for (int i = 0; i < 8; ++i) o.acc[i] = sm_acc[w][dl + i];
      merge_state(st, o);
    }
    if (p.nsplit == 1) {
      const float inv = 1.f / st.l;
      float of[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) of[i] = st.acc[i] * inv;
      *reinterpret_cast<u32x4*>(p.o + b * p.o_sb + h * p.o_sh + dl) = pack8(of);
    } else {
      float* part = p.partials + (((int64_t)b * p.H + h) * p.nsplit + split) * (D + 2);
      if (lane == 0) {
        part[0] = st.m;
        part[1] = st.l;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) part[2 + dl + i] = st.acc[i];
    }
  }
}

// Combines the per-split partials of one (batch, head).  The workgroup is 1 to kCombineThreads / D groups of D
// threads (one group per eight splits), a thread per channel; group g takes the splits g, g + groups, ... (at most
// kCombineUnroll of them) and fetches all of its partials with independent loads -- one memory round trip
// whatever the split count -- and the groups are merged through LDS.
constexpr int kCombineThreads = 512;
constexpr int kCombineUnroll = 16;
constexpr int kMaxSplits = kCombineUnroll * (kCombineThreads / 128);   // 64, for D = 64 and 128 alike
static int combine_threads(int D, int nsplit) {
  const int groups = (nsplit + 7) / 8 < kCombineThreads / D ? (nsplit + 7) / 8 : kCombineThreads / D;
  return groups * D;
}
template <int D>
__global__ __launch_bounds__(kCombineThreads) void decode_combine_kernel(DecodeParams p) {
  constexpr int GMAX = kCombineThreads / D;
  constexpr int U = kCombineUnroll;
  const int G = blockDim.x / D;            // split groups of this launch; g is the same for all lanes of a wavefront
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x % D, g = threadIdx.x / D;
  const float* part = p.partials + ((int64_t)b * p.H + h) * p.nsplit * (D + 2);
  float ms[U], ls[U], as[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int s = g + u * G;
    ms[u] = -INFINITY;
    ls[u] = 0.f;
    as[u] = 0.f;
    if (s < p.nsplit) {
      ms[u] = part[s * (D + 2)];
      ls[u] = part[s * (D + 2) + 1];
      as[u] = part[s * (D + 2) + 2 + d];
    }
  }
  float m = -INFINITY;
#pragma unroll
  for (int u = 0; u < U; ++u) m = fmaxf(m, ms[u]);
  const float mu = (m == -INFINITY) ? 0.f : m;
  float l = 0.f, acc = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const float w = fast_exp2(ms[u] - mu);   // an absent split has m = -inf: weight 0
    l = fmaf(ls[u], w, l);
    acc = fmaf(as[u], w, acc);
  }
  __shared__ float sm_m[GMAX], sm_l[GMAX], sm_acc[GMAX][D];
  if (G > 1) {
    if (d == 0) {
      sm_m[g] = m;
      sm_l[g] = l;
    }
    sm_acc[g][d] = acc;
    __syncthreads();
    if (g != 0) return;
    m = sm_m[0];
    for (int i = 1; i < G; ++i) m = fmaxf(m, sm_m[i]);
    const float mut = (m == -INFINITY) ? 0.f : m;
    l = 0.f;
    acc = 0.f;
    for (int i = 0; i < G; ++i) {
      const float w = fast_exp2(sm_m[i] - mut);
      l = fmaf(sm_l[i], w, l);
      acc = fmaf(sm_acc[i][d], w, acc);
    }
  }
  const float r = acc / l;
  p.o[b * p.o_sb + h * p.o_sh + d] = (uint16_t)(pack_bf16x2(r, 0.f) & 0xffffu);
}

static int choose_nsplit(int B, int H, int n_rows) {
  // About 512 rows per workgroup (two full iterations of every wavefront and some), as long as that does not make
  // more than about 1024 workgroups; when it leaves fewer than 192 workgroups on the 256 compute units (a few
  // (batch, head) pairs: the generator's batch of one), shorter splits down to 128 rows.  From a sweep over
  // B*H = 6..1024, 1024..8192 rows and 1..64 splits; within a few per cent of the best count everywhere.
  const int bh = B * H;
  int by_rows = n_rows / 512 > 0 ? n_rows / 512 : 1;
  const int by_grid = (1024 + bh - 1) / bh;
  int ns = by_rows < by_grid ? by_rows : by_grid;
  if (bh * ns < 192) {
    by_rows = n_rows / 128 > 0 ? n_rows / 128 : 1;
    const int fill = (192 + bh - 1) / bh;
    ns = by_rows < fill ? by_rows : fill;
  }
  if (ns < 1) ns = 1;
  if (ns > kMaxSplits) ns = kMaxSplits;
  return ns;
}

static int resolve_nsplit(int B, int H, int n_rows, int nsplit) {
  if (nsplit <= 0) nsplit = choose_nsplit(B, H, n_rows);
  if (nsplit > kMaxSplits) nsplit = kMaxSplits;   // what the combine kernel takes
  if (nsplit > n_rows) nsplit = n_rows;
  if (nsplit < 1) nsplit = 1;
  const int rps = (n_rows + nsplit - 1) / nsplit;
  // Drop splits that would be empty after rounding rows_per_split up.
  return (n_rows + rps - 1) / rps;
}

// Any even head dim up to 256 (the reference's unit tests use 2 and 8): one wavefront per
// (batch, head), lane l owns channels l, l + 64, ...; rows are visited one after the other with a
// wavefront-wide reduction per score.  Correctness path for small shapes, not a fast one.
template <typename E>
__global__ __launch_bounds__(64) void decode_scalar_kernel(DecodeParams p, int D) {
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const int half = D / 2;
  const DecodeRange rg = decode_range(p);
  const E* qp = reinterpret_cast<const E*>(p.q) + b * p.q_sb + h * p.q_sh;
  const E* knp = reinterpret_cast<const E*>(p.k_new) + b * p.kn_sb + h * p.kn_sh;
  const E* vnp = reinterpret_cast<const E*>(p.v_new) + b * p.vn_sb + h * p.vn_sh;
  E* kc = reinterpret_cast<E*>(p.kc) + b * p.kc_sb + h * p.kc_sh;
  E* vc = reinterpret_cast<E*>(p.vc) + b * p.vc_sb + h * p.vc_sh;
  float qv[4], kn[4], vn[4], acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    qv[i] = kn[i] = vn[i] = acc[i] = 0.f;
    if (d < D) {
      float x = load_elem<E>(qp, d), y = load_elem<E>(knp, d);
      if (p.cos_row != nullptr) {
        const bool lower = d < half;
        const int dp = lower ? d + half : d - half;   // RoPE partner channel
        const float c = p.cos_row[lower ? d : dp], sn = p.sin_row[lower ? d : dp];
        const float xp = load_elem<E>(qp, dp), yp = load_elem<E>(knp, dp);
        x = round_elem<E>(lower ? rope_lo(x, xp, c, sn) : rope_hi(xp, x, c, sn));
        y = round_elem<E>(lower ? rope_lo(y, yp, c, sn) : rope_hi(yp, y, c, sn));
      }
      qv[i] = x;
      kn[i] = y;
      vn[i] = load_elem<E>(vnp, d);
    }
  }
  float m = -INFINITY, l = 0.f;
  for (int r = 0; r < rg.n_rows; ++r) {
    const bool is_new = r == rg.new_idx;
    float kr[4], vr[4], part = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      kr[i] = vr[i] = 0.f;
      if (d < D) {
        kr[i] = is_new ? kn[i] : load_elem<E>(kc, (int64_t)r * p.kc_sr + d);
        vr[i] = is_new ? vn[i] : load_elem<E>(vc, (int64_t)r * p.vc_sr + d);
      }
      part += qv[i] * kr[i];
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) part += __shfl_xor(part, off);
    const float s = part * p.scale_log2e;
    const float m_new = fmaxf(m, s);
    const float alpha = fast_exp2(m - m_new), pr = fast_exp2(s - m_new);
    l = l * alpha + pr;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = acc[i] * alpha + pr * vr[i];
    m = m_new;
  }
  E* op = reinterpret_cast<E*>(p.o) + b * p.o_sb + h * p.o_sh;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < D) {
      store_elem<E>(op, d, acc[i] / l);
      if (p.write_back) {
        store_elem<E>(kc, (int64_t)rg.new_idx * p.kc_sr + d, kn[i]);
        store_elem<E>(vc, (int64_t)rg.new_idx * p.vc_sr + d, vn[i]);
      }
    }
  }
}

}  // namespace daisy

using namespace daisy;

extern "C" size_t daisy_decode_workspace_bytes(int B, int H, int D, int n_rows, int nsplit) {
  if (B <= 0 || H <= 0 || D <= 0 || n_rows <= 0) return 0;
  if (D != 64 && D != 128) return 0;   // the small-head-dim kernel never splits
  const int ns = resolve_nsplit(B, H, n_rows, nsplit);
  if (ns == 1) return 0;
  return (size_t)B * H * ns * (D + 2) * sizeof(float);
}

// What daisy_attn_step_fwd adds to a decode launch: the kernel prepares the rows itself.
struct StepPrep {
  int pos_host; const float* cos; const float* sin; int table_rows; float eps;
  const void* ve; const int64_t* ve_strides; const float* gate;
  int cache_f16; int32_t* status;
};

// Shared by the entry points.  With pos_dev set, n_rows is the ring's slot count (it fixes the
// split count and the grid) and the kernel derives the live rows and the new row's slot from *pos_dev.
static int decode_launch(const void* q, const int64_t* q_strides,
                         const void* k_new, const int64_t* k_new_strides,
                         const void* v_new, const int64_t* v_new_strides,
                         void* k_cache, const int64_t* k_cache_strides,
                         void* v_cache, const int64_t* v_cache_strides,
                         const float* cos_row, const float* sin_row,
                         void* o, const int64_t* o_strides,
                         int B, int H, int D,
                         int n_rows, int new_idx, const int32_t* pos_dev, int write_back,
                         float scale, int nsplit,
                         void* workspace, size_t workspace_bytes, void* stream, const StepPrep* prep = nullptr,
                         bool f32_io = false) {
  DAISY_CHECK_ARG(q && k_new && v_new && o, "decode: q, k_new, v_new and o must be non-NULL");
  DAISY_CHECK_ARG(q_strides && k_new_strides && v_new_strides && o_strides, "decode: stride arrays must be non-NULL");
  DAISY_CHECK_ARG(B > 0 && H > 0, "decode: B=%d and H=%d must be positive", B, H);
  DAISY_CHECK_ARG(B <= 65535 && H <= 65535, "decode: B=%d and H=%d must each be <= 65535", B, H);
  DAISY_CHECK_SUPPORTED(D >= 2 && D <= 256 && D % 2 == 0, "decode: head_dim %d not supported (even, 2..256)", D);
  const bool fast = (D == 64 || D == 128) && !f32_io;   // fp32 tensors always take the one-wavefront kernel
  DAISY_CHECK_ARG(n_rows >= 1, "decode: n_rows=%d must be >= 1 (the new token is always attended)", n_rows);
  DAISY_CHECK_ARG(new_idx >= 0 && new_idx < n_rows, "decode: new_idx=%d outside [0, %d)", new_idx, n_rows);
  DAISY_CHECK_ARG((cos_row == nullptr) == (sin_row == nullptr), "decode: cos_row and sin_row must both be given or both NULL");
  DAISY_CHECK_ARG(n_rows == 1 || (k_cache && v_cache && k_cache_strides && v_cache_strides),
                  "decode: cache pointers and strides are required when n_rows > 1");
  DAISY_CHECK_ARG(!write_back || (k_cache && v_cache), "decode: write_back needs cache pointers");
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(!fast || (al16(q) && al16(k_new) && al16(v_new) && al16(o) && al16(k_cache) && al16(v_cache)),
                  "decode: tensors must be 16-byte aligned");
  static const int64_t zero3[3] = {0, 0, 0};
  if (!k_cache_strides) k_cache_strides = zero3;
  if (!v_cache_strides) v_cache_strides = zero3;
  for (int i = 0; i < 2 && fast; ++i) {
    DAISY_CHECK_ARG(q_strides[i] % 8 == 0 && k_new_strides[i] % 8 == 0 && v_new_strides[i] % 8 == 0 && o_strides[i] % 8 == 0,
                    "decode: vector strides must be multiples of 8 elements");
  }
  for (int i = 0; i < 3 && fast; ++i) {
    DAISY_CHECK_ARG(k_cache_strides[i] % 8 == 0 && v_cache_strides[i] % 8 == 0,
                    "decode: cache strides must be multiples of 8 elements");
  }

  DecodeParams p;
  p.q = (const uint16_t*)q; p.q_sb = q_strides[0]; p.q_sh = q_strides[1];
  p.k_new = (const uint16_t*)k_new; p.kn_sb = k_new_strides[0]; p.kn_sh = k_new_strides[1];
  p.v_new = (const uint16_t*)v_new; p.vn_sb = v_new_strides[0]; p.vn_sh = v_new_strides[1];
  p.kc = (uint16_t*)k_cache; p.kc_sb = k_cache_strides[0]; p.kc_sh = k_cache_strides[1]; p.kc_sr = k_cache_strides[2];
  p.vc = (uint16_t*)v_cache; p.vc_sb = v_cache_strides[0]; p.vc_sh = v_cache_strides[1]; p.vc_sr = v_cache_strides[2];
  if (n_rows == 1 && !k_cache) {
    // Only the new row exists; give the kernel a readable dummy row.
    p.kc = (uint16_t*)k_new; p.kc_sb = k_new_strides[0]; p.kc_sh = k_new_strides[1]; p.kc_sr = 0;
    p.vc = (uint16_t*)v_new; p.vc_sb = v_new_strides[0]; p.vc_sh = v_new_strides[1]; p.vc_sr = 0;
    write_back = 0;
  }
  p.cos_row = cos_row; p.sin_row = sin_row;
  p.o = (uint16_t*)o; p.o_sb = o_strides[0]; p.o_sh = o_strides[1];
  p.B = B; p.H = H; p.n_rows = n_rows; p.new_idx = new_idx; p.write_back = write_back;
  p.nsplit = fast ? resolve_nsplit(B, H, n_rows, nsplit) : 1;
  p.rows_per_split = (n_rows + p.nsplit - 1) / p.nsplit;
  p.pos_dev = pos_dev; p.ring_rows = n_rows;
  p.pos_host = 0; p.cos_tab = p.sin_tab = nullptr; p.table_rows = 0; p.eps = 0.f;
  p.ve = nullptr; p.ve_sb = p.ve_sh = 0; p.gate = nullptr; p.status = nullptr;
  if (prep != nullptr) {
    p.pos_host = prep->pos_host; p.cos_tab = prep->cos; p.sin_tab = prep->sin; p.table_rows = prep->table_rows;
    p.eps = prep->eps; p.ve = (const uint16_t*)prep->ve; p.gate = prep->gate; p.status = prep->status;
    if (prep->ve) { p.ve_sb = prep->ve_strides[0]; p.ve_sh = prep->ve_strides[1]; }
  }
  p.scale_log2e = scale * kLog2e;
  p.partials = nullptr;
  if (p.nsplit > 1) {
    const size_t need = (size_t)B * H * p.nsplit * (D + 2) * sizeof(float);
    if (!workspace || workspace_bytes < need) {
      set_error("decode: workspace of %zu bytes needed for %d splits, got %zu", need, p.nsplit, workspace_bytes);
      return DAISY_ERR_WORKSPACE;
    }
    p.partials = (float*)workspace;
  }

  hipStream_t s = (hipStream_t)stream;
  if (!fast) {
    if (f32_io) hipLaunchKernelGGL(decode_scalar_kernel<float>, dim3(H, B), dim3(64), 0, s, p, D);
    else hipLaunchKernelGGL(decode_scalar_kernel<uint16_t>, dim3(H, B), dim3(64), 0, s, p, D);
    DAISY_CHECK_LAUNCH("decode_scalar_kernel");
    return DAISY_OK;
  }
  dim3 grid(p.nsplit, H, B);
  if (D == 128) {
    if (prep && prep->cache_f16) hipLaunchKernelGGL((decode_kernel<128, true, true>), grid, dim3(kDecodeThreads), 0, s, p);
    else if (prep) hipLaunchKernelGGL((decode_kernel<128, true>), grid, dim3(kDecodeThreads), 0, s, p);
    else hipLaunchKernelGGL((decode_kernel<128, false>), grid, dim3(kDecodeThreads), 0, s, p);
    DAISY_CHECK_LAUNCH("decode_kernel");
    if (p.nsplit > 1) {
      hipLaunchKernelGGL(decode_combine_kernel<128>, dim3(H, B), dim3(combine_threads(128, p.nsplit)), 0, s, p);
      DAISY_CHECK_LAUNCH("decode_combine_kernel");
    }
  } else {
    if (prep && prep->cache_f16) hipLaunchKernelGGL((decode_kernel<64, true, true>), grid, dim3(kDecodeThreads), 0, s, p);
    else if (prep) hipLaunchKernelGGL((decode_kernel<64, true>), grid, dim3(kDecodeThreads), 0, s, p);
    else hipLaunchKernelGGL((decode_kernel<64, false>), grid, dim3(kDecodeThreads), 0, s, p);
    DAISY_CHECK_LAUNCH("decode_kernel");
    if (p.nsplit > 1) {
      hipLaunchKernelGGL(decode_combine_kernel<64>, dim3(H, B), dim3(combine_threads(64, p.nsplit)), 0, s, p);
      DAISY_CHECK_LAUNCH("decode_combine_kernel");
    }
  }
  return DAISY_OK;
}

extern "C" int daisy_decode_fwd(const void* q, const int64_t* q_strides,
                                const void* k_new, const int64_t* k_new_strides,
                                const void* v_new, const int64_t* v_new_strides,
                                void* k_cache, const int64_t* k_cache_strides,
                                void* v_cache, const int64_t* v_cache_strides,
                                const float* cos_row, const float* sin_row,
                                void* o, const int64_t* o_strides,
                                int B, int H, int D,
                                int n_rows, int new_idx, int write_back,
                                float scale, int nsplit,
                                void* workspace, size_t workspace_bytes, void* stream) {
  return decode_launch(q, q_strides, k_new, k_new_strides, v_new, v_new_strides, k_cache, k_cache_strides,
                       v_cache, v_cache_strides, cos_row, sin_row, o, o_strides, B, H, D, n_rows, new_idx, nullptr,
                       write_back, scale, nsplit, workspace, workspace_bytes, stream);
}

// ---- the entry point that allocates nothing ----------------------------------------------------
// The split partials of daisy_decode_fwd_noalloc live in this array of the library's device image.
// In host code the array's name is only a stand-in: the address a kernel can use comes from
// hipGetSymbolAddress, once per device (each GPU holds its own copy at its own address).
static __device__ __align__(256) unsigned char scratch[DAISY_DECODE_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device.  The address is looked up once per device, by
// daisy_decode_noalloc_init or by the first call on the device; the lookup may make the runtime load the
// library's device image, which is not a thing to do while `capturing` (a stream of the caller is recording
// a graph): then only an address found earlier is handed out.
int static_scratch(void** out, bool capturing) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("decode_noalloc: cannot identify the current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
    return DAISY_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    if (capturing) {
      set_error("decode_noalloc: first use on device %d while the stream is capturing; call daisy_decode_noalloc_init() "
                "on this device (or run one call) before the capture starts", dev);
      return DAISY_ERR_INVALID_ARGUMENT;
    }
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("decode_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return DAISY_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return DAISY_OK;
}
}  // namespace

extern "C" int daisy_decode_noalloc_init(void) {
  void* ws = nullptr;
  return static_scratch(&ws, /*capturing=*/false);
}

extern "C" int daisy_decode_fwd_noalloc(const void* q, const int64_t* q_strides,
                                        const void* k_new, const int64_t* k_new_strides,
                                        const void* v_new, const int64_t* v_new_strides,
                                        void* k_cache, const int64_t* k_cache_strides,
                                        void* v_cache, const int64_t* v_cache_strides,
                                        const float* cos_row, const float* sin_row,
                                        void* o, const int64_t* o_strides,
                                        int B, int H, int D,
                                        int n_rows, int new_idx, int write_back,
                                        float scale, int nsplit, void* stream) {
  const size_t need = daisy_decode_workspace_bytes(B, H, D, n_rows, nsplit);
  if (need > DAISY_DECODE_STATIC_SCRATCH_BYTES) {
    set_error("decode_noalloc: %zu bytes of split partials needed (B=%d, H=%d, D=%d, n_rows=%d, nsplit=%d), the built-in "
              "buffer holds %u; use daisy_decode_fwd with a workspace or fewer splits",
              need, B, H, D, n_rows, nsplit, (unsigned)DAISY_DECODE_STATIC_SCRATCH_BYTES);
    return DAISY_ERR_WORKSPACE;
  }
  void* ws = nullptr;
  if (need > 0) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cap) != hipSuccess) {
      (void)hipGetLastError();
      cap = hipStreamCaptureStatusNone;
    }
    const int rc = static_scratch(&ws, cap != hipStreamCaptureStatusNone);
    if (rc != DAISY_OK) return rc;
  }
  // Every split writes its whole partial before the combine kernel reads it: nothing of the last
  // call's contents is ever read, so nothing needs clearing.
  return decode_launch(q, q_strides, k_new, k_new_strides, v_new, v_new_strides, k_cache, k_cache_strides,
                       v_cache, v_cache_strides, cos_row, sin_row, o, o_strides, B, H, D, n_rows, new_idx, nullptr,
                       write_back, scale, nsplit, ws, need, stream);
}

extern "C" int daisy_decode_fwd_f32(const float* q, const int64_t* q_strides,
                                    const float* k_new, const int64_t* k_new_strides,
                                    const float* v_new, const int64_t* v_new_strides,
                                    float* k_cache, const int64_t* k_cache_strides,
                                    float* v_cache, const int64_t* v_cache_strides,
                                    const float* cos_row, const float* sin_row,
                                    float* o, const int64_t* o_strides,
                                    int B, int H, int D,
                                    int n_rows, int new_idx, int write_back,
                                    float scale, void* stream) {
  return decode_launch(q, q_strides, k_new, k_new_strides, v_new, v_new_strides, k_cache, k_cache_strides,
                       v_cache, v_cache_strides, cos_row, sin_row, o, o_strides, B, H, D, n_rows, new_idx, nullptr,
                       write_back, scale, 1, nullptr, 0, stream, nullptr, /*f32_io=*/true);
}

extern "C" int daisy_decode_fwd_at(const void* q, const int64_t* q_strides,
                                   const void* k_new, const int64_t* k_new_strides,
                                   const void* v_new, const int64_t* v_new_strides,
                                   void* k_cache, const int64_t* k_cache_strides,
                                   void* v_cache, const int64_t* v_cache_strides,
                                   void* o, const int64_t* o_strides,
                                   int B, int H, int D,
                                   int ring_rows, const int32_t* pos,
                                   float scale, int nsplit,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  DAISY_CHECK_ARG(pos != nullptr, "decode_at: the device position pointer must be non-NULL");
  DAISY_CHECK_ARG(k_cache && v_cache && k_cache_strides && v_cache_strides, "decode_at: the ring cache is required");
  DAISY_CHECK_ARG(ring_rows >= 1, "decode_at: ring_rows=%d must be >= 1", ring_rows);
  DAISY_CHECK_SUPPORTED(D == 64 || D == 128, "decode_at: head_dim %d not supported (64 or 128)", D);
  return decode_launch(q, q_strides, k_new, k_new_strides, v_new, v_new_strides, k_cache, k_cache_strides,
                       v_cache, v_cache_strides, nullptr, nullptr, o, o_strides, B, H, D, ring_rows, 0, pos,
                       /*write_back=*/1, scale, nsplit, workspace, workspace_bytes, stream);
}

extern "C" int daisy_attn_step_fwd(const void* q, const int64_t* q_strides,
                                   const void* k, const int64_t* k_strides,
                                   const void* v, const int64_t* v_strides,
                                   const void* ve, const int64_t* ve_strides, const float* gate,
                                   const float* cos, const float* sin, int table_rows,
                                   int pos, const int32_t* pos_dev, int32_t* status, float eps,
                                   void* k_cache, const int64_t* k_cache_strides,
                                   void* v_cache, const int64_t* v_cache_strides, int cache_is_f16,
                                   void* o, const int64_t* o_strides,
                                   int B, int H, int D, int ring_rows,
                                   float scale, int nsplit,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  DAISY_CHECK_SUPPORTED(D == 64 || D == 128, "attn_step: head_dim %d not supported (64 or 128)", D);
  DAISY_CHECK_ARG(k_cache && v_cache && k_cache_strides && v_cache_strides, "attn_step: the ring cache is required");
  DAISY_CHECK_ARG(ring_rows >= 1, "attn_step: ring_rows=%d must be >= 1", ring_rows);
  DAISY_CHECK_ARG(cos && sin && table_rows >= 1, "attn_step: the rotary tables are required");
  DAISY_CHECK_ARG((ve == nullptr) == (gate == nullptr), "attn_step: ve and gate must both be given or both NULL");
  DAISY_CHECK_ARG(ve == nullptr || ve_strides != nullptr, "attn_step: ve needs ve_strides");
  DAISY_CHECK_ARG(pos_dev != nullptr || (pos >= 0 && pos < table_rows),
                  "attn_step: position %d outside the rotary tables (%d rows)", pos, table_rows);
  auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  DAISY_CHECK_ARG(al16(ve) && (!ve || (ve_strides[0] % 8 == 0 && ve_strides[1] % 8 == 0)),
                  "attn_step: ve must be 16-byte aligned with strides that are multiples of 8 elements");
  StepPrep prep{pos, cos, sin, table_rows, eps, ve, ve_strides, gate, cache_is_f16 != 0, status};
  // With the position on the host the live rows and the slot are launch arguments (and the split
  // count follows the live rows); with the position on the device the kernel derives them.
  const int n_rows = pos_dev ? ring_rows : (pos + 1 < ring_rows ? pos + 1 : ring_rows);
  const int new_idx = pos_dev ? 0 : pos % ring_rows;
  return decode_launch(q, q_strides, k, k_strides, v, v_strides, k_cache, k_cache_strides, v_cache, v_cache_strides,
                       nullptr, nullptr, o, o_strides, B, H, D, n_rows, new_idx, pos_dev, /*write_back=*/1, scale, nsplit,
                       workspace, workspace_bytes, stream, &prep);
}
