/*
 * daisy_hip.h -- C ABI of libdaisy_hip.so, the gfx950 (MI355X) kernels behind
 * Daisy's attention hot path.
 *
 * Conventions
 *   - All tensor pointers are device pointers, borrowed for the duration of the
 *     call.  The library never allocates or frees device memory and keeps no
 *     tensor state; scratch space is passed in as `workspace`.
 *   - bf16 tensors are passed as `void*` (2-byte elements, the last dimension
 *     contiguous); strides are counted in ELEMENTS, not bytes.
 *   - Every launch is asynchronous on `stream` (a hipStream_t passed as void*;
 *     NULL is the default stream).  No call synchronises the host.
 *   - Return value: DAISY_OK (0) or a negative error code; the text of the last
 *     error on the calling thread is returned by daisy_last_error().  No C++
 *     exception crosses this boundary.
 *
 * The reference is pure Python and has no FFI; each entry point names the
 * reference call it stands in for (paths relative to the reference checkout).
 */
#ifndef DAISY_HIP_H
#define DAISY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DAISY_OK 0
#define DAISY_ERR_INVALID_ARGUMENT (-1)
#define DAISY_ERR_UNSUPPORTED (-2)
#define DAISY_ERR_WORKSPACE (-3)
#define DAISY_ERR_LAUNCH (-4)

/* Bits a kernel raises in a caller-supplied status word (int32 in device memory, never cleared by
 * the library) when it meets a condition that only the device can see. */
#define DAISY_STATUS_POSITION_PAST_TABLES 1   /* a position read from device memory lies past the rotation tables */

/* Text of the last error raised on this thread ("" if none). */
const char* daisy_last_error(void);

/* ABI version of this header (bumped on any signature change). */
int daisy_abi_version(void);

/* ---------------------------------------------------------------------------
 * Kernel 1: sliding-window causal flash-attention prefill with fused RoPE.
 *
 * Replaces, in CausalSelfAttention._sdpa_common / prefill
 * (models/daisy/attention.py:141-150,173-179):
 *   rotary(q), rotary(k)            (attention.py:16-20,57-62,122-125)
 *   build_attn_mask(...)            (models/daisy/daisy_core.py:53-69)
 *   F.scaled_dot_product_attention  (attention.py:145,147)
 *
 *   o[b,t,h,:] = sum_k softmax_k(scale * <rope(q[b,t,h]), rope(k[b,k,h])>) v[b,k,h,:]
 *   over keys k with  max(t - window + 1, doc_start[t]) <= k <= t.
 *
 * q, k, v, o : bf16, logical shape [B, T, H, D]; *_strides = {batch, token, head}
 *              element strides (D contiguous).  D must be 64 or 128 for the MFMA
 *              kernel; any other even D <= 256 runs a scalar kernel.
 * cos, sin   : fp32 [>= T, D/2] row-major rotation tables, or both NULL when
 *              q and k are already rotated.  Row t rotates position t with
 *              y1 = x1*cos + x2*sin, y2 = -x1*sin + x2*cos on pairs (i, i+D/2).
 * doc_start  : int32 [T] or NULL; doc_start[t] = index of the first token of the
 *              document containing t.  Contract: 0 <= doc_start[t] <= t and
 *              non-decreasing in t (the kernel picks the key tiles of a block of
 *              128 queries from the block's first row; a bound that decreases
 *              inside a block silently drops keys, a bound beyond t gives NaN).
 *              Shared by all batches, like the reference's [1,1,T,T] mask.
 * k_out      : bf16 [B, T, H, D] with its own strides.  REQUIRED when cos/sin are
 *              given and D is 64 or 128 (DAISY_ERR_INVALID_ARGUMENT otherwise):
 *              a pre-pass writes the rotated keys there once (what the
 *              reference's prefill returns for the KV cache, attention.py:179)
 *              and the attention kernel reads them from there instead of
 *              rotating every key tile again for every query block.  NULL
 *              when cos/sin are NULL; optional for the scalar kernel.
 * window     : keys visible per query INCLUDING itself; <= 0 means full causal.
 * flags      : reserved, must be 0.
 */
int daisy_prefill_fwd(const void* q, const int64_t* q_strides,
                      const void* k, const int64_t* k_strides,
                      const void* v, const int64_t* v_strides,
                      const float* cos, const float* sin,
                      const int32_t* doc_start,
                      void* o, const int64_t* o_strides,
                      void* k_out, const int64_t* k_out_strides,
                      int B, int T, int H, int D,
                      int window, float scale, int flags, void* stream);

/* The same attention on fp32 tensors with fp32 arithmetic throughout (nothing is rounded to bf16):
 * the mode of a module whose parameters are fp32, as the reference's own unit tests build it
 * (tests/test_attention.py:9, compared at 1e-4).  Any even D <= 256; one wavefront per query, so
 * this is a correctness path, not a fast one.  Strides in fp32 elements; k_out receives the
 * rotated keys in fp32 when cos/sin are given.
 */
int daisy_prefill_fwd_f32(const float* q, const int64_t* q_strides,
                          const float* k, const int64_t* k_strides,
                          const float* v, const int64_t* v_strides,
                          const float* cos, const float* sin,
                          const int32_t* doc_start,
                          float* o, const int64_t* o_strides,
                          float* k_out, const int64_t* k_out_strides,
                          int B, int T, int H, int D,
                          int window, float scale, void* stream);

/* ---------------------------------------------------------------------------
 * Kernel 2: split-K single-token decode over a bf16 KV cache.
 *
 * Replaces, in CausalSelfAttention.step (attention.py:181-202) together with
 * KVCache.view / write (inference/kv_cache.py:26-51):
 *   rotary.step(q, pos), rotary.step(k, pos)       (attention.py:64-70,123)
 *   torch.cat([k_ctx[:, n-r:n], k], 1) ... SDPA    (attention.py:192-199)
 *   cache.k[layer, :, :, t % W] = k_new             (kv_cache.py:44-51)
 *
 * The cache tensors are addressed as rows: row r of (b, h) starts at
 * base + b*strides[0] + h*strides[1] + r*strides[2].  The step attends
 * `n_rows` logical rows 0..n_rows-1; logical row `new_idx` is NOT read from the
 * cache but taken from k_new / v_new (after RoPE), and is stored into the cache
 * at that row when `write_back` is non-zero.  Row order is irrelevant to the
 * result, so a ring buffer is streamed in physical order:
 *   ring of W slots at time t:  n_rows = min(t+1, W), new_idx = t % W, write_back = 1
 *   chronological context [B,n,H,D], r = min(n, window-1) live rows starting at
 *   row n-r:  base += (n-r)*strides[2], n_rows = r+1, new_idx = r, write_back = 0
 *
 * q, k_new, v_new, o : bf16 [B, H, D]; strides = {batch, head}.
 * cos_row, sin_row   : fp32 [D/2] rows of the rotation tables for this position
 *                      (applied to q and k_new), or both NULL.
 * workspace          : >= daisy_decode_workspace_bytes(...) bytes, 256-byte
 *                      aligned; may be NULL when that function returns 0.
 * nsplit             : number of sequence splits per (b, h); 0 = choose; values above 64 are taken as 64.
 * D is 64 or 128 for the streaming kernel; any other even D <= 256 runs a
 * one-wavefront-per-(batch, head) kernel meant for small test shapes (no splits).
 */
size_t daisy_decode_workspace_bytes(int B, int H, int D, int n_rows, int nsplit);

int daisy_decode_fwd(const void* q, const int64_t* q_strides,
                     const void* k_new, const int64_t* k_new_strides,
                     const void* v_new, const int64_t* v_new_strides,
                     void* k_cache, const int64_t* k_cache_strides,
                     void* v_cache, const int64_t* v_cache_strides,
                     const float* cos_row, const float* sin_row,
                     void* o, const int64_t* o_strides,
                     int B, int H, int D,
                     int n_rows, int new_idx, int write_back,
                     float scale, int nsplit,
                     void* workspace, size_t workspace_bytes, void* stream);

/* daisy_decode_fwd on fp32 tensors with fp32 arithmetic (see daisy_prefill_fwd_f32): any even
 * D <= 256, one wavefront per (batch, head), no splits and no workspace.
 */
int daisy_decode_fwd_f32(const float* q, const int64_t* q_strides,
                         const float* k_new, const int64_t* k_new_strides,
                         const float* v_new, const int64_t* v_new_strides,
                         float* k_cache, const int64_t* k_cache_strides,
                         float* v_cache, const int64_t* v_cache_strides,
                         const float* cos_row, const float* sin_row,
                         float* o, const int64_t* o_strides,
                         int B, int H, int D,
                         int n_rows, int new_idx, int write_back,
                         float scale, void* stream);

/* daisy_decode_fwd for callers that cannot allocate device memory or pass a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart
 * in the reference.  The split partials live in a buffer of DAISY_DECODE_STATIC_SCRATCH_BYTES that
 * is part of the library's device image (each GPU the library runs on holds one copy until the
 * process ends); the call allocates nothing and fails with DAISY_ERR_WORKSPACE when
 * daisy_decode_workspace_bytes(B, H, D, n_rows, nsplit) exceeds that size.  All calls on one GPU
 * share the buffer: calls that overlap on one GPU (different streams) race and must be ordered by
 * the caller.  Same results as daisy_decode_fwd.
 *
 * The buffer's device address is looked up once per device, by daisy_decode_noalloc_init() or by the
 * first call on that device.  The lookup is not done while `stream` is capturing: a caller that records
 * the entry point into a HIP graph calls daisy_decode_noalloc_init() (or runs one call) on that device
 * before the capture starts, else the call fails with DAISY_ERR_INVALID_ARGUMENT.
 * daisy_decode_noalloc_init: set-up for the current device; launches nothing, allocates nothing, may be
 * called any number of times.  No counterpart in the reference either.
 */
#define DAISY_DECODE_STATIC_SCRATCH_BYTES (4u << 20)
int daisy_decode_noalloc_init(void);
int daisy_decode_fwd_noalloc(const void* q, const int64_t* q_strides,
                             const void* k_new, const int64_t* k_new_strides,
                             const void* v_new, const int64_t* v_new_strides,
                             void* k_cache, const int64_t* k_cache_strides,
                             void* v_cache, const int64_t* v_cache_strides,
                             const float* cos_row, const float* sin_row,
                             void* o, const int64_t* o_strides,
                             int B, int H, int D,
                             int n_rows, int new_idx, int write_back,
                             float scale, int nsplit, void* stream);

/* The same decode step with the position held in device memory: `pos` points at one
 * int32 t (the number of tokens already in the ring, as DaisyCore.step's `pos`,
 * models/daisy/daisy_core.py:294-323, and KVCache.t, inference/kv_cache.py:52-55).  The
 * kernel reads t when it runs, attends min(t + 1, ring_rows) live rows and writes the new
 * row to slot t % ring_rows, so that a launch recorded once (a HIP graph of the whole
 * model step) can be replayed for every later position; the caller increments *pos
 * between steps.  q and k_new arrive rotated (see daisy_qkv_prep_fwd_at); the new row is
 * always written back.  The grid is fixed by ring_rows: size the workspace with
 * daisy_decode_workspace_bytes(B, H, D, ring_rows, nsplit).  D is 64 or 128.
 */
int daisy_decode_fwd_at(const void* q, const int64_t* q_strides,
                        const void* k_new, const int64_t* k_new_strides,
                        const void* v_new, const int64_t* v_new_strides,
                        void* k_cache, const int64_t* k_cache_strides,
                        void* v_cache, const int64_t* v_cache_strides,
                        void* o, const int64_t* o_strides,
                        int B, int H, int D,
                        int ring_rows, const int32_t* pos,
                        float scale, int nsplit,
                        void* workspace, size_t workspace_bytes, void* stream);

/* The attention part of one decode step in a single launch: what CausalSelfAttention.step
 * (models/daisy/attention.py:181-202) does between its two projections.  q, k, v are the rows
 * of the QKV projection output for the new token, bf16 [B, H, D] with {batch, head} strides
 * (three views of one [B, 3H, D] tensor).  The kernel applies the weightless RMS norm to all
 * three (eps as in daisy_qkv_prep_fwd), rotates q and k with row `pos` of the tables
 * (cos, sin: fp32 [table_rows, D/2]), mixes v with ve through *gate when both are given, writes
 * the new K and V rows into slot pos % ring_rows of the ring cache [B, H, ring_rows, D] and
 * attends the min(pos + 1, ring_rows) live rows.  The position is `pos` when pos_dev is NULL,
 * else the int32 that pos_dev points at, read when the kernel runs (see daisy_decode_fwd_at;
 * the workspace is then sized for ring_rows, otherwise for the live rows).
 * Same results as daisy_qkv_prep_fwd followed by daisy_decode_fwd up to the order of the
 * fp32 sums inside the norm.  D is 64 or 128.  cache_is_f16: the ring holds fp16 rows (the
 * default cache dtype of the reference's Generator, inference/generate.py:62) instead of bf16;
 * the new rows are converted on their way in, which loses nothing for normalised rows.
 * status: NULL, or one int32 in device memory.  A position read from pos_dev that lies past the
 * tables (the reference asserts this on the host, attention.py:66) makes the kernel read the last
 * table row, write NaN outputs for the step and raise DAISY_STATUS_POSITION_PAST_TABLES in *status.
 */
int daisy_attn_step_fwd(const void* q, const int64_t* q_strides,
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
                        void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Kernel 3: chunked Kimi Delta Attention forward.
 *
 * Replaces the call  chunk_kda(q, k, v, g, beta, initial_state=...,
 * output_final_state=..., use_qk_l2norm_in_kernel=True)  at
 * models/daisy/attention_kimi.py:133-134 (the implementation is in the absent
 * third-party package flash-linear-attention).  Per (b, h), with fp32 state
 * S [Dk, Dv]:
 *   S <- diag(exp(g_t)) S;  S <- S + beta_t k_t (v_t - S^T k_t)^T;  o_t = scale * S^T q_t
 *
 * q, k  : bf16 [B, T, H, Dk] contiguous.     v, o : bf16 [B, T, H, Dv] contiguous.
 * g     : log-decay [B, T, H, Dk] contiguous, fp32 (g_is_bf16 = 0) or bf16 (1); <= 0.
 * beta  : fp32 [B, T, H] contiguous.
 * initial_state : fp32 [B, H, Dk, Dv] or NULL (zeros).
 * final_state   : fp32 [B, H, Dk, Dv] or NULL (not wanted).
 * Dk: a multiple of 8 up to 128.  Dv: any multiple of 8 (value columns are independent; they are
 * processed in passes of up to 128 through the same workspace).  chunk = 64.  T is arbitrary.  The
 * kernels are laid out for 128 x 128; narrower heads cost what 128 costs.
 * l2norm_qk : normalise q and k rows as x / sqrt(sum(x^2) + l2_eps) first.
 * workspace : >= daisy_kda_workspace_bytes(...) bytes, 256-byte aligned.
 */
size_t daisy_kda_workspace_bytes(int B, int T, int H, int Dk, int Dv, int chunk);

int daisy_kda_chunk_fwd(const void* q, const void* k, const void* v,
                        const void* g, int g_is_bf16, const float* beta,
                        const float* initial_state, void* o, float* final_state,
                        int B, int T, int H, int Dk, int Dv, int chunk,
                        float scale, int l2norm_qk, float l2_eps,
                        void* workspace, size_t workspace_bytes, void* stream);

/* The same forward over sequences packed along the token axis of a batch of one, the layout the
 * reference hands to chunk_kda(..., cu_seqlens=...) for a padded batch
 * (models/daisy/attention_kimi.py:133-134,150-154).  q, k, g: [T, H, Dk]; v, o: [T, H, Dv];
 * beta: [T, H]; cu_seqlens: int32 [n_seq + 1] in device memory, sequence i = rows
 * cu_seqlens[i] .. cu_seqlens[i+1] - 1, cu_seqlens[0] = 0, cu_seqlens[n_seq] = T, non-decreasing
 * (empty sequences allowed).  The bounds are read by the kernels, never by the host.  Every packed-
 * sequence kernel of this library (this one, daisy_kda_recurrent_varlen_fwd, daisy_short_conv_varlen_fwd)
 * forces each bound into 0..T, so that no bound can lead outside the tensors; rows that belong to no
 * sequence are left unwritten.  Bounds that DECREASE break the contract: every kernel stays inside the
 * tensors, but how tokens are then assigned to sequences differs between the kernels (this one takes
 * the running maximum of the bounds, the recurrent one clamps each pair, the convolution bisects over
 * them as they are) -- the three kernels of one layer agree only on bounds that honour the contract.
 * initial_state / final_state: fp32 [n_seq, H, Dk, Dv].
 */
size_t daisy_kda_varlen_workspace_bytes(int T, int n_seq, int H, int Dk, int Dv, int chunk);

int daisy_kda_chunk_varlen_fwd(const void* q, const void* k, const void* v,
                               const void* g, int g_is_bf16, const float* beta,
                               const int32_t* cu_seqlens, int n_seq,
                               const float* initial_state, void* o, float* final_state,
                               int T, int H, int Dk, int Dv, int chunk,
                               float scale, int l2norm_qk, float l2_eps,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Token-by-token KDA (the recurrence of daisy_kda_chunk_fwd evaluated one token
 * at a time, state in registers).  This is the "fused_recurrent" mode that
 * models/daisy/attention_kimi.py:70,144 names and leaves unsupported; a
 * generation loop calls it with T = 1 per step, carrying the state.
 *
 * Tensors and head widths as in daisy_kda_chunk_fwd (contiguous [B, T, H, D]).
 * initial_state NULL = zeros; final_state NULL = not wanted; the two may alias.
 */
int daisy_kda_recurrent_fwd(const void* q, const void* k, const void* v,
                            const void* g, int g_is_bf16, const float* beta,
                            const float* initial_state, void* o, float* final_state,
                            int B, int T, int H, int Dk, int Dv,
                            float scale, int l2norm_qk, float l2_eps, void* stream);

/* daisy_kda_recurrent_fwd over packed sequences (layout and cu_seqlens as in
 * daisy_kda_chunk_varlen_fwd; states [n_seq, H, Dk, Dv]). */
int daisy_kda_recurrent_varlen_fwd(const void* q, const void* k, const void* v,
                                   const void* g, int g_is_bf16, const float* beta,
                                   const int32_t* cu_seqlens, int n_seq,
                                   const float* initial_state, void* o, float* final_state,
                                   int T, int H, int Dk, int Dv,
                                   float scale, int l2norm_qk, float l2_eps, void* stream);

/* ---------------------------------------------------------------------------
 * KDA log-decay gate:  out[..., h, d] = -exp(A_log[h]) * softplus(g[..., h, d] + bias[h, d])
 * (softplus is the identity above `threshold`).  Replaces fused_kda_gate
 * (models/daisy/fla_custom_ops.py:71-103,190-200), forward only.
 *
 * g, out : [rows, H, Dk] contiguous, both bf16 (io_is_bf16 = 1) or both fp32 (0).
 * A_log  : fp32 [H].   bias : fp32 [H, Dk] or NULL.
 */
int daisy_kda_gate_fwd(const void* g, const float* A_log, const float* bias, void* out,
                       int64_t rows, int H, int Dk, int io_is_bf16,
                       float softplus_beta, float threshold, void* stream);

/* ---------------------------------------------------------------------------
 * Fused pre-attention pass over the QKV projection output.  Replaces, in one
 * streaming kernel, the elementwise chain of CausalSelfAttention._calc_qkv and
 * _qkv_common (models/daisy/attention.py:116-135): weightless RMS norm of q, k
 * and v (models/daisy/functional.py:6-7), RoPE of q and k (attention.py:16-20)
 * at table rows pos0 + t, and the value-embedding mix
 * v = gate * v + (1 - gate) * ve (attention.py:132-135).  Intermediates are
 * rounded to bf16 where the reference materialises bf16 tensors.
 *
 * q, k, v : bf16, logical [B, T, H, D], strides {b, t, h} in elements, D
 *           contiguous (typically three views of the [B, T, 3H, D] GEMM output).
 * ve, gate: ve bf16 [B, T, H, D] with strides, gate = device pointer to one fp32
 *           holding sigmoid(g_ve) already rounded to bf16; both NULL = no mix.
 * cos, sin: fp32 [>= pos0 + T, D/2] or both NULL = no RoPE.
 * q_out, k_out, v_out : bf16 with their own {b, t, h} strides (e.g. k_out and
 *           v_out may be laid out [B, H, T, D] or be rows of a KV cache).
 * eps     : added to mean(x^2) before the reciprocal square root.
 * D is 64 or 128.
 */
int daisy_qkv_prep_fwd(const void* q, const int64_t* q_strides,
                       const void* k, const int64_t* k_strides,
                       const void* v, const int64_t* v_strides,
                       const void* ve, const int64_t* ve_strides, const float* gate,
                       const float* cos, const float* sin, int pos0,
                       void* q_out, const int64_t* q_out_strides,
                       void* k_out, const int64_t* k_out_strides,
                       void* v_out, const int64_t* v_out_strides,
                       int B, int T, int H, int D, float eps, void* stream);

/* The same pass with the first position read from device memory when the kernel runs
 * (`pos0` points at one int32; the decode-step counterpart of Rotary.step's host `pos`,
 * models/daisy/attention.py:64-70).  cos, sin are fp32 [table_rows, D/2] and required; a
 * position whose rows would leave the table is held at the table's end, the rotated outputs of
 * the call are NaN and, when status (one int32 in device memory) is given,
 * DAISY_STATUS_POSITION_PAST_TABLES is raised in it.
 */
int daisy_qkv_prep_fwd_at(const void* q, const int64_t* q_strides,
                          const void* k, const int64_t* k_strides,
                          const void* v, const int64_t* v_strides,
                          const void* ve, const int64_t* ve_strides, const float* gate,
                          const float* cos, const float* sin, const int32_t* pos0, int table_rows, int32_t* status,
                          void* q_out, const int64_t* q_out_strides,
                          void* k_out, const int64_t* k_out_strides,
                          void* v_out, const int64_t* v_out_strides,
                          int B, int T, int H, int D, float eps, void* stream);

/* ---------------------------------------------------------------------------
 * The two projections of a decode step, F.linear(x, qkvo_w[:3].flatten(end_dim=1)) and
 * F.linear(y, qkvo_w[3]) (models/daisy/attention.py:119-120 and :201), for the one activation row per
 * sequence that a step has:
 *     y[m, n] = sum_k x[m, k] * w[n, k]        m < M <= 8
 * bf16 in and out, fp32 accumulation, one rounding at the end.  The call reads the weights once
 * (N * K * 2 bytes: bound by HBM bandwidth); more rows than 8 belong to a library GEMM
 * (DAISY_ERR_UNSUPPORTED).
 * x : [M, K] bf16, row stride x_row_stride elements;  w : [N, K] bf16 (the layout of a Linear weight),
 *     row stride w_row_stride;  y : [M, N] bf16, row stride y_row_stride.  K a multiple of 8; x, w and
 *     their row strides such that every row starts on a 16-byte boundary.
 */
int daisy_linear_rows_fwd(const void* x, int64_t x_row_stride, const void* w, int64_t w_row_stride,
                          void* y, int64_t y_row_stride, int M, int N, int K, void* stream);

/* One decode step of an attention layer in one call: CausalSelfAttention.step
 * (models/daisy/attention.py:181-202) from its input rows to its output rows,
 *     qkv = x W_qkv^T  (daisy_linear_rows_fwd);   o = daisy_attn_step_fwd on the three thirds of qkv;
 *     y = o W_out^T    (daisy_linear_rows_fwd),
 * as three launches (four with split partials) on `stream`.  Results are those of the three calls.
 * x      : bf16 [B, dim], row stride x_row_stride;  y : bf16 [B, dim], row stride y_row_stride;  B <= 8.
 * w_qkv  : bf16 [3*H*D, dim] (qkvo_w[:3] flattened: q rows, then k rows, then v rows);  w_out : bf16 [dim, H*D].
 * ve, gate, cos, sin, table_rows, pos, pos_dev, status, eps, the ring cache, cache_is_f16, ring_rows,
 * scale, nsplit : as for daisy_attn_step_fwd (ve: bf16 [B, H, D] with {batch, head} strides).
 * workspace : >= daisy_attn_layer_step_workspace_bytes(B, H, D, ring_rows, nsplit) bytes, 256-byte aligned
 *          (the projected rows, the attention output and the split partials; sized for the whole ring).
 */
size_t daisy_attn_layer_step_workspace_bytes(int B, int H, int D, int ring_rows, int nsplit);
int daisy_attn_layer_step_fwd(const void* x, int64_t x_row_stride,
                              const void* w_qkv, int64_t w_qkv_row_stride,
                              const void* w_out, int64_t w_out_row_stride,
                              const void* ve, const int64_t* ve_strides, const float* gate,
                              const float* cos, const float* sin, int table_rows,
                              int pos, const int32_t* pos_dev, int32_t* status, float eps,
                              void* k_cache, const int64_t* k_cache_strides,
                              void* v_cache, const int64_t* v_cache_strides, int cache_is_f16,
                              void* y, int64_t y_row_stride,
                              int B, int H, int D, int dim, int ring_rows,
                              float scale, int nsplit,
                              void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * The KDA layer's elementwise neighbours (models/daisy/attention_kimi.py:155-158: three
 * ShortConvolution modules in front of chunk_kda; :136-137: the gated RMS norm behind it; both
 * modules come from a package absent from the reference checkout and are restated from their
 * documented arithmetic).
 *
 * daisy_short_conv_fwd: depthwise causal convolution over time with K taps (2..4) per channel,
 * optional bias and SiLU, bf16 in and out:
 *     y[b, t, c] = act( bias[c] + sum_j weight[c, j] * x[b, t - (K-1) + j, c] )
 * x, y       : [B, T, C] bf16, channel stride 1, strides = {batch, time} in elements (multiples of 8)
 * weight     : [C, K] bf16 (the layout of a grouped Conv1d weight [C, 1, K]); bias: [C] bf16 or NULL
 * cache_in   : [B, C, K] bf16 or NULL -- the last K inputs before t = 0 (zeros if NULL)
 * cache_out  : [B, C, K] bf16 or NULL -- receives the last K inputs of (cache_in | x); may be the
 *              same buffer as cache_in when T <= 32 (decode steps update their window in place)
 * C must be a multiple of 8.
 */
int daisy_short_conv_fwd(const void* x, const int64_t* x_strides, const void* weight, const void* bias,
                         const void* cache_in, void* y, const int64_t* y_strides, void* cache_out,
                         int B, int T, int C, int K, int apply_silu, void* stream);

/* daisy_short_conv_fwd over sequences packed along T of a batch of one (the cu_seqlens argument of
 * the reference's ShortConvolution calls, attention_kimi.py:155-158): no tap reaches across the
 * start of its sequence.  x, y: [T, C] with a row stride; cu_seqlens as in
 * daisy_kda_chunk_varlen_fwd; cache_in / cache_out: [n_seq, C, K] or NULL (must differ).
 */
int daisy_short_conv_varlen_fwd(const void* x, int64_t x_row_stride, const void* weight, const void* bias,
                                const int32_t* cu_seqlens, int n_seq, const void* cache_in,
                                void* y, int64_t y_row_stride, void* cache_out,
                                int T, int C, int K, int apply_silu, void* stream);

/* daisy_gated_rmsnorm_fwd: out = x * rsqrt(mean(x^2) + eps) * weight * sigmoid(gate) over the last
 * dim, statistics in fp32, one rounding.  x, gate, out: [rows, D] bf16 contiguous; weight: [D] bf16;
 * D = 32, 64, 128 or 256.
 */
int daisy_gated_rmsnorm_fwd(const void* x, const void* gate, const void* weight, void* out,
                            int64_t rows, int D, float eps, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DAISY_HIP_H */
