// One decode step of an attention layer as one call: the two projections of
// CausalSelfAttention.step (models/daisy/attention.py:181-202) and everything between them.
//
// Three launches (four when the ring is split) on the caller's stream:
//   qkv = x W_qkv^T                         linear_rows_kernel            (linear.hip)
//   o   = attention of the new row over the ring, rows normalised, rotated, mixed and appended
//                                           decode_kernel<D, true, ...>   (decode.hip)
//   y   = o W_out^T                         linear_rows_kernel
// No device code of its own: for a host that drives the step token by token the cost of a layer is
// then one call instead of three (a Python caller spends more time between the launches of a
// one-sequence step than the GPU spends inside them).  The intermediate rows live in the caller's
// workspace, in front of the split partials.
#include "common.h"

namespace daisy {

static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

struct LayerStepLayout { size_t qkv_off, o_off, partials_off, partials_bytes, total; };

static LayerStepLayout layer_step_layout(int B, int H, int D, int rows_for_splits, int nsplit) {
  LayerStepLayout l;
  l.qkv_off = 0;
  l.o_off = align256((size_t)B * 3 * H * D * 2);
  l.partials_off = l.o_off + align256((size_t)B * H * D * 2);
  l.partials_bytes = daisy_decode_workspace_bytes(B, H, D, rows_for_splits, nsplit);
  l.total = l.partials_off + align256(l.partials_bytes);
  return l;
}

}  // namespace daisy

using namespace daisy;

extern "C" size_t daisy_attn_layer_step_workspace_bytes(int B, int H, int D, int ring_rows, int nsplit) {
  if (B <= 0 || H <= 0 || D <= 0 || ring_rows <= 0) return 0;
  return layer_step_layout(B, H, D, ring_rows, nsplit).total;
}

extern "C" int daisy_attn_layer_step_fwd(const void* x, int64_t x_row_stride,
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
                                         void* workspace, size_t workspace_bytes, void* stream) {
  DAISY_CHECK_ARG(x && w_qkv && w_out && y, "attn_layer_step: x, w_qkv, w_out and y must be non-NULL");
  DAISY_CHECK_ARG(B >= 1 && H >= 1 && dim >= 8 && ring_rows >= 1, "attn_layer_step: B=%d, H=%d, dim=%d, ring_rows=%d", B, H, dim, ring_rows);
  DAISY_CHECK_SUPPORTED(D == 64 || D == 128, "attn_layer_step: head_dim %d not supported (64 or 128)", D);
  DAISY_CHECK_ARG(pos_dev != nullptr || (pos >= 0 && pos < table_rows),
                  "attn_layer_step: position %d outside the rotary tables (%d rows)", pos, table_rows);
  // The partials are sized like daisy_attn_step_fwd sizes them: for the live rows when the host knows the
  // position, for the whole ring when only the device does.
  const int live = pos_dev ? ring_rows : (pos + 1 < ring_rows ? pos + 1 : ring_rows);
  const LayerStepLayout l = layer_step_layout(B, H, D, live, nsplit);
  DAISY_CHECK_ARG(workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 255) == 0 && workspace_bytes >= l.total,
                  "attn_layer_step: a 256-byte aligned workspace of %zu bytes is needed, got %zu", l.total, workspace_bytes);
  char* ws = static_cast<char*>(workspace);
  uint16_t* qkv = reinterpret_cast<uint16_t*>(ws + l.qkv_off);
  uint16_t* o = reinterpret_cast<uint16_t*>(ws + l.o_off);
  const int HD = H * D;

  int rc = daisy_linear_rows_fwd(x, x_row_stride, w_qkv, w_qkv_row_stride, qkv, 3 * (int64_t)HD, B, 3 * HD, dim, stream);
  if (rc != DAISY_OK) return rc;
  const int64_t row_strides[2] = {3 * (int64_t)HD, D};
  const int64_t o_strides[2] = {HD, D};
  rc = daisy_attn_step_fwd(qkv, row_strides, qkv + HD, row_strides, qkv + 2 * HD, row_strides, ve, ve_strides, gate,
                           cos, sin, table_rows, pos, pos_dev, status, eps, k_cache, k_cache_strides, v_cache,
                           v_cache_strides, cache_is_f16, o, o_strides, B, H, D, ring_rows, scale, nsplit,
                           l.partials_bytes ? ws + l.partials_off : nullptr, l.partials_bytes, stream);
  if (rc != DAISY_OK) return rc;
  return daisy_linear_rows_fwd(o, HD, w_out, w_out_row_stride, y, y_row_stride, B, dim, HD, stream);
}
