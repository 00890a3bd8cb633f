// One call per MixedQLinear forward: the layer's buffers are described once (quik_layer), a forward picks the
// kernels (weight-streaming kernel up to 32 rows, tile-ordered paths above when the layer has a tile-ordered
// weight copy) and launches quantize + fused GEMM.  Host code only; every kernel is reached through the entry
// points declared in quik_hip.h.  (Replaces the op sequence of MixedQLinear.forward, experiments/qlinear.py:80-148
// of the reference, for callers that want one boundary crossing per layer.)
#include "common.h"

#include <atomic>

namespace quik {
namespace {

inline int64_t align256(int64_t v) { return (v + 255) & ~int64_t(255); }

// quik_layer_set_one_launch: tests and measurements switch the one-launch form of small calls off to compare
std::atomic<bool> layer_one_launch{true};  // (read by every forward, possibly from several host threads)

struct LayerPlan {
  bool tiled;
  int64_t off_q, off_meta, off_fp, bytes;
};

bool layer_valid(const quik_layer *l) {
  return l && l->struct_bytes == static_cast<int32_t>(sizeof(quik_layer)) && (l->bits == 4 || l->bits == 8) &&
         (l->dtype == QUIK_F16 || l->dtype == QUIK_BF16) && l->num_int > 0 && l->num_fp >= 0 &&
         l->num_int + l->num_fp == l->in_features && l->out_features > 0;
}

// tile-ordered path: the layer has a tile-ordered weight copy, enough rows, a column map that streams, a shape the
// operand formats take; symmetric activations are fp16 only
bool use_tiled(const quik_layer *l, int64_t rows) {
  if (!l->tiled_weight || rows < l->tiled_min_rows || !l->colmap_streams) return false;
  if (l->symmetric && l->dtype != QUIK_F16) return false;
  return (l->bits == 4 ? quik_fp6_operand_bytes(rows, l->num_int, l->num_fp)
                       : quik_tile8_operand_bytes(rows, l->num_int, l->num_fp)) > 0;
}

LayerPlan plan_layer(const quik_layer *l, int64_t rows) {
  LayerPlan p{};
  p.tiled = use_tiled(l, rows);
  const int64_t meta_bytes = align256((l->symmetric ? 1 : 2) * rows * 2);
  if (p.tiled) {
    const int64_t qb = l->bits == 4 ? quik_fp6_operand_bytes(rows, l->num_int, l->num_fp)
                                    : quik_tile8_operand_bytes(rows, l->num_int, l->num_fp);
    p.off_q = 0;
    p.off_meta = align256(qb);
    p.off_fp = p.off_meta + meta_bytes;
    p.bytes = p.off_fp;
  } else {
    p.off_q = 0;
    p.off_meta = align256(rows * (l->bits == 4 ? l->num_int / 2 : l->num_int));
    p.off_fp = p.off_meta + meta_bytes;
    p.bytes = p.off_fp + align256(rows * l->num_fp * 2);
  }
  return p;
}

}  // namespace
}  // namespace quik

using namespace quik;

extern "C" void quik_layer_set_one_launch(int on) { layer_one_launch.store(on != 0, std::memory_order_relaxed); }

extern "C" int64_t quik_layer_workspace_bytes(const quik_layer *layer, int64_t rows) {
  if (!layer_valid(layer) || rows <= 0) return 0;
  return plan_layer(layer, rows).bytes;
}

extern "C" int quik_layer_forward(const quik_layer *layer, const void *x, int64_t rows, void *workspace,
                                  int64_t workspace_bytes, void *splitk_workspace, int64_t splitk_bytes, void *out,
                                  void *mid_event, void *stream) {
  if (!layer_valid(layer)) return QUIK_ERR_SHAPE;
  if (rows < 0) return QUIK_ERR_SHAPE;
  if (rows == 0) return QUIK_OK;
  if (!x || !workspace || !out || !layer->colmap || !layer->weights_scales) return QUIK_ERR_NULL;
  if (!layer->symmetric && !layer->reduced_w) return QUIK_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(workspace) % 256 != 0) return QUIK_ERR_ALIGN;
  const quik_layer &l = *layer;
  const LayerPlan p = plan_layer(layer, rows);
  // the row-major weights are read only by calls that do not take the tile-ordered path: a layer whose every call
  // does (tiled_min_rows <= 1) may leave them NULL
  if (!p.tiled && (!l.int_weight || (l.num_fp > 0 && !l.fp_weight))) return QUIK_ERR_NULL;
  if (workspace_bytes < p.bytes) return QUIK_ERR_RANGE;
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  void *q = ws + p.off_q, *meta = ws + p.off_meta, *fp_x = l.num_fp > 0 ? ws + p.off_fp : nullptr;
  const void *w_red = l.symmetric ? nullptr : l.reduced_w;
  if (!p.tiled && l.colmap_streams && layer_one_launch.load(std::memory_order_relaxed) && (!l.symmetric || l.dtype == QUIK_F16)) {
    // one or two token rows: one launch, the quantize inside the weight-streaming kernel (the workspace is not used)
    const int rc = gemv_forward_one_launch(x, l.dtype, rows, l.in_features, l.colmap, l.num_int, l.num_fp, l.bits,
                                           l.int_weight, l.weights_scales, w_red, l.fp_weight, l.bias, l.out_features,
                                           out, l.sym_divisor, as_stream(stream));
    if (rc != kChainNotHandled) {
      if (rc == QUIK_OK && mid_event) {  // (profiling hook: there is no second launch to mark)
        if (hipError_t e = hipEventRecord(static_cast<hipEvent_t>(mid_event), as_stream(stream)); e != hipSuccess) {
          set_last_hip_error(e);
          return QUIK_ERR_LAUNCH;
        }
      }
      return rc;
    }
  }
  if (l.symmetric) {
    if (l.dtype != QUIK_F16 || !l.colmap_streams) return QUIK_ERR_DTYPE;  // the caller's op sequence serves these
    if (int rc = quik_sym_quantize_mapped(x, rows, l.in_features, l.colmap, l.num_int, l.num_fp, l.bits, l.sym_divisor,
                                          p.tiled ? 1 : 0, q, meta, fp_x, stream))
      return rc;
  } else if (p.tiled) {
    if (int rc = l.bits == 4 ? quik_asym_quantize_fp6(x, l.dtype, rows, l.in_features, l.colmap, l.num_int, l.num_fp, q,
                                                      meta, stream)
                             : quik_asym_quantize_tile8(x, l.dtype, rows, l.in_features, l.colmap, l.num_int, l.num_fp,
                                                        q, meta, stream))
      return rc;
  } else {
    if (int rc = quik_asym_quantize(x, l.dtype, rows, l.in_features, l.colmap, l.num_int, l.num_fp, l.bits, q, meta, fp_x,
                                    stream))
      return rc;
  }
  if (mid_event) {  // profiling hook: the boundary between the two launches, on the launch stream
    hipError_t e = hipEventRecord(static_cast<hipEvent_t>(mid_event), as_stream(stream));
    if (e != hipSuccess) {
      set_last_hip_error(e);
      return QUIK_ERR_LAUNCH;
    }
  }
  if (p.tiled) {
    return l.bits == 4 ? quik_mixed_linear_fwd_fp6_ws(q, l.tiled_weight, meta, l.weights_scales, w_red, l.bias, l.dtype,
                                                      rows, l.out_features, l.num_int, l.num_fp, out, splitk_workspace,
                                                      splitk_bytes, stream)
                       : quik_mixed_linear_fwd_tile8_ws(q, l.tiled_weight, meta, l.weights_scales, w_red, l.bias, l.dtype,
                                                        rows, l.out_features, l.num_int, l.num_fp, out,
                                                        splitk_workspace, splitk_bytes, stream);
  }
  return quik_mixed_linear_fwd(q, l.int_weight, meta, l.weights_scales, w_red, fp_x, l.fp_weight, l.bias, l.dtype, rows,
                               l.out_features, l.num_int, l.num_fp, l.bits, out, stream);
}
