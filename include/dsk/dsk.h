// dsk:: - the DeepSeek engine's MoE operator names (ds41f-4xgx10-switchless/engine/kernels/dsk.h:171-241,268-295) over
// the C ABI in dsgx.h, for the FP8 e4m3 / 128 x 128 block-scaled configuration. The reference's own expert format
// here is MXFP4 with FP8-quantised activations and ue8m0 scales; that arithmetic is not built, and a MoeWeights that
// carries MXFP4 tensors is refused with a message instead of being reinterpreted.
#pragma once
#include <cstddef>
#include <cstdint>

#include "../gx/check.h"

namespace dsk {

// dsk.h:171-176: scores sqrt(softplus(l)), top-k of scores + bias, weights = scores / (sum + 1e-20) * route_scale
inline void router_topk(const float* logits, const float* bias, int M, int E, int* idx, float* wts, float route_scale, void* st,
                        int topk = 6, int score_fn = 1) {
  DSGX_DIE_ON(dsgx_route(logits, bias, M, E, topk, route_scale, score_fn, idx, wts, st));
}

// dsk.h:199-209 keeps MXFP4 fields; this build takes the layer as a dsgx_layer_w of FP8_B128 matrices.
struct MoeWeights {
  const uint8_t *w1 = nullptr, *s1 = nullptr, *w3 = nullptr, *s3 = nullptr, *w2 = nullptr, *s2 = nullptr;  // MXFP4: refused
  const dsgx_layer_w* fp8 = nullptr;  // the FP8-128 layer (routed pool + descriptors + fused shared expert)
};
struct MoeCfg {
  int up = 0, down = 0;
  bool pdl = true;
  int phases = 3;
};
inline size_t moe_workspace_bytes(const MoeWeights& w) { return w.fp8 ? dsgx_decode_ws_bytes(w.fp8) : 0; }
// y [M][H] f32 = sum over each row's picks in expert-id order + the shared expert (dsk.h:226-233). x is bf16 here
// (the FP8-128 decode contract keeps bf16 activations); ys is scratch for the shared expert's output.
inline void moe(const uint16_t* x, int M, const int* idx, const float* wts, const MoeWeights& w, void* ws, float* y, float* ys,
                MoeCfg cfg, void* st) {
  if (w.w1 || w.w2 || w.w3) die("dsk::moe: MXFP4 experts are not built on this path; pass an FP8_B128 layer");
  if (!w.fp8) die("dsk::moe: no layer");
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.parts = cfg.phases, d.ysum = 1;
  DSGX_DIE_ON(dsgx_moe_decode(w.fp8, x, idx, wts, M, ws, y, ys, st, &d));
}
// the router's selection fused in (dsk.h:234-241)
inline void moe_routed(const uint16_t* x, int M, const float* logits, const float* bias, float route_scale, const MoeWeights& w,
                       void* ws, float* y, float* ys, MoeCfg cfg, void* st, int score_fn = 0) {
  if (w.w1 || w.w2 || w.w3) die("dsk::moe_routed: MXFP4 experts are not built on this path; pass an FP8_B128 layer");
  if (!w.fp8) die("dsk::moe_routed: no layer");
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.parts = cfg.phases, d.ysum = 1, d.logits = logits, d.bias = bias, d.route_scale = route_scale, d.score_fn = score_fn;
  DSGX_DIE_ON(dsgx_moe_decode(w.fp8, x, nullptr, nullptr, M, ws, y, ys, st, &d));
}
inline size_t moe_prefill_workspace_bytes(const MoeWeights& w, int M) { return w.fp8 ? dsgx_prefill_ws_bytes(w.fp8, M) : 0; }
inline void moe_prefill(const uint16_t* x, int M, const int* idx, const float* wts, const MoeWeights& w, void* ws, float* y, float* ys,
                        void* st, int phases = 31) {
  if (w.w1 || w.w2 || w.w3) die("dsk::moe_prefill: MXFP4 experts are not built on this path; pass an FP8_B128 layer");
  if (!w.fp8) die("dsk::moe_prefill: no layer");
  dsgx_prefill_cfg p;
  dsgx_prefill_cfg_default(&p);
  p.phases = phases;
  DSGX_DIE_ON(dsgx_moe_prefill(w.fp8, x, idx, wts, M, ws, y, ys, st, &p));
}

}  // namespace dsk
