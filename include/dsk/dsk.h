// dsk:: - the DeepSeek engine's MoE operator names (ds41f-4xgx10-switchless/engine/kernels/dsk.h:171-241,268-295) over
// the C ABI in dsgx.h. Two layer kinds: the reference's own - MXFP4 routed experts + FP8 shared expert with ue8m0 scales,
// FP8-quantised rows, its expert arithmetic (MoeWeights::mx: a dsgx_layer_w of MXFP4_G32 matrices in the checkpoint's
// row-major form; the reference's tiled L3 tensors w1 / s1 ... are a GB10 lane order and are refused, never reinterpreted)
// - and the FP8 e4m3 / 128 x 128 block-scaled configuration with bf16 rows (MoeWeights::fp8).
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
  const uint8_t *w1 = nullptr, *s1 = nullptr, *w3 = nullptr, *s3 = nullptr, *w2 = nullptr, *s2 = nullptr;  // tiled L3: refused
  const dsgx_layer_w* fp8 = nullptr;  // the FP8-128 layer (routed pool + descriptors + fused shared expert)
  const dsgx_layer_w* mx = nullptr;   // the MXFP4_G32 layer (pool + descriptors; sh.g/u/d + sh.gs/us/ds as ue8m0 bytes: FP8_B32E)
};
struct MoeCfg {
  int up = 0, down = 0;
  bool pdl = true;
  int phases = 3;
};
inline size_t moe_workspace_bytes(const MoeWeights& w) { return w.mx ? dsgx_decode_ws_bytes(w.mx) : w.fp8 ? dsgx_decode_ws_bytes(w.fp8) : 0; }
// y [M][H] f32 = sum over each row's picks in expert-id order + the shared expert (dsk.h:226-233). x is bf16 here
// (the FP8-128 decode contract keeps bf16 activations); ys is scratch for the shared expert's output.
inline void moe(const uint16_t* x, int M, const int* idx, const float* wts, const MoeWeights& w, void* ws, float* y, float* ys,
                MoeCfg cfg, void* st) {
  if (w.w1 || w.w2 || w.w3) die("dsk::moe: bf16 rows go with an FP8_B128 layer (MoeWeights::fp8); MXFP4 layers take act_quant(x)");
  if (!w.fp8) die("dsk::moe: no layer");
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.parts = cfg.phases, d.ysum = 1;
  DSGX_DIE_ON(dsgx_moe_decode(w.fp8, x, idx, wts, M, ws, y, ys, st, &d));
}
// dsk.h:226-233, the reference's own form: xq / xs = act_quant(x) (e4m3 [M][H], ue8m0 [M][H / 32]), MXFP4 experts, the
// shared expert last. ys: scratch f32 [M][H] (receives the shared expert's output; the reference keeps it in shared memory).
inline void moe(const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* wts, const MoeWeights& w, void* ws, float* y,
                MoeCfg cfg, void* st, float* ys, float swiglu_limit = 10.f) {
  if (w.w1 || w.w2 || w.w3) die("dsk::moe: the tiled MXFP4 tensors are a GB10 lane order; pass the layer in row-major form (MoeWeights::mx)");
  if (!w.mx) die("dsk::moe: no MXFP4 layer");
  dsgx_dsk_cfg d;
  dsgx_dsk_cfg_default(&d);
  d.parts = cfg.phases, d.swiglu_limit = swiglu_limit;
  DSGX_DIE_ON(dsgx_dsk_moe(w.mx, xq, xs, M, idx, wts, ws, y, ys, st, &d));
}
// dsk.h:234-241: the same with router_topk's selection inside the kernels
inline void moe_routed(const uint8_t* xq, const uint8_t* xs, int M, const float* logits, const float* bias, int E, float route_scale,
                       const MoeWeights& w, void* ws, float* y, MoeCfg cfg, void* st, float* ys, float swiglu_limit = 10.f) {
  if (w.w1 || w.w2 || w.w3) die("dsk::moe_routed: the tiled MXFP4 tensors are a GB10 lane order; pass the layer in row-major form (MoeWeights::mx)");
  if (!w.mx) die("dsk::moe_routed: no MXFP4 layer");
  if (E != w.mx->E) die("dsk::moe_routed: %d logits a row for a layer of %d experts", E, w.mx->E);
  dsgx_dsk_cfg d;
  dsgx_dsk_cfg_default(&d);
  d.parts = cfg.phases, d.swiglu_limit = swiglu_limit, d.logits = logits, d.bias = bias, d.route_scale = route_scale;
  DSGX_DIE_ON(dsgx_dsk_moe(w.mx, xq, xs, M, nullptr, nullptr, ws, y, ys, st, &d));
}
// the router's selection fused in (dsk.h:234-241), FP8-128 layers
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
