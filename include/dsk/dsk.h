// dsk:: - the DeepSeek engine's MoE operators (ds41f-4xgx10-switchless/engine/kernels/dsk.h:171-241, 268-295) with the
// reference's names, argument lists and defaults, over the C ABI in dsgx.h. A caller written against the reference's
// header compiles against this one: cudaStream_t becomes a HIP stream (taken as void*), device pointers stay as they are.
//
// What differs, and why:
//  - Layouts. The reference's MoeWeights tensors are re-laid at load time for the GB10 lane map (tile_fp4 / tile_fp8, dsk.h:
//    177-180). Here the load-time step keeps the checkpoint's row-major form (DSGX_FMT_MXFP4_G32 / DSGX_FMT_FP8_B32E), which
//    is the coalesced streaming layout on gfx950: tile_fp4 / tile_fp8 below are plain copies, so a loader that calls them
//    and stacks the results by expert id, as the reference's does, produces what these operators read.
//  - Shapes. The reference compiles its shapes in (hidden 5120, intermediate 576 a rank at TP = 4, top-6). They are runtime
//    values here, set once with dsk::set_shape (default: the whole layer on one GPU, hidden 5120, intermediate 2304,
//    256 routed experts, top-6); moe_workspace_bytes() and moe() read them.
//  - The 1-bit scale code (ScaleCode, dsk.h:181-198) is accepted and must be empty: scales are read as stored.
//  - moe_prefill is grouped GEMMs on the block-scaled matrix instruction (dsgx_dsk_moe_prefill). The reference promises
//    "the same result as moe()" (dsk.h:284-286) because its two paths share one MMA; here the chunk's dot products are
//    summed by the block-scaled MFMA and moe()'s by the bf16 MFMA, so a row's y agrees between the two to the tolerance both
//    are tested at (relative L2 ~1e-3), not bit for bit. moe_prefill_rows() is moe() over the chunk sixteen rows at a
//    time for a caller that needs moe()'s bits.
// The FP8 e4m3 / 128 x 128 block-scaled configuration (bf16 rows, a dsgx_layer_w) is served by the overloads at the end.
#pragma once
#include <cstddef>
#include <cstdint>

#include "../gx/check.h"

namespace dsk {

constexpr int kLowRows = 8;    // dsk.h:22-27
constexpr int kMaxRows = 16;
constexpr int kTopK = 6;
constexpr int kMaxUnion = kMaxRows * kTopK;
constexpr int row_budget(int M) { return M <= kLowRows ? kLowRows : kMaxRows; }

struct Shape {
  int dim = 5120, inter = 2304, experts = 256, topk = kTopK;
};
inline Shape& shape() {
  static Shape s;
  return s;
}
inline void set_shape(int dim, int inter, int experts, int topk = kTopK) { shape() = Shape{dim, inter, experts, topk}; }

// dsk.h:171-176: scores sqrt(softplus(l)), top-6 of scores + bias (descending), weights = scores / (sum + 1e-20) * route_scale
inline void router_topk(const float* logits, const float* bias, int M, int E, int* idx, float* wts, float route_scale, void* st) {
  DSGX_DIE_ON(dsgx_route(logits, bias, M, E, shape().topk, route_scale, 1, idx, wts, st));
}

// dsk.h:177-180 (tile_fp4) and its FP8 twin: the load-time re-layout. Row-major is this build's layout, so both copy:
// w [N][K/2] (e2m1 pairs, low nibble first), s [N][K/32] -> wt, st of the same sizes; FP8: w [N][K], s [N/32][K/32].
inline void tile_fp4(const uint8_t* w, const uint8_t* s, uint8_t* wt, uint8_t* st, int N, int K, void* stream) {
  DSGX_DIE_ON(dsgx_stream_copy(w, wt, (size_t)N * K / 2, stream));
  DSGX_DIE_ON(dsgx_stream_copy(s, st, (size_t)N * K / 32, stream));
}
inline void tile_fp8(const uint8_t* w, const uint8_t* s, uint8_t* wt, uint8_t* st, int N, int K, void* stream) {
  DSGX_DIE_ON(dsgx_stream_copy(w, wt, (size_t)N * K, stream));
  DSGX_DIE_ON(dsgx_stream_copy(s, st, (size_t)(N / 32) * (K / 32), stream));
}

// dsk.h:181-198: the reference's 1-bit code of the scale tensors, a GB10 bandwidth saving. Accepted empty only.
struct ScaleCode {
  const uint32_t* code = nullptr;
  uint32_t base4 = 0;
};

// dsk.h:199-209. Routed experts stacked by expert id ([E][rows][...]: expert e at e times the per-expert size): w1, w3
// [inter][dim] and w2 [dim][inter] MXFP4 with their ue8m0 scales; the shared expert FP8 with [N/32][K/32] scales.
struct MoeWeights {
  const uint8_t *w1, *s1, *w3, *s3, *w2, *s2;
  const uint8_t *sh_w1, *sh_s1, *sh_w3, *sh_s3, *sh_w2, *sh_s2;
  ScaleCode c1{}, c3{}, c2{};
};

// dsk.h:211-223. The variants name the reference's GB10 launch shapes; one implementation serves them all here.
struct MoeCfg {
  int up = 0, down = 4;
  int up_grid = 0;
  bool pdl = true;
  int phases = 3;  // bit 0: moe_up, bit 1: moe_down (benchmarks)
  bool dyn = false;
  int up16 = 4, down16 = 2;
};

namespace detail {
inline dsgx_dsk_weights c_weights(const MoeWeights& w, const char* who) {
  if (w.c1.code || w.c3.code || w.c2.code) die("%s: the 1-bit scale code is a GB10 format; pass the scales as stored (ScaleCode empty)", who);
  const Shape& s = shape();
  return dsgx_dsk_weights{w.w1, w.s1, w.w3, w.s3, w.w2, w.s2, w.sh_w1, w.sh_s1, w.sh_w3, w.sh_s3, w.sh_w2, w.sh_s2, s.dim, s.inter, s.experts, s.topk};
}
}  // namespace detail

// dsk.h:225
inline size_t moe_workspace_bytes() { return dsgx_dsk_ws_bytes(shape().dim, shape().inter); }

// dsk.h:226-233: y [M][dim] f32 = the sum over each row's picks, in expert-id order, of bf16(expert(x) * weight), plus the
// shared expert. xq / xs = act_quant(x); idx / wts [M][6] from the router; ws of moe_workspace_bytes(), zeroed once.
inline void moe(const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* wts, const MoeWeights& w, void* ws, float* y,
                MoeCfg cfg, void* st) {
  const dsgx_dsk_weights c = detail::c_weights(w, "dsk::moe");
  dsgx_dsk_cfg d;
  dsgx_dsk_cfg_default(&d);
  d.parts = cfg.phases;
  DSGX_DIE_ON(dsgx_dsk_moe_stacked(&c, xq, xs, M, idx, wts, ws, y, st, &d, nullptr, nullptr));
}
// dsk.h:234-241: the same with router_topk's selection inside the kernel; idx_out / wts_out [M][6] (optional) receive it
inline void moe_routed(const uint8_t* xq, const uint8_t* xs, int M, const float* logits, const float* bias, int E, float route_scale,
                       const MoeWeights& w, void* ws, float* y, MoeCfg cfg, void* st, int* idx_out = nullptr, float* wts_out = nullptr) {
  if (E != shape().experts) die("dsk::moe_routed: %d logits a row for a layer of %d experts (dsk::set_shape)", E, shape().experts);
  if ((idx_out == nullptr) != (wts_out == nullptr)) die("dsk::moe_routed: idx_out and wts_out go together");
  const dsgx_dsk_weights c = detail::c_weights(w, "dsk::moe_routed");
  dsgx_dsk_cfg d;
  dsgx_dsk_cfg_default(&d);
  d.parts = cfg.phases, d.logits = logits, d.bias = bias, d.route_scale = route_scale;
  DSGX_DIE_ON(dsgx_dsk_moe_stacked(&c, xq, xs, M, nullptr, nullptr, ws, y, st, &d, idx_out, wts_out));
}

// dsk.h:268-295: picks bucketed by expert, grouped GEMMs, each pick's output rounded to bf16, then per row summed in
// expert-id order in fp32, shared expert last. ws: moe_prefill_workspace_bytes(M, E) bytes, no initialisation needed.
struct MoePCfg {
  int phases = 31;        // 1 bucketing, 2 shared expert, 4 routed up, 8 routed down, 16 combine
  void* side = nullptr;   // accepted, unused: the shared expert runs on st
  int col0 = 0, cols = 0; // must be 0: all columns
};
inline size_t moe_prefill_workspace_bytes(int M, int E) {
  const Shape& s = shape();
  const size_t a = dsgx_dsk_prefill_ws_bytes(s.dim, s.inter, E, s.topk, M), b = moe_workspace_bytes();
  return a > b ? a : b;  // (so that moe_prefill_rows can use the same buffer)
}
inline void moe_prefill(const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* wts, int E, const MoeWeights& w, void* ws,
                        float* y, void* st, MoePCfg cfg = MoePCfg{}) {
  if (E != shape().experts) die("dsk::moe_prefill: E %d for a layer of %d experts (dsk::set_shape)", E, shape().experts);
  if (cfg.col0 || cfg.cols) die("dsk::moe_prefill: columns [%d, +%d): all columns only", cfg.col0, cfg.cols);
  const dsgx_dsk_weights c = detail::c_weights(w, "dsk::moe_prefill");
  dsgx_dsk_prefill_cfg p;
  dsgx_dsk_prefill_cfg_default(&p);
  p.phases = cfg.phases;
  DSGX_DIE_ON(dsgx_dsk_moe_prefill(&c, xq, xs, M, idx, wts, ws, y, st, &p));
}
// moe() over a chunk, sixteen rows at a time: moe()'s bits for every row. ws: moe_workspace_bytes(), ZEROED once.
inline void moe_prefill_rows(const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* wts, const MoeWeights& w, void* ws,
                             float* y, void* st) {
  const Shape& s = shape();
  for (int m0 = 0; m0 < M; m0 += kMaxRows) {
    const int m = M - m0 < kMaxRows ? M - m0 : kMaxRows;
    moe(xq + (size_t)m0 * s.dim, xs + (size_t)m0 * (s.dim / 32), m, idx + (size_t)m0 * s.topk, wts + (size_t)m0 * s.topk, w, ws,
        y + (size_t)m0 * s.dim, MoeCfg{}, st);
  }
}

// ---- the FP8 e4m3 / 128 x 128 block-scaled configuration: bf16 rows, a dsgx_layer_w (pool + descriptors + fused shared expert) ----
inline size_t moe_workspace_bytes(const dsgx_layer_w& L) { return dsgx_decode_ws_bytes(&L); }
// y = the routed sum + the shared expert's rows; ys: scratch f32 [M][H] for the latter
inline void moe(const uint16_t* x, int M, const int* idx, const float* wts, const dsgx_layer_w& L, void* ws, float* y, float* ys, MoeCfg cfg,
                void* st) {
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.parts = cfg.phases, d.ysum = 1;
  DSGX_DIE_ON(dsgx_moe_decode(&L, x, idx, wts, M, ws, y, ys, st, &d));
}
inline void moe_routed(const uint16_t* x, int M, const float* logits, const float* bias, float route_scale, const dsgx_layer_w& L, void* ws,
                       float* y, float* ys, MoeCfg cfg, void* st, int score_fn = 0) {
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.parts = cfg.phases, d.ysum = 1, d.logits = logits, d.bias = bias, d.route_scale = route_scale, d.score_fn = score_fn;
  DSGX_DIE_ON(dsgx_moe_decode(&L, x, nullptr, nullptr, M, ws, y, ys, st, &d));
}
inline size_t moe_prefill_workspace_bytes(const dsgx_layer_w& L, int M) { return dsgx_prefill_ws_bytes(&L, M); }
inline void moe_prefill(const uint16_t* x, int M, const int* idx, const float* wts, const dsgx_layer_w& L, void* ws, float* y, float* ys, void* st,
                        int phases = 31) {
  dsgx_prefill_cfg p;
  dsgx_prefill_cfg_default(&p);
  p.phases = phases;
  DSGX_DIE_ON(dsgx_moe_prefill(&L, x, idx, wts, M, ws, y, ys, st, &p));
}

}  // namespace dsk
