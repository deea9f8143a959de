// gx:: - the routed-expert operators with the reference engine's names and argument order
// (altar1-4xgx10-switchless/engine/experts/experts.h:15-195), forwarding to the C ABI in dsgx.h.
//
// What differs from the reference header, and why:
//  * cudaStream_t -> a hipStream_t passed as void*; __nv_bfloat16 -> uint16_t bit patterns.
//  * the per-rank shape constants (kH, kI, kE, kTopK: experts.h:18-26) are fields of LayerW, defaulting to the
//    reference's values, so the whole-layer shapes of one GPU (intermediate 2048) and the DeepSeek-shaped layer fit.
//  * Fmt gains the tags of the MI355X layouts (the checkpoint's row-major tensors); the reference's tags name GB10
//    block tilings and are refused by every operator.
//  * DecodeCfg::post (ring posting) must stay null; pdl is accepted and ignored (HIP has no programmatic dependent launch).
#pragma once
#include <cstddef>
#include <cstdint>

#include "check.h"

namespace gx {

constexpr int kH = 6144, kI = 512, kE = 168, kTopK = 8;  // the reference's per-rank defaults (experts.h:18-22)
constexpr float kRouteScale = 2.5f;
constexpr int kMaxRows = DSGX_MAX_ROWS, kMaxUnion = DSGX_MAX_UNION, kShSlot = DSGX_SH_SLOT, kMaxChunk = DSGX_MAX_CHUNK;

enum Fmt : uint32_t {
  kNVFP4 = DSGX_FMT_REF_NVFP4, kINT4 = DSGX_FMT_REF_INT4, kBF16 = DSGX_FMT_REF_BF16,  // GB10 tilings: refused
  kFP8B128 = DSGX_FMT_FP8_B128, kINT4G32 = DSGX_FMT_INT4_G32, kBF16Rows = DSGX_FMT_BF16
};
constexpr bool fmt_known(uint32_t f) { return f == kFP8B128 || f == kINT4G32 || f == kBF16Rows; }
inline size_t mat_bytes(uint32_t fmt, int N, int K) { return dsgx_mat_bytes(fmt, N, K); }
constexpr const char* fmt_name(uint32_t f) {
  return f == kFP8B128 ? "FP8_B128" : f == kINT4G32 ? "INT4_G32" : f == kBF16Rows ? "BF16" : "unknown";
}

using MatDesc = dsgx_mat_desc;
static_assert(sizeof(MatDesc) == 64, "MatDesc is 64 B");
// make_desc / desc_ok of the reference (engine/experts/layout.h:165-183)
inline MatDesc make_desc(uint64_t off, float s2, uint32_t fmt) {
  if (!fmt_known(fmt)) die("make_desc: expert format %u is not FP8_B128 (16), INT4_G32 (18) or BF16 (19)", fmt);
  MatDesc d{};
  d.off = off, d.s2 = s2, d.fmt = fmt;
  return d;
}
inline bool desc_ok(const MatDesc& d, uint32_t fmt) {
  if (d.fmt != fmt || !fmt_known(fmt) || d.off % 256) return false;
  if (!(d.s2 > 0.f) || d.s2 != d.s2 || d.s2 > 3.4e38f || d.s2 != 1.f) return false;
  for (uint32_t r : d.rsv)
    if (r) return false;
  return true;
}

struct SharedW : dsgx_shared_w {
  SharedW() : dsgx_shared_w{} {}
  bool fused() const { return g != nullptr; }
  bool bf16() const { return bgu != nullptr; }
};

struct LayerW {
  const uint8_t* pool = nullptr;
  const MatDesc* desc = nullptr;  // [E][3]: gate, up, down (device memory)
  SharedW sh;
  uint32_t fmt = kINT4G32;
  int H = kH, I = kI, E = kE, topk = kTopK;
  dsgx_layer_w c() const { return dsgx_layer_w{pool, desc, sh, fmt, H, I, E, topk}; }
};

// ---- routing (experts.h:99-102) -----------------------------------------------------------------------------------
// The first seven arguments are the reference's; the rest carry what its compile-time constants fix (168 experts, top-8,
// sigmoid scores scaled by 2.5). score_fn: 0 sigmoid, 1 sqrt(softplus) (the DeepSeek engine's router).
inline void route(const float* logits, const float* bias, int M, int* idx, float* w, void* st, bool pdl = true, int E = kE,
                  int topk = kTopK, float scale = kRouteScale, int score_fn = 0) {
  (void)pdl;
  DSGX_DIE_ON(dsgx_route(logits, bias, M, E, topk, scale, score_fn, idx, w, st));
}

// ---- decode (experts.h:104-147) -----------------------------------------------------------------------------------
// The reference's variant numbers name its launch shapes (decode.cu:624-698); here up / down are this build's variants
// (dsgx_decode_cfg). kUpPrefillOrder (experts.h:111-113,138: decode = prefill bit for bit) keeps its number and its
// promise: the rows go through the prefill kernels (DSGX_UP_PREFILL_ORDER).
constexpr int kUpPrefillOrder = DSGX_UP_PREFILL_ORDER;
struct DecodeCfg {
  int up = -1, down = 0;   // up -1: the faster variant for the layer's format and the row count
  int up_ctas_per_sm = 0;  // accepted, unused: the grid is sized to the chip
  bool pdl = true;         // accepted, unused
  bool dyn = true;         // accepted, unused: batches are claimed from a counter in LDS
  bool xpf = true;         // accepted, unused
  int parts = 3;
  const float* logits = nullptr;
  const float* bias = nullptr;
  float route_scale = kRouteScale;  // fused routing's scale (the reference's is the constant 2.5)
  int score_fn = 0;                 // fused routing's score: 0 sigmoid, 1 sqrt(softplus)
  const void* post = nullptr;       // must be null
  bool ysum = false;
};
inline size_t decode_ws_bytes(const LayerW& L) { const dsgx_layer_w c = L.c(); return dsgx_decode_ws_bytes(&c); }
// the reference's form (experts.h:139): the workspace of a layer of its compile-time shape (LayerW's defaults)
inline size_t decode_ws_bytes() { return decode_ws_bytes(LayerW()); }
inline void moe_decode(const LayerW& L, const uint16_t* x, const int* idx, const float* w, int M, void* ws, float* yr, float* ys,
                       void* st, const DecodeCfg& cfg = DecodeCfg()) {
  const dsgx_layer_w c = L.c();
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.up = cfg.up, d.down = cfg.down, d.parts = cfg.parts, d.ysum = cfg.ysum, d.logits = cfg.logits, d.bias = cfg.bias;
  d.route_scale = cfg.route_scale, d.score_fn = cfg.score_fn, d.post = cfg.post;
  DSGX_DIE_ON(dsgx_moe_decode(&c, x, idx, w, M, ws, yr, ys, st, &d));
}
// Dies if a fused decode step since the last check gave up at its grid barrier (its outputs are invalid). Waits for the
// stream: call it where the host waits for results anyway. No counterpart in the reference, whose two kernels are
// ordered by the stream.
inline void decode_check(const LayerW& L, void* ws, void* st) {
  const dsgx_layer_w c = L.c();
  DSGX_DIE_ON(dsgx_decode_status(&c, ws, st));
}
inline int decode_up_variants() { return 2; }
inline int decode_down_variants() { return 2; }
inline const char* decode_up_name(int v) { return v == 1 ? "mfma16 kslices" : "rows4 lanes64"; }
inline const char* decode_down_name(int v) { return v == 1 ? "two launches" : "rows2 lanes64"; }
// out[m][n] = bf16(bf16(R) + bf16(S)) over M rows (experts.h:146-147, decode.cu:591-598). The reference's form takes M and
// uses its compile-time hidden size, 6144: for a layer of another width pass the layer.
inline void finalize(const float* R, const float* S, int M, uint16_t* out, void* st, bool pdl = true) {
  (void)pdl;
  DSGX_DIE_ON(dsgx_finalize(R, S, M * kH, out, st));
}
inline void finalize(const LayerW& L, const float* R, const float* S, int M, uint16_t* out, void* st) {
  DSGX_DIE_ON(dsgx_finalize(R, S, M * L.H, out, st));
}

// ---- prefill (experts.h:149-193) ----------------------------------------------------------------------------------
enum PrefillPhase { kPhBucket = 1, kPhUp = 2, kPhDown = 4, kPhCombine = 8, kPhShared = 16, kPhAll = 31 };
struct PrefillCfg {
  bool shared = true;
  int diag = 0, ddiag = 0;  // accepted, must be 0
  int down = 1, up = 1;     // accepted, unused (one implementation of each)
  int sh_rows = 128, yr_kb = 0, chain_q = 4;
  void* side = nullptr;     // accepted, unused
  bool act_fp8 = true;      // FP8 layers: e4m3 activations on the fp8 MFMA (see dsgx_prefill_cfg)
  bool fast_act = false;    // ... with SwiGLU by the hardware's exp2 / rcp (see dsgx_prefill_cfg)
  int tile_order = -1;      // ... and the order the grouped GEMMs walk the tiles in (see dsgx_prefill_cfg; the same bits in any)
};
inline size_t prefill_ws_bytes(const LayerW& L, int T) { const dsgx_layer_w c = L.c(); return dsgx_prefill_ws_bytes(&c, T); }
inline size_t prefill_ws_bytes(int T) { return prefill_ws_bytes(LayerW(), T); }  // the reference's form (experts.h:180)
inline void moe_prefill_phases(const LayerW& L, const uint16_t* x, const int* idx, const float* w, int T, void* ws, float* yr,
                               float* ys, void* st, const PrefillCfg& cfg, int phases) {
  if (cfg.diag || cfg.ddiag) die("moe_prefill: bench diagnostics are not built");
  const dsgx_layer_w c = L.c();
  dsgx_prefill_cfg p;
  dsgx_prefill_cfg_default(&p);
  p.shared = cfg.shared, p.phases = phases, p.act_fp8 = cfg.act_fp8, p.fast_act = cfg.fast_act, p.tile_order = cfg.tile_order;
  DSGX_DIE_ON(dsgx_moe_prefill(&c, x, idx, w, T, ws, yr, ys, st, &p));
}
inline void moe_prefill(const LayerW& L, const uint16_t* x, const int* idx, const float* w, int T, void* ws, float* yr, float* ys,
                        void* st, const PrefillCfg& cfg = PrefillCfg()) {
  moe_prefill_phases(L, x, idx, w, T, ws, yr, ys, st, cfg, kPhAll);
}
struct PrefillView {
  const int *rpos, *re;
  const uint16_t *h, *hsh;
};
inline PrefillView prefill_view(const LayerW& L, void* ws, int T) {
  const dsgx_layer_w c = L.c();
  dsgx_prefill_view v;
  DSGX_DIE_ON(dsgx_prefill_view_get(&c, ws, T, &v));
  return PrefillView{v.rpos, v.re, v.h, v.hsh};
}
inline PrefillView prefill_view(void* ws, int T) { return prefill_view(LayerW(), ws, T); }  // the reference's form (experts.h:190)

}  // namespace gx
