// Compiles the C++ mirror headers as plain C++17 (no HIP) and checks, without a GPU, what they promise at the type
// level: the reference's names, the 64-byte descriptor, and the descriptor verdicts of the reference's loader check
// (altar1-4xgx10-switchless/engine/experts/tests/test_experts.cu:135-158) at this build's tags.
#include <cstdio>
#include <cmath>
#include <initializer_list>

#include "dsk/dsk.h"
#include "glm/attn.h"
#include "gx/experts.h"

int main() {
  int bad = 0, n = 0;
  for (uint32_t f : {gx::kFP8B128, gx::kINT4G32, gx::kBF16Rows}) {
    const gx::MatDesc d = gx::make_desc(4096, 1.f, f);
    bad += !gx::desc_ok(d, f), ++n;
    for (uint32_t g : {(uint32_t)gx::kFP8B128, (uint32_t)gx::kINT4G32, (uint32_t)gx::kBF16Rows, 0u, 1u, 2u, 3u, 4u})
      if (g != f) bad += gx::desc_ok(d, g), ++n;
    gx::MatDesc e = d;
    e.off += 128;
    bad += gx::desc_ok(e, f), ++n;
    e = d;
    e.rsv[7] = 1;
    bad += gx::desc_ok(e, f), ++n;
    e = d;
    e.s2 = 2.f;
    bad += gx::desc_ok(e, f), ++n;
    e = d;
    e.s2 = NAN;
    bad += gx::desc_ok(e, f), ++n;
  }
  bad += gx::mat_bytes(1, 512, 6144) != 0 || gx::mat_bytes(7, 512, 6144) != 0 || gx::mat_bytes(gx::kINT4, 512, 6144) != 0, ++n;
  bad += gx::mat_bytes(gx::kINT4G32, 2048, 6144) != 7274496, ++n;
  gx::LayerW L;
  bad += !(L.H == 6144 && L.I == 512 && L.E == 168 && L.topk == 8), ++n;
  gx::DecodeCfg dc;
  gx::PrefillCfg pc;
  glm::GemvSeg seg;
  dsk::MoeWeights mw{};
  dsk::MoeCfg mc;
  bad += dc.parts != 3 || !pc.shared || seg.rs != 128 || mw.sh_w1 != nullptr || mw.c1.code != nullptr || mc.phases != 3 || mc.down != 4, ++n;
  // the reference's argument lists (ds41f-4xgx10-switchless/engine/kernels/dsk.h:171-176, 225-241, 284-295): these initialisations
  // only compile if the mirror declares exactly them
  void (*p_topk)(const float*, const float*, int, int, int*, float*, float, void*) = &dsk::router_topk;
  size_t (*p_ws)() = &dsk::moe_workspace_bytes;
  void (*p_moe)(const uint8_t*, const uint8_t*, int, const int*, const float*, const dsk::MoeWeights&, void*, float*, dsk::MoeCfg, void*) = &dsk::moe;
  void (*p_routed)(const uint8_t*, const uint8_t*, int, const float*, const float*, int, float, const dsk::MoeWeights&, void*, float*, dsk::MoeCfg,
                   void*, int*, float*) = &dsk::moe_routed;
  size_t (*p_pws)(int, int) = &dsk::moe_prefill_workspace_bytes;
  void (*p_pf)(const uint8_t*, const uint8_t*, int, const int*, const float*, int, const dsk::MoeWeights&, void*, float*, void*, dsk::MoePCfg) =
      &dsk::moe_prefill;
  bad += !p_topk || !p_ws || !p_moe || !p_routed || !p_pws || !p_pf, ++n;
  bad += dsk::kTopK != 6 || dsk::row_budget(9) != 16 || dsk::shape().dim != 5120, ++n;
  bad += gx::decode_ws_bytes(L) < (size_t)(128 + 1) * 16 * 512 * 2 + 256, ++n;  // h as decode.cu:33-35, then the counters
  std::printf("CHECK mirror headers %s  %d wrong of %d\n", bad ? "FAIL" : "ok", bad, n);
  return bad != 0;
}
