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
  dsk::MoeWeights mw;
  bad += dc.parts != 3 || !pc.shared || seg.rs != 128 || mw.fp8 != nullptr, ++n;
  bad += gx::decode_ws_bytes(L) < (size_t)(128 + 1) * 16 * 512 * 2 + 256, ++n;  // h as decode.cu:33-35, then the counters
  std::printf("CHECK mirror headers %s  %d wrong of %d\n", bad ? "FAIL" : "ok", bad, n);
  return bad != 0;
}
