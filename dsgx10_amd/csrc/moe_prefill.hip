// The prefill expert step (gx::moe_prefill of the reference, altar1-4xgx10-switchless/engine/experts/prefill.cu).
#include "abi_internal.h"
#include "common.cuh"

using namespace dsgx;

extern "C" {

void dsgx_prefill_cfg_default(dsgx_prefill_cfg* c) {
  if (!c) return;
  c->shared = 1;
  c->phases = 31;
  c->act_fp8 = 1;
}
size_t dsgx_prefill_ws_bytes(const dsgx_layer_w*, int) { return 0; }
int dsgx_moe_prefill(const dsgx_layer_w*, const uint16_t*, const int*, const float*, int, void*, float*, float*, void*,
                     const dsgx_prefill_cfg*) {
  return fail(DSGX_EUNSUPPORTED, "moe_prefill: not built yet");
}
int dsgx_prefill_view_get(const dsgx_layer_w*, void*, int, dsgx_prefill_view*) {
  return fail(DSGX_EUNSUPPORTED, "prefill_view: not built yet");
}

}  // extern "C"
