// INT4-g32 experts, decode variant 1 (the expert matmuls on the bf16 MFMA): instantiations of moe_decode_mfma.cuh
// shared: 0 none, DSGX_FMT_BF16 (altar-1's shared expert) or DSGX_FMT_FP8_B128 (GLM-5.3's fused FP8 shared expert,
// engine/experts/experts.h:66-87 of the reference)
#include "moe_decode_mfma.cuh"
namespace dsgx {
int launch_decode_int4_mfma(const DecodeArgs& a, int parts, int shared, hipStream_t st) {
  if (shared == DSGX_FMT_BF16) return launch_decode_mfma_m<DSGX_FMT_INT4_G32, DSGX_FMT_BF16>(a, parts, st);
  if (shared == DSGX_FMT_FP8_B128) return launch_decode_mfma_m<DSGX_FMT_INT4_G32, DSGX_FMT_FP8_B128>(a, parts, st);
  return launch_decode_mfma_m<DSGX_FMT_INT4_G32, 0>(a, parts, st);
}
}  // namespace dsgx
