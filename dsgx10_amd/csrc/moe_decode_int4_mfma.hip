// INT4-g32 experts, decode variant 1 (the expert matmuls on the bf16 MFMA): instantiations of moe_decode_mfma.cuh
#include "moe_decode_mfma.cuh"
namespace dsgx {
int launch_decode_int4_mfma(const DecodeArgs& a, int parts, bool shared_bf16, hipStream_t st) {
  return shared_bf16 ? launch_decode_mfma_m<DSGX_FMT_INT4_G32, DSGX_FMT_BF16>(a, parts, st) : launch_decode_mfma_m<DSGX_FMT_INT4_G32, 0>(a, parts, st);
}
}  // namespace dsgx
