// FP8-128x128 experts (with or without the fused FP8 shared expert): instantiations of moe_decode_impl.cuh
#include "moe_decode_impl.cuh"
#include "moe_decode_mfma.cuh"
namespace dsgx {
int launch_decode_fp8(const DecodeArgs& a, int parts, bool shared, hipStream_t st) {
  return shared ? launch_decode_m<DSGX_FMT_FP8_B128, DSGX_FMT_FP8_B128>(a, parts, st) : launch_decode_m<DSGX_FMT_FP8_B128, 0>(a, parts, st);
}
int launch_decode_fp8_mfma(const DecodeArgs& a, int parts, bool shared, hipStream_t st) {
  return shared ? launch_decode_mfma_m<DSGX_FMT_FP8_B128, DSGX_FMT_FP8_B128>(a, parts, st) : launch_decode_mfma_m<DSGX_FMT_FP8_B128, 0>(a, parts, st);
}
}  // namespace dsgx
