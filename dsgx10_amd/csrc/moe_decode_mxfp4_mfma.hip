// MXFP4-g32 experts (DeepSeek's layers: ds41f-4xgx10-switchless/engine/kernels/dsk.h:199-241 of the reference) with or
// without the fused FP8 shared expert whose scales are ue8m0 bytes per 32 x 32 block: instantiations of moe_decode_mfma.cuh.
// Both formats' values times their power-of-two scales are bf16 values, and so are the e4m3 activations times theirs: the
// block-scaled products of the reference's MMA are exact bf16 x bf16 products here, summed in f32 by the bf16 MFMA.
#include "moe_decode_mfma.cuh"
namespace dsgx {
int launch_decode_mxfp4_mfma(const DecodeArgs& a, int parts, bool shared_fp8e, hipStream_t st) {
  if (shared_fp8e) return launch_decode_mfma_m<DSGX_FMT_MXFP4_G32, DSGX_FMT_FP8_B32E>(a, parts, st);
  return launch_decode_mfma_m<DSGX_FMT_MXFP4_G32, 0>(a, parts, st);
}
}  // namespace dsgx
