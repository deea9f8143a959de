// INT4-g32 experts (with or without the fused BF16 shared expert): instantiations of moe_decode_impl.cuh
#include "moe_decode_impl.cuh"
namespace dsgx {
int launch_decode_int4(const DecodeArgs& a, int parts, bool shared_bf16, hipStream_t st) {
  return shared_bf16 ? launch_decode_m<DSGX_FMT_INT4_G32, DSGX_FMT_BF16>(a, parts, st) : launch_decode_m<DSGX_FMT_INT4_G32, 0>(a, parts, st);
}
}  // namespace dsgx
