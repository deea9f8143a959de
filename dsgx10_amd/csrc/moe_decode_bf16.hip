// BF16 experts (the reference's layers 3, 77, 78): instantiations of moe_decode_impl.cuh
#include "moe_decode_impl.cuh"
namespace dsgx {
int launch_decode_bf16(const DecodeArgs& a, int parts, hipStream_t st) { return launch_decode_m<DSGX_FMT_BF16, 0>(a, parts, st); }
}  // namespace dsgx
