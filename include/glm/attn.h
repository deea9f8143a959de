// glm:: - the dense GEMV operators with the reference engine's names and argument order
// (altar1-4xgx10-switchless/engine/attn/attn.h:59-158), forwarding to the C ABI in dsgx.h. Only the weight-streaming
// GEMV, its many-row form gemm() and dequant_int4 are on this build's path; the attention side of attn.h is not mirrored.
#pragma once
#include <cstddef>
#include <cstdint>

#include "../gx/check.h"

namespace glm {

inline constexpr int kMaxRows = DSGX_MAX_ROWS, kMaxSegs = 4;

// attn.h:80-92. kINT4 / kFP8 / kBF16 here mean the checkpoint's row-major tensors (dsgx.h), not the reference's tiles.
enum class WFmt : int { kNone = 0, kBF16 = 1, kINT4 = 2, kFP8 = 3, kBF16T = 4 };
enum class GemvOut : int { kBF16 = DSGX_OUT_BF16, kF32 = DSGX_OUT_F32, kSwiGLU = DSGX_OUT_SWIGLU };

struct GemvSeg {
  WFmt fmt = WFmt::kNone;
  const void* w = nullptr;   // bf16 rows, INT4 weight_packed, or e4m3 codes
  const float* s = nullptr;  // FP8 scales (attn.h:96-98)
  int n = 0;
  int rs = 128, ks = 128;
  void* y = nullptr;
  int ldy = 0;
  int group_rows = 0, x_group = 0;  // grouped input: not built, must be 0
  // INT4 on this build: the checkpoint's two other tensors
  const void* s16 = nullptr;  // weight_scale bf16 [N][K/32]
  const void* zp = nullptr;   // weight_zero_point u32 [N/8][K/32]
};

inline void gemv(const uint16_t* x, int ldx, int rows, int K, const GemvSeg* segs, int nseg, GemvOut out, int splitk, void* st,
                 bool pdl = false, const void* iw = nullptr) {
  (void)pdl;
  if (iw) die("gemv: the index weights are not part of this build");
  if (nseg < 1 || nseg > kMaxSegs) die("gemv: K %d, %d segments", K, nseg);
  dsgx_gemv_seg g[kMaxSegs];
  for (int i = 0; i < nseg; ++i) {
    const GemvSeg& a = segs[i];
    if (a.group_rows || a.x_group) die("gemv: grouped inputs are not built");
    if (a.fmt == WFmt::kBF16T) die("gemv: kBF16T names a GB10 lane order; use kBF16");
    g[i].fmt = a.fmt == WFmt::kBF16 ? DSGX_FMT_BF16 : a.fmt == WFmt::kINT4 ? DSGX_FMT_INT4_G32 : a.fmt == WFmt::kFP8 ? DSGX_FMT_FP8_B128 : 0;
    g[i].w = a.w;
    g[i].s = a.fmt == WFmt::kINT4 ? a.s16 : static_cast<const void*>(a.s);
    g[i].zp = a.zp, g[i].n = a.n, g[i].rs = a.rs, g[i].ks = a.ks, g[i].y = a.y, g[i].ldy = a.ldy;
  }
  DSGX_DIE_ON(dsgx_gemv(x, ldx, rows, K, g, nseg, (int)out, splitk, st));
}
// attn.h:141-157: the GEMM for prefill chunks (any number of rows), "every output equals gemv()'s at the same splitk bit
// for bit". Here that holds by construction: the rows go through gemv() sixteen at a time (the weights are read once a
// group of sixteen rows; a tiled MFMA GEMM for long chunks is the FP8 / INT4 prefill path of gx::moe_prefill, not this).
// scratch (the reference's INT4 staging buffer) is not needed and ignored.
inline void gemm(const uint16_t* x, int ldx, int rows, int K, const GemvSeg* segs, int nseg, GemvOut out, int splitk, void* st,
                 bool pdl = false, uint16_t* scratch = nullptr, size_t scratch_elems = 0) {
  (void)scratch, (void)scratch_elems;
  if (nseg < 1 || nseg > kMaxSegs) die("gemm: K %d, %d segments", K, nseg);
  const size_t esz = out == GemvOut::kF32 ? 4 : 2;
  for (int r0 = 0; r0 < rows; r0 += kMaxRows) {
    GemvSeg g[kMaxSegs];
    for (int i = 0; i < nseg; ++i) {
      g[i] = segs[i];
      g[i].y = static_cast<uint8_t*>(segs[i].y) + (size_t)r0 * segs[i].ldy * esz;
    }
    gemv(x + (size_t)r0 * ldx, ldx, rows - r0 < kMaxRows ? rows - r0 : kMaxRows, K, g, nseg, out, splitk, st, pdl);
  }
}
// attn.h:150-152: BF16 weights only (the router, the head): every segment taken as BF16 (kNone allowed)
inline void gemm_bf16(const uint16_t* x, int ldx, int rows, int K, const GemvSeg* segs, int nseg, GemvOut out, int splitk, void* st,
                      bool pdl = false) {
  if (nseg < 1 || nseg > kMaxSegs) die("gemm_bf16: K %d, %d segments", K, nseg);
  GemvSeg g[kMaxSegs];
  for (int i = 0; i < nseg; ++i) {
    g[i] = segs[i];
    if (g[i].fmt != WFmt::kNone && g[i].fmt != WFmt::kBF16) die("gemm_bf16: segment %d is not BF16", i);
    g[i].fmt = WFmt::kBF16;
  }
  gemm(x, ldx, rows, K, g, nseg, out, splitk, st, pdl);
}
// attn.h:154-158 (row-major output only; the tiled form is a GB10 layout)
inline void dequant_int4(const void* packed, const void* scale, const void* zp, int N, int K, uint16_t* out, size_t ld, void* st,
                         bool pdl = false, bool tiled = false) {
  (void)pdl;
  if (tiled) die("dequant_int4: the tiled output is a GB10 layout and is not built");
  DSGX_DIE_ON(dsgx_dequant_int4(packed, scale, zp, N, K, out, ld, st));
}

}  // namespace glm
