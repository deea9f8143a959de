// The residual add and RMSNorm of one row by a workgroup of 256 threads: the local half of the reference's
// comm::glm::allreduce_add_norm / allreduce2_add_norm (altar1-4xgx10-switchless/engine/comm/glmcoll.h:34-62) at one rank,
// the norm as engine/attn/prep.cu:12-66 (k_rmsnorm):
//   sum        = part                                   (one partial: the reference's decision 8, yr already holds yr + ys)
//              | bf16(bf16(part) + bf16(part2))         (two partials: the old combine, experts.h finalize)
//   h          = bf16(f32(res) + sum)                   (the contract: the f32 sum rounded once, with the residual)
//              | bf16(f32(res) + bf16(sum))             (round2: the sum rounded first)
//   xn         = bf16(w * bf16(h * rstd)),  rstd = 1 / sqrt(mean(h^2) + eps), IEEE division and square root
// mean(h^2) in f32 in a fixed order: a thread's H / 256 contiguous values in order, the wave by a butterfly, the waves in
// order (the reference fixes an order too, its own: the statistics' order is not part of the contract).
// Used by k_add_norm (a launch of its own) and as the prologue of the dense GEMV kernels (the normed rows go straight
// into the GEMV's staged activations): one code, so both give the same bits.
#pragma once
#include "common.cuh"

namespace dsgx {

struct NormIn {
  const float* part;   // f32 [M][H]; null: no add + norm (the GEMV reads x)
  const float* part2;
  const uint16_t* res;
  uint16_t* res_out;   // may be null
  const uint16_t* w;
  uint16_t* xn;        // may be null
  float eps;
  int round2;
};

// red: 4 floats of LDS. put_h(q, chunk) / put_xn(q, chunk): chunk q of the row (8 values, k = 8 q ...) as packed bf16;
// either may do nothing. All 256 threads call it; it contains workgroup barriers.
template <class PutH, class PutXn>
__device__ __forceinline__ void add_norm_row(const NormIn& a, int row, int H, float* red, bool want_xn, PutH&& put_h, PutXn&& put_xn) {
  const int tid = threadIdx.x, per = H / 256;  // (per a multiple of 8, at most 64: the host checks)
  const size_t base = (size_t)row * H + (size_t)tid * per;
  float hv[64];
  float ss = 0.f;
  // the norm's weights are fetched with the row's other inputs: one memory round trip for the call, not two
  u32x4_t wq[8];
#pragma unroll
  for (int i = 0; i < 64; i += 8)
    if (want_xn && i < per) wq[i >> 3] = *reinterpret_cast<const DSGX_GLOBAL u32x4_t*>((uintptr_t)(a.w + (size_t)tid * per + i));
#pragma unroll
  for (int i = 0; i < 64; i += 8) {
    if (i >= per) break;
    const u32x4_t rq = *reinterpret_cast<const DSGX_GLOBAL u32x4_t*>((uintptr_t)(a.res + base + i));
    uint32_t ho[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float r = bf16_bits_to_f32(j & 1 ? rq[j >> 1] >> 16 : rq[j >> 1] & 0xFFFFu);
      float s = a.part[base + i + j];
      if (a.part2) s = __fadd_rn(bf16_round(s), bf16_round(a.part2[base + i + j])), s = bf16_round(s);
      else if (a.round2) s = bf16_round(s);
      const uint32_t hb = f32_to_bf16_bits(__fadd_rn(r, s));
      const float h = bf16_bits_to_f32(hb);
      hv[i + j] = h;
      ss = __fadd_rn(ss, __fmul_rn(h, h));
      if (j & 1) ho[j >> 1] |= hb << 16;
      else ho[j >> 1] = hb;
    }
    put_h((tid * per + i) >> 3, u32x4_t{ho[0], ho[1], ho[2], ho[3]});
  }
  if (!want_xn) return;
  ss = wave_sum(ss);
  __syncthreads();  // (red may still be read for the row before)
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  const float tot = __fadd_rn(__fadd_rn(__fadd_rn(red[0], red[1]), red[2]), red[3]);
  const float rstd = __fdiv_rn(1.f, sqrtf(__fadd_rn(__fdiv_rn(tot, (float)H), a.eps)));  // (sqrtf: the correctly rounded root)
#pragma unroll
  for (int i = 0; i < 64; i += 8) {
    if (i >= per) break;
    const u32x4_t wv4 = wq[i >> 3];
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float wv = bf16_bits_to_f32(j & 1 ? wv4[j >> 1] >> 16 : wv4[j >> 1] & 0xFFFFu);
      const uint32_t b = f32_to_bf16_bits(__fmul_rn(wv, bf16_round(__fmul_rn(hv[i + j], rstd))));
      if (j & 1) o[j >> 1] |= b << 16;
      else o[j >> 1] = b;
    }
    put_xn((tid * per + i) >> 3, u32x4_t{o[0], o[1], o[2], o[3]});
  }
}

}  // namespace dsgx
