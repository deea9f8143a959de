// The streaming inner loop shared by the dense GEMV and the decode MoE kernels.
//
// A wavefront owns whole output rows. Per "step" it reads one segment of RB rows: every lane one 16-byte load a row
// (1 KiB a row and wave instruction, K-contiguous), which is KL = 16 (FP8), 32 (INT4) or 8 (BF16) consecutive k of the
// row; the lane decodes them in registers to packed bf16 pairs and accumulates dot products against the M activation
// rows, whose matching chunks it reads from LDS (staged once per workgroup in a conflict-free order, common.cuh).
// K is therefore split over the 64 lanes; after the last segment the lanes' partial sums are added with cross-lane
// shuffles (DPP). Steps are software-pipelined: the loads of step t + D are issued before step t is computed.
#pragma once
#include "common.cuh"

namespace dsgx {

struct Raw {
  uint4 v;       // 16 bytes of the row
  uint32_t aux;  // FP8: the lane's block scale (f32 bits); INT4: bf16 scale bits | zero-point nibble << 16
};

// One matrix on the device in a pool format (include/dsgx.h).
struct MatDev {
  const uint8_t* w;   // FP8 codes / INT4 weight_packed / bf16 rows
  const uint8_t* s;   // FP8: f32 scales; INT4: bf16 scales
  const uint8_t* zp;  // INT4: weight_zero_point
  int lrs, lks;       // FP8: log2 of the scale block (rows, k)
  int srow;           // FP8: scale row stride in floats, K >> lks
  float s2;
};

template <int FMT> struct FmtT;
template <> struct FmtT<DSGX_FMT_FP8_B128> {
  static constexpr int KL = 16, XC = 2, SEGK = 1024;
  __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)K; }
};
template <> struct FmtT<DSGX_FMT_INT4_G32> {
  static constexpr int KL = 32, XC = 4, SEGK = 2048;
  __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)K / 2; }
};
template <> struct FmtT<DSGX_FMT_BF16> {
  static constexpr int KL = 8, XC = 1, SEGK = 512;
  __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)K * 2; }
};

// the lane's 16 bytes of (row n, segment seg) and what it needs to decode them
template <int FMT>
__device__ __forceinline__ void load_raw(Raw& r, const MatDev& m, int n, int seg, int lane, int K) {
  using F = FmtT<FMT>;
  const int k0 = seg * F::SEGK + lane * F::KL;
  r.v = make_uint4(0, 0, 0, 0);
  r.aux = 0;
  if (k0 >= K) return;  // the partial last segment: zeros (INT4: scale +0, so every value decodes to 0)
  r.v = ldg_stream(m.w + (size_t)n * F::row_bytes(K) + (size_t)seg * 1024 + lane * 16);
  if constexpr (FMT == DSGX_FMT_FP8_B128) {
    r.aux = reinterpret_cast<const uint32_t*>(m.s)[(size_t)(n >> m.lrs) * m.srow + (k0 >> m.lks)];
  } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
    const int g = k0 >> 5, G = K >> 5;
    const uint32_t sb = reinterpret_cast<const uint16_t*>(m.s)[(size_t)n * G + g];
    const uint32_t zw = reinterpret_cast<const uint32_t*>(m.zp)[(size_t)(n >> 3) * G + g];
    r.aux = sb | (((zw >> (4 * (n & 7))) & 15u) << 16);
  }
}

// RB rows of one segment against M activation rows. xs: the workgroup's staged activations, row m at xs + m * nq
// (nq chunks a row); acc[r][m] are the lanes' running sums.
template <int FMT, int M, int RB>
__device__ __forceinline__ void step_dot(const Raw (&raw)[RB], const uint4* __restrict__ xs, int nq, int seg, int lane,
                                         float (&acc)[RB][M]) {
  using F = FmtT<FMT>;
  const uint4* xl = xs + (size_t)seg * F::XC * 64 + lane;
  if constexpr (FMT == DSGX_FMT_FP8_B128) {
    // per (row, 128-k block): the unscaled sum from zero, then acc = fma(S, sum, acc); a lane's 16 k lie in one block
    float p[RB][M];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) p[r][m] = 0.f;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      uint4 xf[M];
#pragma unroll
      for (int m = 0; m < M; ++m) xf[m] = xl[(size_t)m * nq + c * 64];
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        uint32_t o[4];
        fp8x8_to_bf16(c ? raw[r].v.z : raw[r].v.x, c ? raw[r].v.w : raw[r].v.y, o);
#pragma unroll
        for (int m = 0; m < M; ++m) {
          float t = p[r][m];
          t = dot2(o[0], xf[m].x, t);
          t = dot2(o[1], xf[m].y, t);
          t = dot2(o[2], xf[m].z, t);
          t = dot2(o[3], xf[m].w, t);
          p[r][m] = t;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const float s = __uint_as_float(raw[r].aux);
#pragma unroll
      for (int m = 0; m < M; ++m) acc[r][m] = fmaf(s, p[r][m], acc[r][m]);
    }
  } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
    float s[RB], nzs[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      s[r] = bf16_bits_to_f32(raw[r].aux & 0xFFFFu);
      nzs[r] = -((float)(raw[r].aux >> 16) * s[r]);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint4 xf[M];
#pragma unroll
      for (int m = 0; m < M; ++m) xf[m] = xl[(size_t)m * nq + c * 64];
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const uint32_t w = c == 0 ? raw[r].v.x : c == 1 ? raw[r].v.y : c == 2 ? raw[r].v.z : raw[r].v.w;
        uint32_t o[4];
        i4x8_to_bf16(w, s[r], nzs[r], o);
#pragma unroll
        for (int m = 0; m < M; ++m) {
          float t = acc[r][m];
          t = dot2(o[0], xf[m].x, t);
          t = dot2(o[1], xf[m].y, t);
          t = dot2(o[2], xf[m].z, t);
          t = dot2(o[3], xf[m].w, t);
          acc[r][m] = t;
        }
      }
    }
  } else {
    uint4 xf[M];
#pragma unroll
    for (int m = 0; m < M; ++m) xf[m] = xl[(size_t)m * nq];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float t = acc[r][m];
        t = dot2(raw[r].v.x, xf[m].x, t);
        t = dot2(raw[r].v.y, xf[m].y, t);
        t = dot2(raw[r].v.z, xf[m].z, t);
        t = dot2(raw[r].v.w, xf[m].w, t);
        acc[r][m] = t;
      }
  }
}

// number of segments of a K in a format, and K rounded up to whole segments
template <int FMT> __host__ __device__ inline int num_segs(int K) { return (K + FmtT<FMT>::SEGK - 1) / FmtT<FMT>::SEGK; }

}  // namespace dsgx
