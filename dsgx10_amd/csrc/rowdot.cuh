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
  u32x4_t v;     // 16 bytes of the row
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

// The lane's 16 bytes of (row n, segment seg) and what it needs to decode them. The loads are unconditional: a lane
// past the end of K (TAIL: the dense GEMV's partial last segment) reads the row's first bytes instead and step_dot
// drops them; with `dummy` set (the pipeline's loads past the wave's last step) every lane reads there instead.
// `pin`: a value of the preceding compute, see pin_after().
template <int FMT, bool TAIL>
__device__ __forceinline__ void load_raw(Raw& r, const MatDev& m, int n, int seg, int lane, int K, float pin, const uint8_t* dummy) {
  using F = FmtT<FMT>;
  int k0 = seg * F::SEGK + lane * F::KL;
  if (TAIL && k0 >= K) k0 = 0;
  const uint8_t* wp = m.w + (size_t)n * F::row_bytes(K) + F::row_bytes(k0);
  const uint8_t* ap = nullptr;
  if constexpr (FMT == DSGX_FMT_FP8_B128) ap = m.s + ((size_t)(n >> m.lrs) * m.srow + (k0 >> m.lks)) * 4;
  if (dummy) wp = ap = dummy;  // (every lane the same 16 bytes: one cache line a load)
  r.v = ldg_stream(pin_after(wp, pin));
  if constexpr (FMT == DSGX_FMT_FP8_B128) {
    r.aux = ldg_u32(ap);
  } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
    const int g = k0 >> 5, G = K >> 5;
    const uint8_t* sp = m.s + ((size_t)n * G + g) * 2;
    const uint8_t* zp = m.zp + ((size_t)(n >> 3) * G + g) * 4;
    if (dummy) sp = zp = dummy;
    r.aux = ldg_u16(sp) | (((ldg_u32(zp) >> (4 * (n & 7))) & 15u) << 16);
  } else {
    r.aux = 0;
  }
}

// The same loads with the wave-uniform part of the addresses kept apart: a RowSrc is one weight row's bases, set up
// once a row on the scalar unit; load_row() then issues the step's loads as scalar base + lane offset.
struct RowSrc {
  const uint8_t* w;  // the row's first byte
  const uint8_t* a;  // FP8: the row's scale row; INT4: the row's scales
  const uint8_t* z;  // INT4: the zero-point words of the row's group of 8 rows
  uint32_t zsh;      // INT4: the row's nibble in those words
};
// m, n, K wave-uniform
template <int FMT>
__device__ __forceinline__ RowSrc row_src(const MatDev& m, int n, int K) {
  using F = FmtT<FMT>;
  RowSrc r;
  r.w = m.w + (size_t)n * F::row_bytes(K);
  r.a = r.z = nullptr, r.zsh = 0;
  if constexpr (FMT == DSGX_FMT_FP8_B128) {
    r.a = m.s + (size_t)(n >> m.lrs) * m.srow * 4;
  } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
    const int G = K >> 5;
    r.a = m.s + (size_t)n * G * 2;
    r.z = m.zp + (size_t)(n >> 3) * G * 4;
    r.zsh = 4 * (n & 7);
  }
  return r;
}
// seg wave-uniform; lks: log2 of the FP8 scale block along k (wave-uniform). No tail handling: K is whole segments.
template <int FMT>
__device__ __forceinline__ void load_row(Raw& r, const RowSrc& s, int seg, uint32_t lane, int lks, float pin) {
  r.v = ldg_stream(s.w + seg * 1024, pin_after(lane * 16u, pin));
  if constexpr (FMT == DSGX_FMT_FP8_B128) {
    r.aux = ldg_u32(s.a + (size_t)(seg * FmtT<FMT>::SEGK >> lks) * 4, ((lane * 16u) >> lks) * 4u);
  } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
    r.aux = ldg_u16(s.a + seg * 128, lane * 2u) | (((ldg_u32(s.z + seg * 256, lane * 4u) >> s.zsh) & 15u) << 16);
  } else {
    r.aux = 0;
  }
}

// RB rows of one segment against M activation rows. xs: the workgroup's staged activations, row m at xs + m * nq
// (nq chunks a row); acc[r][m] are the lanes' running sums.
template <int FMT, int M, int RB, bool TAIL = false>
__device__ __forceinline__ void step_dot(const Raw (&raw_in)[RB], const uint4* __restrict__ xs, int nq, int seg, int lane,
                                         float (&acc)[RB][M], int K = 0) {
  using F = FmtT<FMT>;
  const uint4* xl = xs + (size_t)seg * F::XC * 64 + lane;
  Raw raw[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    raw[r].v = keep_whole(raw_in[r].v);
    raw[r].aux = raw_in[r].aux;
    if (TAIL && seg * F::SEGK + lane * F::KL >= K) raw[r].v = u32x4_t{0, 0, 0, 0}, raw[r].aux = 0;  // INT4: scale +0
  }
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
