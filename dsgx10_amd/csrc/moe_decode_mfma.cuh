// Decode variant 1 (dsgx_decode_cfg::up = 1) for FP8-128x128 layers (with or without the fused FP8 shared expert) and
// INT4-g32 layers (with or without the fused BF16 shared expert): the expert matmuls on v_mfma_f32_16x16x32_bf16.
// The reference's decode kernels are tensor-core kernels too (engine/experts/decode.cu:307-343, 526-587: one MMA tile
// holds up to 16 activation rows); here a tile is 16 WEIGHT rows as the MFMA's A operand and the step's rows (up to 16,
// zero beyond M) as its B operand, so a row count costs nothing extra and no sum crosses lanes.
//   * a unit = 16 weight rows x all of K; K is cut into `ns` slices (mf_slices) and the workgroup's eight waves form
//     8 / ns groups: the waves of a group walk one unit, a slice each, in steps of 128 bytes a row (2 KiB a step: two
//     loads, each eight rows x 128 contiguous bytes; 128 k of FP8, 256 k of INT4, 64 k of BF16), a register ring kMfD
//     steps ahead; the bytes reach the MFMA's lane order (row l % 16, k part l / 16) through 2 KiB of the wave's LDS;
//   * FP8: e4m3 -> bf16 exactly in registers; per 128-k scale block the four MFMAs sum from zero, then
//     acc = fma(S, sum, acc) (the contract of the FP8 paths: decode.cu:269-306);
//   * INT4: a lane reads 16 bytes = the 32 values of one scale group of its row and feeds them to four MFMAs, eight
//     values each (the activation fragment of MFMA j takes the same k: a sum does not mind the order of k inside a
//     step); W = bf16((u - u_z) s) in registers, the decode kernels' routine and bits; the MFMAs accumulate over K;
//   * the slices' sums are added in slice order through LDS (one workgroup barrier a round of units), then the epilogue.
// gate/up: unit = 8 channels, rows interleaved (g0, u0, g1, u1, ...), so that g and u of a channel meet in one lane.
// down: units are (slot, 16 output rows), cut into equal contiguous ranges a workgroup; the complete dots go to memory
// as f32 [slot][M][H] and k_down_combine chains them in slot order (as after k_down_part).
// Every output depends on its own activation row only: a row's bits do not depend on the rows beside it.
#pragma once
#include "moe_decode_impl.cuh"

namespace dsgx {

typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
#ifndef DSGX_MFD
#define DSGX_MFD 4
#endif
constexpr int kMfD = DSGX_MFD;    // ring depth in steps
// Bytes between activation rows in LDS beyond their length, by the routed experts' format: the lanes of one MFMA
// operand read (position l % 16, k part l / 16) 16 bytes each, parts 16 bytes apart (FP8, BF16: rows 64 bytes apart
// mod 256 spread four rows over the banks) or 128 bytes apart (INT4: rows 16 bytes apart spread eight).
__host__ __device__ constexpr int mf_pad(int fmt) { return fmt == DSGX_FMT_INT4_G32 || fmt == DSGX_FMT_MXFP4_G32 ? 16 : 64; }
constexpr int kMfThreads = 512;   // eight waves a workgroup, one workgroup a CU
constexpr int kMfWaves = kMfThreads / 64;

// k a step (128 bytes of a weight row)
template <int FMT> struct MfFmt;
// MINSTEPS: the fewest steps of a K slice (mf_slices), measured: 4 for FP8; 8 for the steps of INT4, which hold four
// times the arithmetic
template <> struct MfFmt<DSGX_FMT_FP8_B128> { static constexpr int STEPK = 128, MINSTEPS = 4; };
template <> struct MfFmt<DSGX_FMT_INT4_G32> { static constexpr int STEPK = 256, MINSTEPS = 8; };
template <> struct MfFmt<DSGX_FMT_BF16> { static constexpr int STEPK = 64, MINSTEPS = 8; };
// MXFP4: INT4's bytes and k map (a lane's 16 bytes are one scale group of 32 values); FP8_B32E: FP8's
template <> struct MfFmt<DSGX_FMT_MXFP4_G32> { static constexpr int STEPK = 256, MINSTEPS = 8; };
template <> struct MfFmt<DSGX_FMT_FP8_B32E> { static constexpr int STEPK = 128, MINSTEPS = 4; };

// The slices of K: a power of two (1 .. 8) that divides the steps of K, `minsteps` steps or more a slice where K allows
// (fewer steps between two workgroup barriers cost more than they spread). With ns < 8 slices, 8 / ns groups of waves
// work on different units at a time.
__host__ __device__ inline int mf_slices(int K, int stepk, int minsteps) {
  const int steps = K / stepk;
  int ns = kMfWaves;
  while (ns > 1 && (steps % ns || steps / ns < minsteps)) ns >>= 1;
  return ns;
}
__host__ __device__ inline size_t mf_rows_bytes(int M, int K, int pad) { return (size_t)M * ((size_t)K * 2 + pad) + 256; }
// + one step's weights a wave + the waves' slice sums of two rounds (the lanes of positions < M only: 4 M x 16 bytes a wave)
__host__ __device__ inline size_t mf_lds_bytes(int M, int K, int pad) { return mf_rows_bytes(M, K, pad) + kMfWaves * 2048 + 2 * kMfWaves * 64 * M; }

// M rows of K bf16 (row m at src + m * ld) to LDS with the padded stride.
// COHERENT: rows written by other workgroups of the same kernel (h after the grid barrier)
template <bool COHERENT>
__device__ __forceinline__ void mf_stage_rows(uint8_t* lds, const uint16_t* src, size_t ld, int M, int K, int pad) {
  const int nq = K / 8, total = M * nq;
  const size_t rs = (size_t)K * 2 + pad;
  for (int i0 = threadIdx.x; i0 < total; i0 += 4 * blockDim.x) {
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = min(i0 + u * (int)blockDim.x, total - 1);
      v[u] = load_chunk<COHERENT>(src + (size_t)(i / nq) * ld + 8 * (i % nq));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * blockDim.x;
      if (i < total) *reinterpret_cast<uint4*>(lds + (size_t)(i / nq) * rs + 16 * (i % nq)) = v[u];
    }
  }
}
// The same from DeepSeek's quantised rows: e4m3 codes q [M][K] with a ue8m0 scale s [M][K / 32] per 32 values, widened
// exactly (code x 2^(scale - 127) is a bf16 value), a thread eight values at a time
__device__ __forceinline__ void mf_stage_rows_q(uint8_t* lds, const uint8_t* q, const uint8_t* s, int M, int K, int pad) {
  const int nq = K / 8, total = M * nq;
  const size_t rs = (size_t)K * 2 + pad;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int m = i / nq, c = i - m * nq;
    const uint2 w = *reinterpret_cast<const uint2*>(q + (size_t)m * K + 8 * c);
    const float sc = __uint_as_float((uint32_t)s[(size_t)m * (K / 32) + c / 4] << 23);
    u32x4_t o;
    o.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.x, sc, false));
    o.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.x, sc, true));
    o.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.y, sc, false));
    o.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.y, sc, true));
    *reinterpret_cast<u32x4_t*>(lds + (size_t)m * rs + 16 * c) = o;
  }
}
// the 256 zero bytes that the lanes of positions beyond the step's rows read (a step's fragments lie within 208 bytes)
__device__ __forceinline__ void mf_zero_bytes(uint8_t* at) {
  if (threadIdx.x < 16) *reinterpret_cast<uint4*>(at + 16 * threadIdx.x) = make_uint4(0, 0, 0, 0);
}

// e2m1 x 8 (one 32-bit word, value i at bits 4 i) times the power of two sc -> exact bf16 values
__device__ __forceinline__ void fp4x8_to_bf16(uint32_t w, float sc, uint32_t (&o)[4]) {
  o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 0));
  o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 1));
  o[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 2));
  o[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 3));
}
// act_quant in place on `rows` staged rows of K bf16 values (row stride rs bytes): per 32 values the ue8m0 scale byte
// e = exponent of max(amax, 1e-4) / 448 rounded up to a power of two (ds41f engine/kernels/common.cuh:53-66), the values
// to e4m3 (round to nearest even) and back: x -> e4m3(x * 2^(127 - e)) * 2^(e - 127), a thread a group
__device__ __forceinline__ void mf_quant_rows(uint8_t* lds, int rows, int K, size_t rs) {
  const int G = K / 32;
  for (int i = threadIdx.x; i < rows * G; i += blockDim.x) {
    uint32_t* p = reinterpret_cast<uint32_t*>(lds + (size_t)(i / G) * rs + (size_t)(i % G) * 64);
    uint32_t v[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u32x4_t q = *reinterpret_cast<const u32x4_t*>(p + 4 * j);
      v[4 * j] = q.x, v[4 * j + 1] = q.y, v[4 * j + 2] = q.z, v[4 * j + 3] = q.w;
    }
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fmaxf(fabsf(bf16_bits_to_f32(v[j] & 0xFFFFu)), fabsf(bf16_bits_to_f32(v[j] >> 16))));
    const uint32_t b = __float_as_uint(__fmul_rn(fmaxf(amax, 1e-4f), 1.0f / 448.0f));
    const uint32_t e = ((b >> 23) & 0xFFu) + ((b & 0x7FFFFFu) != 0 ? 1u : 0u);
    const float inv = __uint_as_float((254u - e) << 23), sc = __uint_as_float(e << 23);
#pragma unroll
    for (int j = 0; j < 16; j += 2) {
      auto qf = [&](uint32_t bits) { return fminf(448.f, fmaxf(-448.f, __fmul_rn(bf16_bits_to_f32(bits), inv))); };
      uint32_t c = __builtin_amdgcn_cvt_pk_fp8_f32(qf(v[j] & 0xFFFFu), qf(v[j] >> 16), 0, false);
      c = __builtin_amdgcn_cvt_pk_fp8_f32(qf(v[j + 1] & 0xFFFFu), qf(v[j + 1] >> 16), c, true);
      v[j] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c, sc, false));
      v[j + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c, sc, true));
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4_t*>(p + 4 * j) = u32x4_t{v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
  }
}

// What a lane needs to walk a unit: set per unit by the caller's `open`. The weight loads are row-major (lane l: rows
// l / 8 and 8 + l / 8 of the unit, piece l % 8 of the step's 128 bytes); scales and zero points are loaded by the lane
// that uses them, in the MFMA's order (unit row l % 16, k part l / 16).
struct MfUnit {
  const uint8_t* wp;  // the lane's 16 bytes of the unit's first step, this wave's K slice
  size_t half;        // bytes from row l / 8 to row 8 + l / 8
  const uint8_t* sp;  // FP8: the first step's f32 scale of the unit's even rows (even lanes) or odd rows (odd lanes);
                      // INT4: the bf16 scales of groups 2 (l / 16), 2 (l / 16) + 1 of the first step, row l % 16
  const uint8_t* zp;  // INT4: the zero-point words of the same two groups (the row's group of 8 rows)
  uint32_t zsh;       // INT4: the row's nibble in those words
};

// The core: `nu` units of `steps` steps each. Wave w works on slice w % ns of the units of group w / ns: in round i the
// groups work on units i ng + group; with ns > 1 a workgroup barrier ends the round and one wave of each group (they
// take turns) adds the slices' sums in slice order. open(u) -> MfUnit (for this wave's slice); done(u, sum) gets the
// unit's complete sums (v4f: rows 4 (l / 16) + q, position l % 16). k0: the first k of this wave's slice. Every wave
// of the workgroup calls this with the same nu, ns, steps. The activation rows of unit u start xoff_of(u) bytes into
// the LDS (units of different slots in one stream); zoff: 256 zero bytes. pre() is called once by every wave, after
// its first kMfD steps' loads are issued and before anything is read from LDS: the caller waits for and stages the
// activations there (a workgroup barrier at its end), with the first weights already on their way.
template <int FMT, int M, class Open, class XOff, class Done, class Pre>
__device__ __forceinline__ void mf_stream(uint8_t* smem, size_t rows_bytes, uint32_t zoff, int pad, int K, int k0, int ns, int nu, int steps, Open&& open,
                                          XOff&& xoff_of, Done&& done, Pre&& pre) {
  constexpr int STEPK = MfFmt<FMT>::STEPK;
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6));
  const int ng = kMfWaves / ns, grp = wave / ns, slice = wave - grp * ns, rounds = (nu + ng - 1) / ng;
  float* red = reinterpret_cast<float*>(smem + rows_bytes + kMfWaves * 2048);
  auto finish = [&](int rnd) {  // after the round's barrier: one wave a group adds the slices' sums in slice order
    const int u = rnd * ng + grp;
    if (u < nu && slice == rnd % ns) {
      v4f_t sum = {0.f, 0.f, 0.f, 0.f};
      const int pos = lane & 15, part4 = lane >> 4;
      if (pos < M)
        for (int w = 0; w < ns; ++w)
          sum += *reinterpret_cast<const v4f_t*>(red + (((size_t)(rnd & 1) * kMfWaves + grp * ns + w) * 4 * M + part4 * M + pos) * 4);
      done(u, sum);
    }
  };
  const int mine = (nu - grp + ng - 1) / ng;  // this wave's units: grp, grp + ng, ...
  if (mine <= 0) {  // (no unit: only the barriers)
    pre();
    if (ns > 1)
      for (int i = 0; i < rounds; ++i) __syncthreads();
    return;
  }
  const int r8 = lane >> 3, q = lane & 7, r16 = lane & 15, part = lane >> 4;
  uint8_t* W = smem + rows_bytes + wave * 2048;  // one step's weights: 16 rows x 128 bytes
  const size_t rs = (size_t)K * 2 + pad;
  // LDS offsets. The row-major writes stay whole 128-byte rows; a row's eight 16-byte pieces are exchanged so that the
  // MFMA-order reads (16 lanes: 16 rows, one k part) touch every bank once: by (row / 2) % 8 for FP8's reads of 8 bytes,
  // by row % 8 for the reads of 16 bytes.
  constexpr bool F8 = FMT == DSGX_FMT_FP8_B128 || FMT == DSGX_FMT_FP8_B32E;   // 8-byte fragment reads, four MFMAs a 128-k step
  constexpr bool G32 = FMT == DSGX_FMT_INT4_G32 || FMT == DSGX_FMT_MXFP4_G32;  // a lane's 16 bytes = one scale group of 32 values
  constexpr int RSH = F8 ? 1 : 0;
  int wr_off[2], rd_off[F8 ? 4 : 2];
#pragma unroll
  for (int h = 0; h < 2; ++h) wr_off[h] = (8 * h + r8) * 128 + ((q ^ (((8 * h + r8) >> RSH) & 7)) * 16);
  if constexpr (F8) {
#pragma unroll
    for (int j = 0; j < 4; ++j) rd_off[j] = r16 * 128 + (((2 * j + (part >> 1)) ^ ((r16 >> 1) & 7)) * 16) + 8 * (part & 1);
  } else if constexpr (G32) {  // pieces 2 part, 2 part + 1: two scale groups
#pragma unroll
    for (int j = 0; j < 2; ++j) rd_off[j] = r16 * 128 + (((2 * part + j) ^ (r16 & 7)) * 16);
  } else {  // pieces part, 4 + part: the lane's 8 k of the step's two MFMAs
#pragma unroll
    for (int j = 0; j < 2; ++j) rd_off[j] = r16 * 128 + (((4 * j + part) ^ (r16 & 7)) * 16);
  }
  const bool live = r16 < M;  // positions beyond the step's rows read the zero bytes
  // the lane's activations: row r16 from k0 + (FP8, BF16: 8 part; INT4: 64 part)
  constexpr int XPART = G32 ? 64 : 8;
  const uint32_t xl = (uint32_t)(r16 * rs) + (uint32_t)(k0 + XPART * part) * 2;
  // xp: the lane's activations of the step at hand (the fragments' offsets within a step are immediates); the lanes of
  // positions beyond the step's rows stay on the zero bytes
  uint32_t xp = live ? xl + xoff_of(grp) : zoff;
  const uint32_t xstep = live ? (uint32_t)STEPK * 2 : 0u;

  struct Entry {
    u32x4_t a, b;  // rows l / 8 and 8 + l / 8
    uint32_t s;    // FP8: the block's scale (even lanes: of the even rows; odd lanes: of the odd rows); INT4: two scales
    u32x2_t z;     // INT4: the two groups' zero-point words
  };
  Entry ring[kMfD];
  int lu = 0, lstep = 0, cu = 0, cstep = 0;
  bool ltail = false;
  MfUnit cur = open(grp);
  v4f_t acc = {0.f, 0.f, 0.f, 0.f};
  auto load = [&](Entry& e) {
    const uint8_t* p = pin_after(cur.wp + (size_t)lstep * 128, acc[0]);
    e.a = ldg_stream(p);
    e.b = ldg_stream(p + cur.half);
    if constexpr (FMT == DSGX_FMT_FP8_B128) {
      e.s = ldg_u32(cur.sp + (size_t)lstep * 4);
    } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
      e.s = ldg_u32(cur.sp + (size_t)lstep * 16);
      e.z = *(const DSGX_GLOBAL u32x2_t*)(uintptr_t)(cur.zp + (size_t)lstep * 32);
    } else if constexpr (FMT == DSGX_FMT_MXFP4_G32) {  // the two groups' ue8m0 bytes (8 groups a row and step)
      e.s = *(const DSGX_GLOBAL uint16_t*)(uintptr_t)(cur.sp + (size_t)lstep * 8);
    } else if constexpr (FMT == DSGX_FMT_FP8_B32E) {   // the step's four k blocks' ue8m0 bytes of the lane's row block
      e.s = ldg_u32(cur.sp + (size_t)lstep * 4);
    }
    if (!ltail && ++lstep == steps) {
      lstep = 0;
      if (lu + 1 < mine) {
        cur = open(++lu * ng + grp);
      } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
        lstep = steps - 1;  // (the INT4 stream waits for the vector unit, not for these loads: whole last steps, measured)
      } else {
        // Past the end the ring keeps loading (unused): every lane the first lane's 16 bytes of the last step, which are
        // still cached - one line a load, and other lines than the other waves'. (Re-reading the last unit from its start
        // fetched it from memory again, 2 KB a step and wave; whole steps of cached lines still cost the L2 their bytes.)
        ltail = true;
        const size_t last = (size_t)(steps - 1);
        cur.wp = uni(cur.wp + last * 128), cur.half = 0;
        if constexpr (FMT == DSGX_FMT_FP8_B128 || FMT == DSGX_FMT_FP8_B32E) cur.sp = uni(cur.sp + last * 4);
        else if constexpr (FMT == DSGX_FMT_MXFP4_G32) cur.sp = uni(cur.sp + last * 8);
      }
    }
  };
  const uint32_t zsh = cur.zsh;  // (the same for every unit of a stream)
  auto mfma = [&](const uint32_t (&o)[4], uint32_t koff, v4f_t c) {  // koff: k within the step
    const u32x4_t av = u32x4_t{o[0], o[1], o[2], o[3]};
    const u32x4_t bv = *reinterpret_cast<const u32x4_t*>(smem + xp + 2 * koff);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, av), __builtin_bit_cast(v8bf_t, bv), c, 0, 0, 0);
  };
  auto compute = [&](const Entry& e) {
    *reinterpret_cast<u32x4_t*>(W + wr_off[0]) = keep_whole(e.a);
    *reinterpret_cast<u32x4_t*>(W + wr_off[1]) = keep_whole(e.b);
    if constexpr (FMT == DSGX_FMT_FP8_B128) {
      v4f_t part_sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint2 wq = *reinterpret_cast<const uint2*>(W + rd_off[j]);
        uint32_t o[4];
        fp8x8_to_bf16(wq.x, wq.y, o);
        part_sum = mfma(o, 32 * j, part_sum);
      }
      // the 128-k block is complete: the scaled add (even rows of the unit: lane 0's scale, odd rows: lane 1's)
      const float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane((int)e.s, 0));
      const float s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane((int)e.s, 1));
      acc[0] = fmaf(s0, part_sum[0], acc[0]), acc[1] = fmaf(s1, part_sum[1], acc[1]);
      acc[2] = fmaf(s0, part_sum[2], acc[2]), acc[3] = fmaf(s1, part_sum[3], acc[3]);
    } else if constexpr (FMT == DSGX_FMT_FP8_B32E) {
      // e4m3 * 2^(scale - 127) is a bf16 value: the scale goes into the conversion and the MFMAs accumulate over K
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint2 wq = *reinterpret_cast<const uint2*>(W + rd_off[j]);
        const float sc = __uint_as_float(((e.s >> (8 * j)) & 0xFFu) << 23);
        uint32_t o[4];
        o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wq.x, sc, false));
        o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wq.x, sc, true));
        o[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wq.y, sc, false));
        o[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wq.y, sc, true));
        acc = mfma(o, 32 * j, acc);
      }
    } else if constexpr (FMT == DSGX_FMT_MXFP4_G32) {
      // e2m1 * 2^(scale - 127) is a bf16 value too: two values an instruction (v_cvt_scalef32_pk_bf16_fp4)
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const u32x4_t pc = *reinterpret_cast<const u32x4_t*>(W + rd_off[jj]);
        const float sc = __uint_as_float(((e.s >> (8 * jj)) & 0xFFu) << 23);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t o[4];
          fp4x8_to_bf16(pc[j], sc, o);
          acc = mfma(o, 32 * jj + 8 * j, acc);
        }
      }
    } else if constexpr (FMT == DSGX_FMT_INT4_G32) {
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const u32x4_t pc = *reinterpret_cast<const u32x4_t*>(W + rd_off[jj]);
        const float s = bf16_bits_to_f32(jj ? e.s >> 16 : e.s & 0xFFFFu);
        const float nzs = -((float)(((jj ? e.z.y : e.z.x) >> zsh) & 15u) * s);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t o[4];
          i4x8_to_bf16(pc[j], s, nzs, o);
          acc = mfma(o, 32 * jj + 8 * j, acc);
        }
      }
    } else {
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const u32x4_t pc = *reinterpret_cast<const u32x4_t*>(W + rd_off[jj]);
        const uint32_t o[4] = {pc[0], pc[1], pc[2], pc[3]};
        acc = mfma(o, 32 * jj, acc);
      }
    }
    xp += xstep;
    if (++cstep < steps) return;
    cstep = 0;
    // the unit is complete in this wave's slice
    if (ns == 1) {
      done(cu * ng + grp, acc);
    } else {
      if (live) *reinterpret_cast<v4f_t*>(red + (((size_t)(cu & 1) * kMfWaves + wave) * 4 * M + part * M + r16) * 4) = acc;
      __syncthreads();
      finish(cu);  // (cu: the round)
    }
    acc = v4f_t{0.f, 0.f, 0.f, 0.f};
    if (++cu < mine && live) xp = xl + xoff_of(cu * ng + grp);
  };
#pragma unroll
  for (int d = 0; d < kMfD; ++d) load(ring[d]);
  pre();
  const int total = mine * steps;
  for (int t = 0; t < total; t += kMfD) {
#pragma unroll
    for (int d = 0; d < kMfD; ++d) {
      if (t + d < total) compute(ring[d]);
      load(ring[d]);
    }
  }
  if (ns > 1 && mine < rounds) __syncthreads();  // (the last round has no unit for this group)
}

// UP: the launch has a gate/up phase: the activation rows are staged with the set-up's other loads, and with a shared
// expert in another format (INT4 or MXFP4 experts) its first tiles - tile g by workgroup g - stream while the routing is
// being resolved (mf_shared_early), when nothing else could.
template <int FMT, int SHFMT, int M, bool UP>
__device__ __forceinline__ void mf_setup(Step<M>& S, const DecodeArgs& a, uint8_t* mf_smem);
// A unit of a gate/up matrix pair in format F: tile t = channels 8 t .. 8 t + 7, unit rows 2 c and 2 c + 1 gate and up of
// channel 8 t + c. (BF16: the shared expert's interleaved matrix, whose rows already come in this order.)
template <int F>
__device__ __forceinline__ MfUnit mf_open_up(const Slot& T, int t, int H, int I, int k0, uint32_t lane) {
  const int r8 = lane >> 3, p8 = lane & 7, r16 = lane & 15, part = lane >> 4;
  const uint8_t* gw = T.g.w;
  const uint8_t* uw = T.u.w;
  const uint8_t* gs = T.g.s;
  const uint8_t* us = T.u.s;
  MfUnit q{};
  if constexpr (F == DSGX_FMT_FP8_B128) {
    q.wp = ((r8 & 1) ? uw : gw) + (size_t)(8 * t + (r8 >> 1)) * H + k0 + p8 * 16;
    q.half = (size_t)4 * H;  // row 8 + r is gate / up (the same parity) of channel 4 further
    q.sp = ((lane & 1) ? us : gs) + ((size_t)((8 * t) >> 7) * (H >> 7) + (k0 >> 7)) * 4;
  } else if constexpr (F == DSGX_FMT_FP8_B32E) {
    q.wp = ((r8 & 1) ? uw : gw) + (size_t)(8 * t + (r8 >> 1)) * H + k0 + p8 * 16;
    q.half = (size_t)4 * H;
    q.sp = ((r16 & 1) ? us : gs) + (size_t)((8 * t) >> 5) * (H >> 5) + (k0 >> 5);  // the lane's own row (MFMA order): gate or up
  } else if constexpr (F == DSGX_FMT_MXFP4_G32) {
    const int G = H >> 5;
    q.wp = ((r8 & 1) ? uw : gw) + (size_t)(8 * t + (r8 >> 1)) * (H >> 1) + (k0 >> 1) + p8 * 16;
    q.half = (size_t)4 * (H >> 1);
    q.sp = ((r16 & 1) ? us : gs) + (size_t)(8 * t + (r16 >> 1)) * G + (size_t)(k0 >> 5) + 2 * part;
  } else if constexpr (F == DSGX_FMT_INT4_G32) {
    const int G = H >> 5;
    q.wp = ((r8 & 1) ? uw : gw) + (size_t)(8 * t + (r8 >> 1)) * (H >> 1) + (k0 >> 1) + p8 * 16;
    q.half = (size_t)4 * (H >> 1);
    const uint8_t* sb = (r16 & 1) ? us : gs;
    const size_t g0 = (size_t)(k0 >> 5) + 2 * part;
    q.sp = sb + ((size_t)(8 * t + (r16 >> 1)) * G + g0) * 2;
    q.zp = sb + al256d((size_t)I * G * 2) + ((size_t)t * G + g0) * 4;
    q.zsh = 4 * (r16 >> 1);
  } else {
    q.wp = gw + ((size_t)(16 * t + r8) * H + k0) * 2 + p8 * 16;
    q.half = (size_t)16 * H;
  }
  return q;
}
// A unit of a down matrix: tile t = output rows 16 t .. 16 t + 15
template <int F>
__device__ __forceinline__ MfUnit mf_open_down(const Slot& T, int t, int H, int I, int k0, uint32_t lane) {
  const int r8 = lane >> 3, p8 = lane & 7, r16 = lane & 15, part = lane >> 4;
  const uint8_t* dw = T.d.w;
  const uint8_t* ds = T.d.s;
  MfUnit q{};
  if constexpr (F == DSGX_FMT_FP8_B128) {
    q.wp = dw + (size_t)(16 * t + r8) * I + k0 + p8 * 16;
    q.half = (size_t)8 * I;
    q.sp = ds + ((size_t)((16 * t) >> 7) * (I >> 7) + (k0 >> 7)) * 4;
  } else if constexpr (F == DSGX_FMT_FP8_B32E) {
    q.wp = dw + (size_t)(16 * t + r8) * I + k0 + p8 * 16;
    q.half = (size_t)8 * I;
    q.sp = ds + (size_t)((16 * t) >> 5) * (I >> 5) + (k0 >> 5);
  } else if constexpr (F == DSGX_FMT_MXFP4_G32) {
    const int G = I >> 5;
    q.wp = dw + (size_t)(16 * t + r8) * (I >> 1) + (k0 >> 1) + p8 * 16;
    q.half = (size_t)8 * (I >> 1);
    q.sp = ds + (size_t)(16 * t + r16) * G + (size_t)(k0 >> 5) + 2 * part;
  } else if constexpr (F == DSGX_FMT_INT4_G32) {
    const int G = I >> 5;
    q.wp = dw + (size_t)(16 * t + r8) * (I >> 1) + (k0 >> 1) + p8 * 16;
    q.half = (size_t)8 * (I >> 1);
    const size_t g0 = (size_t)(k0 >> 5) + 2 * part;
    q.sp = ds + ((size_t)(16 * t + r16) * G + g0) * 2;
    q.zp = ds + al256d((size_t)H * G * 2) + ((size_t)(2 * t + (r16 >> 3)) * G + g0) * 4;
    q.zsh = 4 * (r16 & 7);
  } else {
    q.wp = dw + ((size_t)(16 * t + r8) * I + k0) * 2 + p8 * 16;
    q.half = (size_t)16 * I;
  }
  return q;
}

// The gate/up epilogue of a unit's complete sums (v4f of lane l: gate, up of channel 8 t + 2 (l / 16) and of the next,
// activation row l % 16): SwiGLU and the store of h
template <int SHFMT, int M>
__device__ __forceinline__ void mf_up_store(Step<M>& S, const DecodeArgs& a, int sl, int t, v4f_t sum, uint32_t lane) {
  constexpr int nsh = SHFMT != 0 ? 1 : 0;
  const int I = a.L.I;
  const int pos = lane & 15, part = lane >> 4;
  if (pos >= M) return;
  const Slot& T = S.slots[sl];
  const float sg = T.g.s2, su = T.u.s2;
  uint32_t h0, h1;
  if (a.dsk) {
    // ds41f engine/kernels/moe.cu:519-528: gate and up rounded to bf16, up clamped to +-limit and gate from above,
    // silu(gate) * up, times the row's routing weight (routed slots), rounded to bf16; quantised per 32 when the down
    // phase stages it
    auto hd = [&](float gs, float us) {
      float gt = bf16_round(gs), up = bf16_round(us);
      up = fminf(fmaxf(up, -a.dsk_limit), a.dsk_limit);
      gt = fminf(gt, a.dsk_limit);
      float h = __fmul_rn(__fdiv_rn(gt, __fadd_rn(1.f, expf(-gt))), up);
      if (!T.shared) h = __fmul_rn(S.wslot[sl - nsh][pos], h);
      return f32_to_bf16_bits(h);
    };
    h0 = hd(sum[0], sum[1]), h1 = hd(sum[2], sum[3]);
  } else {
    h0 = swiglu_bits(bf16_round(__fmul_rn(sum[0], sg)), bf16_round(__fmul_rn(sum[1], su)));
    h1 = swiglu_bits(bf16_round(__fmul_rn(sum[2], sg)), bf16_round(__fmul_rn(sum[3], su)));
  }
  uint16_t* dst = a.h + ((size_t)T.hslot * M + pos) * I + 8 * t + 2 * part;
  __hip_atomic_store((DSGX_GLOBAL uint32_t*)(uintptr_t)dst, h0 | (h1 << 16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The shared expert's gate/up tile `blockIdx.x` (if there is one) between the set-up's two barriers, by the waves that do
// not resolve the routing (the first four at most): a wave a K slice at a time, the slices of mf_slices as in the main
// stream, their sums left in LDS; mf_shared_early_finish, after the second barrier, adds them in slice order and stores h:
// the bits of the main stream. No workgroup barrier inside (mf_stream with one slice a unit has none).
#ifndef DSGX_MF_EARLY
#define DSGX_MF_EARLY 1
#endif
__host__ __device__ inline int mf_early_tiles(int I, int G) { return DSGX_MF_EARLY ? (I / 8 < G ? I / 8 : G) : 0; }
template <int FMT, int SHFMT, int M>
__device__ __forceinline__ void mf_shared_early(Step<M>& S, const DecodeArgs& a, uint8_t* mf_smem) {
  constexpr int F = SHFMT, pad = mf_pad(FMT);
  const int H = a.L.H, I = a.L.I, t = blockIdx.x;
  if (t >= mf_early_tiles(I, gridDim.x)) return;
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6));
  const int ns = mf_slices(H, MfFmt<F>::STEPK, MfFmt<F>::MINSTEPS), KS = H / ns, act = ns < 4 ? ns : 4;
  if (wave >= act) return;
  const size_t rows_bytes = mf_rows_bytes(M, H, pad);
  float* red = reinterpret_cast<float*>(mf_smem + rows_bytes + kMfWaves * 2048);
  // mf_stream's unit u of this wave (u = wave, wave + 8, ...) is K slice wave + act (u / 8)
  auto slice_of = [&](int u) { return (u & 7) + act * (u >> 3); };
  auto open = [&](int u) { return mf_open_up<F>(S.slots[0], t, H, I, slice_of(u) * KS, lane); };
  auto xoff = [&](int u) { return (uint32_t)(slice_of(u) * KS * 2); };
  auto fin = [&](int u, v4f_t sum) {
    const int pos = lane & 15, part = lane >> 4;
    if (pos < M) *reinterpret_cast<v4f_t*>(red + ((size_t)slice_of(u) * 4 * M + part * M + pos) * 4) = sum;
  };
  mf_stream<F, M>(mf_smem, rows_bytes, (uint32_t)(M * ((size_t)H * 2 + pad)), pad, H, 0, 1, kMfWaves * (ns / act), KS / MfFmt<F>::STEPK, open, xoff, fin,
                  [] {});
}
template <int FMT, int SHFMT, int M>
__device__ __forceinline__ void mf_shared_early_finish(Step<M>& S, const DecodeArgs& a, uint8_t* mf_smem) {
  constexpr int F = SHFMT, pad = mf_pad(FMT);
  const int H = a.L.H, I = a.L.I, t = blockIdx.x;
  if (t >= mf_early_tiles(I, gridDim.x) || threadIdx.x >= 64) return;
  const uint32_t lane = threadIdx.x;
  const int ns = mf_slices(H, MfFmt<F>::STEPK, MfFmt<F>::MINSTEPS);
  const float* red = reinterpret_cast<const float*>(mf_smem + mf_rows_bytes(M, H, pad) + kMfWaves * 2048);
  const int pos = lane & 15, part = lane >> 4;
  v4f_t sum = {0.f, 0.f, 0.f, 0.f};
  if (pos < M)
    for (int w = 0; w < ns; ++w) sum += *reinterpret_cast<const v4f_t*>(red + ((size_t)w * 4 * M + part * M + pos) * 4);
  mf_up_store<SHFMT, M>(S, a, 0, t, sum, lane);
}
template <int FMT, int SHFMT, int M, bool UP>
__device__ __forceinline__ void mf_setup(Step<M>& S, const DecodeArgs& a, uint8_t* mf_smem) {
  constexpr int NR = resolver_waves<M>();
#ifndef DSGX_MF_EARLY_SAME
#define DSGX_MF_EARLY_SAME 1
#endif
  constexpr bool EARLY = UP && SHFMT != 0 && (SHFMT != FMT || DSGX_MF_EARLY_SAME);
  const int wave = uni((int)(threadIdx.x >> 6)), nw = blockDim.x >> 6;
  ResolveRegs rr;
  if (wave >= nw - NR) resolve_fetch(S, a, wave - (nw - NR), NR, rr);
  prep<FMT, SHFMT, M>(S, a);
  if constexpr (UP) {
    constexpr int pad = mf_pad(FMT);
    const int H = a.L.H;
    if (a.dsk_xq) mf_stage_rows_q(mf_smem, a.dsk_xq, a.dsk_xs, M, H, pad);
    else mf_stage_rows<false>(mf_smem, a.x, H, M, H, pad);
    mf_zero_bytes(mf_smem + (size_t)M * ((size_t)H * 2 + pad));
  }
  __syncthreads();
  if (wave >= nw - NR) resolve<FMT, SHFMT, M>(S, a, wave - (nw - NR), NR, rr);
  else if constexpr (EARLY) mf_shared_early<FMT, SHFMT, M>(S, a, mf_smem);
  __syncthreads();
  if constexpr (EARLY) {
    mf_shared_early_finish<FMT, SHFMT, M>(S, a, mf_smem);
    __syncthreads();  // (the slices' sums are read: the main stream reuses their LDS)
  }
}

// SHFMT: 0 (no fused shared expert), FMT (slot 0 streams with the routed slots) or another format (slot 0 first, in a
// stream of its own)
template <int FMT, int SHFMT, int M>
__device__ __forceinline__ void mf_up_phase(Step<M>& S, const DecodeArgs& a, uint8_t* mf_smem) {
  constexpr int nsh = SHFMT != 0 ? 1 : 0;
  const int H = a.L.H, I = a.L.I;
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6));
  constexpr int pad = mf_pad(FMT);
  // (the activation rows are in LDS: mf_setup)
  // Units are (slot, tile of 8 channels), numbered slot-major; workgroup g of G walks the units g, g + G, g + 2 G, ...
  // (with as many tiles a slot as workgroups that is one tile of every slot; with fewer, a narrow intermediate size, the
  // workgroups still share the slots' tiles evenly)
  const int tiles = I / 8;
  auto done = [&](int sl, int t, v4f_t sum) { mf_up_store<SHFMT, M>(S, a, sl, t, sum, lane); };
  // slots s0 .. s0 + nslots - 1 in format F, from the first slot's tile t0 on, by workgroup g of G
  auto run = [&](auto fmt_tag, int s0, int nslots, int g, int G, int t0) {
    constexpr int F = decltype(fmt_tag)::value;
    const int total = nslots * tiles - t0;
    const int mine = uni(g < total ? (total - g + G - 1) / G : 0);  // this workgroup's units
    if (mine == 0) return;  // (the same for every wave of the workgroup)
    const int ns = mf_slices(H, MfFmt<F>::STEPK, MfFmt<F>::MINSTEPS), KS = H / ns, k0 = (wave % ns) * KS;
    auto open = [&](int u) {
      const int q = t0 + g + u * G, sl = uni(q / tiles);
      return mf_open_up<F>(S.slots[s0 + sl], q - sl * tiles, H, I, k0, lane);
    };
    auto fin = [&](int u, v4f_t sum) {
      const int q = t0 + g + u * G, sl = uni(q / tiles);
      done(s0 + sl, q - sl * tiles, sum);
    };
    mf_stream<F, M>(mf_smem, mf_rows_bytes(M, H, pad), (uint32_t)(M * ((size_t)H * 2 + pad)), pad, H, k0, ns, mine, KS / MfFmt<F>::STEPK, open,
                    [](int) { return 0u; }, fin, [] {});
  };
  const int nrouted = uni(S.n);
  const int G = gridDim.x, g = blockIdx.x;
  if constexpr (SHFMT != 0 && SHFMT != FMT) {
    // The shared slot in its own format: the first workgroups take it, the others the routed slots, both at once, so that a
    // stream that waits for memory (BF16) and one that waits for the vector unit (INT4) share the chip instead of taking
    // turns. The split goes by bytes, a routed byte counted kShCost times (its stream is that much slower a byte).
#ifndef DSGX_MF_SHCOST
#define DSGX_MF_SHCOST 2.0f
#endif
    constexpr float kShCost = FMT == DSGX_FMT_INT4_G32 ? DSGX_MF_SHCOST : 1.f;  // (only the INT4 stream waits for the vector unit)
    auto bpv = [](int f) { return f == DSGX_FMT_BF16 ? 2.f : f == DSGX_FMT_FP8_B128 || f == DSGX_FMT_FP8_B32E ? 1.f : 0.5703f; };  // bytes a value
    // (the shared slot's first tiles were done while the routing was being resolved: mf_shared_early)
    const int t0 = mf_early_tiles(I, G);
    const float bsh = bpv(SHFMT) * (float)(tiles - t0) / (float)tiles, bro = kShCost * (float)nrouted * bpv(FMT);
    const int nshw = uni(t0 == tiles ? 0 : nrouted > 0 ? max(1, min(G - 1, (int)((float)G * bsh / (bsh + bro) + 0.5f))) : G);
    if (g < nshw) run(std::integral_constant<int, SHFMT>{}, 0, 1, g, nshw, t0);
    else if (nrouted > 0) run(std::integral_constant<int, FMT>{}, 1, nrouted, g - nshw, G - nshw, 0);
  } else {
    const int t0 = nsh && DSGX_MF_EARLY_SAME ? mf_early_tiles(I, G) : 0;
    if (nsh + nrouted > 0) run(std::integral_constant<int, FMT>{}, 0, nsh + nrouted, g, G, t0);
  }
  // the wave's h stores are complete before it goes on to the grid barrier (see up_phase)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// The units (slot, tile of 16 output rows) are cut into equal contiguous ranges a workgroup; a shared slot in another
// format counts WSH units a tile (BF16 beside INT4: 3.5 times the bytes, but streamed at the memory's rate where an INT4
// tile waits for the vector unit: twice the time, measured). A workgroup's range is walked in segments of
// up to two slots, a stream each (with no more slots than workgroups, the whole range is one segment): the h rows of
// the segment's slots are staged together and the ring runs on across the slot boundary. FUSED: h was written by this
// launch; the first segment's weights are requested before the grid barrier is waited for.
template <int FMT, int SHFMT, int M, bool FUSED>
__device__ __forceinline__ void mf_down_phase(Step<M>& S, const DecodeArgs& a, uint8_t* mf_smem) {
  constexpr int nsh = SHFMT != 0 ? 1 : 0;
  constexpr bool SH2 = SHFMT != 0 && SHFMT != FMT;
  constexpr int WSH = 2;
  const int H = a.L.H, I = a.L.I;
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6));
  const int nrouted = uni(S.n);
  if (blockIdx.x == 0) {  // the slot table for k_down_combine
    if (threadIdx.x == 0) reinterpret_cast<int*>(a.fac)[0] = nrouted;
    for (int i = threadIdx.x; i < nrouted * M; i += blockDim.x)
      a.fac[8 + (i / M) * 8 + i % M] = __fmul_rn(S.slots[nsh + i / M].d.s2, S.wslot[i / M][i % M]);
  }
  const int tps = H / 16;  // tiles a slot
  const int s0 = SH2 ? 1 : 0, nsl = nsh + nrouted - s0;  // the slots in format FMT
  const long csh = SH2 ? (long)WSH * tps : 0;
  const long total = csh + (long)nsl * tps;
  const long c_lo = total * blockIdx.x / gridDim.x, c_hi = total * (blockIdx.x + 1) / gridDim.x;
  constexpr int pad = mf_pad(FMT);
  const size_t rs = (size_t)I * 2 + pad;
  const size_t rows_bytes = mf_rows_bytes(2 * M, I, pad);
  bool waited = !FUSED;  // the grid barrier is behind this workgroup
  // units [ua, ub) of the slots from sl0 on (unit = slot * tps + tile, slots counted from sl0), all in format F
  auto run = [&](auto fmt_tag, int sl0, int ua, int ub) {
    constexpr int F = decltype(fmt_tag)::value;
    const int nss = (ub - 1) / tps + 1;  // 1 or 2 slots
    auto pre = [&] {
      if (!waited) grid_barrier(a.bar, S.gen, a.spin_limit);
      else __syncthreads();
      waited = true;
      for (int j = 0; j < nss; ++j)
        mf_stage_rows<FUSED>(mf_smem + (size_t)j * M * rs, a.h + (size_t)S.slots[sl0 + j].hslot * M * I, I, M, I, pad);
      mf_zero_bytes(mf_smem + (size_t)2 * M * rs);
      __syncthreads();
      if (a.dsk) {  // w2's input is act_quant(h): e4m3 with a ue8m0 scale per 32 values (moe.cu:529-534), again bf16 values
        mf_quant_rows(mf_smem, nss * M, I, rs);
        __syncthreads();
      }
    };
    const int ns = mf_slices(I, MfFmt<F>::STEPK, MfFmt<F>::MINSTEPS), KS = I / ns, k0 = (wave % ns) * KS;
    auto open = [&](int u) {
      const int j = uni((ua + u) / tps);
      return mf_open_down<F>(S.slots[sl0 + j], ua + u - j * tps, H, I, k0, lane);
    };
    auto xoff = [&](int u) { return (uint32_t)(uni((ua + u) / tps) * M * rs); };
    auto fin = [&](int u, v4f_t sum) {
      const int j = uni((ua + u) / tps), t = ua + u - j * tps, pos = lane & 15, part = lane >> 4;
      if (pos < M) *reinterpret_cast<v4f_t*>(a.dpart + ((size_t)(sl0 + j) * M + pos) * H + 16 * t + 4 * part) = sum;
    };
    mf_stream<F, M>(mf_smem, rows_bytes, (uint32_t)(2 * M * rs), pad, I, k0, ns, ub - ua, KS / MfFmt<F>::STEPK, open, xoff, fin, pre);
  };
  if constexpr (SH2) {  // the shared slot's tiles whose first cost unit lies in this workgroup's range
    const long lo = c_lo < csh ? c_lo : csh, hi = c_hi < csh ? c_hi : csh;
    const int ta = (int)((lo + WSH - 1) / WSH), tb = (int)((hi + WSH - 1) / WSH);
    if (tb > ta) run(std::integral_constant<int, SHFMT>{}, 0, ta, tb);
  }
  const int u_lo = (int)((c_lo > csh ? c_lo : csh) - csh), u_hi = (int)((c_hi > csh ? c_hi : csh) - csh);
  for (int sl = u_lo / tps; sl * tps < u_hi; sl += 2) {  // (the same for every wave of the workgroup)
    const int ua = max(u_lo, sl * tps) - sl * tps, ub = min(u_hi, (sl + 2) * tps) - sl * tps;
    run(std::integral_constant<int, FMT>{}, s0 + sl, ua, ub);
  }
  if (!waited) grid_barrier(a.bar, S.gen, a.spin_limit);  // (a workgroup without a unit)
}

template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(kMfThreads) k_up_mfma(DecodeArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t mf_smem[];  // (read and written 16 bytes at a time)
  __shared__ Step<M> S;
  mf_setup<FMT, SHFMT, M, true>(S, a, mf_smem);
  mf_up_phase<FMT, SHFMT, M>(S, a, mf_smem);
}
template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(kMfThreads) k_down_mfma(DecodeArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t mf_smem[];  // (read and written 16 bytes at a time)
  __shared__ Step<M> S;
  mf_setup<FMT, SHFMT, M, false>(S, a, mf_smem);
  mf_down_phase<FMT, SHFMT, M, false>(S, a, mf_smem);
}
// Both phases in one launch, a grid barrier between them (every workgroup resident: one a CU); the step's set-up runs once
template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(kMfThreads) k_decode_mfma(DecodeArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t mf_smem[];  // (read and written 16 bytes at a time)
  __shared__ Step<M> S;
  if (threadIdx.x == 0) S.gen = grid_barrier_gen(a.bar);
  mf_setup<FMT, SHFMT, M, true>(S, a, mf_smem);
  mf_up_phase<FMT, SHFMT, M>(S, a, mf_smem);
  mf_down_phase<FMT, SHFMT, M, true>(S, a, mf_smem);
}

template <int FMT, int SHFMT, int M>
int launch_decode_mfma(const DecodeArgs& a, int parts, hipStream_t st) {
  const int H = a.L.H, I = a.L.I, cus = num_cus_cached();
  if (H % 256 || I % 256)
    return fail(DSGX_EINVAL, "moe_decode (variant 1): hidden %d, intermediate %d (whole steps of 256 k)", H, I);
  if (parts == 3) {
    auto kern = k_decode_mfma<FMT, SHFMT, M>;
    const size_t lds = std::max(mf_lds_bytes(M, H, mf_pad(FMT)), mf_lds_bytes(2 * M, I, mf_pad(FMT)));
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
    int per_cu = 0;  // the grid barrier needs every workgroup resident
    DSGX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, kMfThreads, lds));
    if (per_cu >= 1) {
      hipLaunchKernelGGL(kern, dim3(cus), dim3(kMfThreads), lds, st, a);
      hipLaunchKernelGGL((k_down_combine<M, SHFMT != 0>), dim3((M * H + 255) / 256), dim3(256), 0, st, a);
      DSGX_HIP(hipGetLastError());
      return DSGX_OK;
    }
  }
  if (parts & 1) {
    auto kern = k_up_mfma<FMT, SHFMT, M>;
    const size_t lds = mf_lds_bytes(M, H, mf_pad(FMT));
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(kMfThreads), lds, st, a);
    DSGX_HIP(hipGetLastError());
  }
  if (parts & 2) {
    auto kern = k_down_mfma<FMT, SHFMT, M>;
    const size_t lds = mf_lds_bytes(2 * M, I, mf_pad(FMT));
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(kMfThreads), lds, st, a);
    hipLaunchKernelGGL((k_down_combine<M, SHFMT != 0>), dim3((M * H + 255) / 256), dim3(256), 0, st, a);
    DSGX_HIP(hipGetLastError());
  }
  return DSGX_OK;
}

template <int FMT, int SHFMT>
int launch_decode_mfma_m(const DecodeArgs& a, int parts, hipStream_t st) {
  switch (a.M) {
    case 1: return launch_decode_mfma<FMT, SHFMT, 1>(a, parts, st);
    case 2: return launch_decode_mfma<FMT, SHFMT, 2>(a, parts, st);
    case 3: return launch_decode_mfma<FMT, SHFMT, 3>(a, parts, st);
    case 4: return launch_decode_mfma<FMT, SHFMT, 4>(a, parts, st);
    case 5: return launch_decode_mfma<FMT, SHFMT, 5>(a, parts, st);
    case 6: return launch_decode_mfma<FMT, SHFMT, 6>(a, parts, st);
    case 7: return launch_decode_mfma<FMT, SHFMT, 7>(a, parts, st);
    case 8: return launch_decode_mfma<FMT, SHFMT, 8>(a, parts, st);
  }
  return fail(DSGX_EUNSUPPORTED, "moe_decode (variant 1): %d rows", a.M);
}

}  // namespace dsgx
