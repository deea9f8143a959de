// Device helpers shared by the gfx950 kernels: bf16 / e4m3 / INT4 decode in registers, wave64 reductions, the
// streaming loads, the activation staging layout and the router's row function.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dsgx.h"

namespace dsgx {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// ---- scalar codecs ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
// Round to nearest even, the contract's integer form (engine/experts/formats.cuh:33-37 of the reference): used where
// a single value is rounded (epilogues); the packed hardware conversion below is used in the streaming loops.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ float bf16_round(float f) { return __uint_as_float(f32_to_bf16_bits(f) << 16); }
// two f32 -> packed bf16 (lo = a, hi = b), round to nearest even: v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2_t v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}
// acc + a.lo * b.lo + a.hi * b.hi on packed bf16 pairs: v_dot2c_f32_bf16
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc, false);
}

// ---- weight decode: 8 consecutive k -> four packed bf16 pairs (k, k+1) ---------------------------------------------------
// FP8 e4m3fn: two 32-bit words (8 codes) -> exact bf16 values (v_cvt_scalef32_pk_bf16_fp8 with scale 1).
__device__ __forceinline__ void fp8x8_to_bf16(uint32_t w0, uint32_t w1, uint32_t (&o)[4]) {
  o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w0, 1.0f, false));
  o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w0, 1.0f, true));
  o[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w1, 1.0f, false));
  o[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w1, 1.0f, true));
}
// INT4-g32: one 32-bit word = 8 stored nibbles u (value i at bits 4i) of one group with scale s (f32 of the bf16) and
// nzs = -(u_z * s). W = bf16_rne((u - u_z) * s): u * s and u_z * s are exact in f32 (4 x 8 significant bits), so
// fma(u, s, nzs) is the exact product (u - u_z) * s, and the packed conversion rounds it once to nearest even.
// (Exact while u_z * s stays finite, i.e. |s| < 2^124; dequant_int4's own kernel uses the subtract-first form.)
// byte k of a word as a float, in one instruction (written as shifts and masks the compiler turns the masked nibbles
// back into a bit-field extract followed by a conversion: two instructions a value)
template <int K>
__device__ __forceinline__ float ubyte_to_f32(uint32_t w) {
  float f;
  if (K == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(w));
  else if (K == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(w));
  else if (K == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(w));
  else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(w));
  return f;
}
__device__ __forceinline__ void i4x8_to_bf16(uint32_t w, float s, float nzs, uint32_t (&o)[4]) {
  const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;  // lo: values 0,2,4,6; hi: 1,3,5,7
  o[0] = pack_bf16(fmaf(ubyte_to_f32<0>(lo), s, nzs), fmaf(ubyte_to_f32<0>(hi), s, nzs));
  o[1] = pack_bf16(fmaf(ubyte_to_f32<1>(lo), s, nzs), fmaf(ubyte_to_f32<1>(hi), s, nzs));
  o[2] = pack_bf16(fmaf(ubyte_to_f32<2>(lo), s, nzs), fmaf(ubyte_to_f32<2>(hi), s, nzs));
  o[3] = pack_bf16(fmaf(ubyte_to_f32<3>(lo), s, nzs), fmaf(ubyte_to_f32<3>(hi), s, nzs));
}
// the contract in its subtract-first form, exact for every finite scale: bf16_rne(float(u - u_z) * s)
__device__ __forceinline__ uint32_t i4_value_bits(int u, int uz, uint32_t sbits) {
  return f32_to_bf16_bits((float)(u - uz) * bf16_bits_to_f32(sbits));
}

// ---- streaming loads (weights are read once: non-temporal) ---------------------------------------------------------------
// Pointers that come out of LDS tables (the slot descriptors) have lost their address space: the loads below cast
// them back to the global address space, so that they are global_load (vmcnt only) and not flat_load instructions.
#define DSGX_GLOBAL __attribute__((address_space(1)))
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4_t ldg_stream(const void* p) {
  return __builtin_nontemporal_load((const DSGX_GLOBAL u32x4_t*)(uintptr_t)p);
}
// The software pipelines below keep D steps of loads in flight in a ring of registers: step t is computed, then the
// load of step t + D is issued into the same registers. Two empty asm statements keep the compiler from undoing that:
// pin_after() makes a load's address depend on a value the preceding compute produced, so the load is not hoisted
// above the compute (which would need a second set of registers and copies that wait for the new data); keep_whole()
// passes a loaded 16-byte value through as one register tuple, so the loop-carried value is not split into scalars
// that no longer line up with the load's destination.
__device__ __forceinline__ const uint8_t* pin_after(const uint8_t* p, float dep) {
  uint64_t a = (uint64_t)p;
  asm volatile("" : "+v"(a) : "v"(dep));
  return (const uint8_t*)a;
}
__device__ __forceinline__ u32x4_t keep_whole(u32x4_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
// Wave-uniform values. The compiler cannot know that a value read from LDS or derived from the wave's index is the
// same in every lane; uni() says so (v_readfirstlane), which moves the value and all arithmetic on it (row bases,
// cursors, loop bounds, branches) to the scalar unit and lets loads use the "scalar base + lane offset" addressing.
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint32_t uni(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ float uni(float v) { return __uint_as_float(uni(__float_as_uint(v))); }
__device__ __forceinline__ const uint8_t* uni(const uint8_t* p) {
  const uint64_t a = (uint64_t)p;
  return (const uint8_t*)(((uint64_t)uni((uint32_t)(a >> 32)) << 32) | uni((uint32_t)a));
}
// loads at (wave-uniform base) + (32-bit lane offset)
__device__ __forceinline__ u32x4_t ldg_stream(const uint8_t* base, uint32_t voff) {
  return __builtin_nontemporal_load((const DSGX_GLOBAL u32x4_t*)((const DSGX_GLOBAL uint8_t*)(uintptr_t)base + voff));
}
__device__ __forceinline__ uint32_t ldg_u32(const uint8_t* base, uint32_t voff) {
  return *(const DSGX_GLOBAL uint32_t*)((const DSGX_GLOBAL uint8_t*)(uintptr_t)base + voff);
}
__device__ __forceinline__ uint32_t ldg_u16(const uint8_t* base, uint32_t voff) {
  return *(const DSGX_GLOBAL uint16_t*)((const DSGX_GLOBAL uint8_t*)(uintptr_t)base + voff);
}
// pin_after() for a lane offset
__device__ __forceinline__ uint32_t pin_after(uint32_t voff, float dep) {
  asm volatile("" : "+v"(voff) : "v"(dep));
  return voff;
}
__device__ __forceinline__ uint32_t ldg_u32(const void* p) { return *(const DSGX_GLOBAL uint32_t*)(uintptr_t)p; }
__device__ __forceinline__ uint32_t ldg_u16(const void* p) { return *(const DSGX_GLOBAL uint16_t*)(uintptr_t)p; }

// ---- wave64 reductions, result valid in every lane -------------------------------------------------------------------------
// Steps 1, 2, 4, 8 run inside a row of 16 lanes with DPP (quad permutes and mirrors); rows are joined with gfx950's
// v_permlane16_swap / v_permlane32_swap: with both operands v, the two results hold each lane's own half and the other
// half, so their sum (or max) is the xor-16 / xor-32 butterfly step without a trip through LDS.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) { return v + __uint_as_float(dpp_mov<CTRL>(__float_as_uint(v))); }
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror: every lane of a row of 16 holds the row's sum
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// The sums over the wave of N values a lane (N a power of two up to 16) for little more than the price of one: the two
// widest butterfly steps (lane distance 32, then 16) are done as FOLDS, a lane-half swap of two values' registers
// leaving one register with the first value's pair sums in one half of the lanes and the second's in the other, so
// N registers become N / 4 before the four narrow steps (8, 4, 2, 1 within a row of 16 lanes). Every value is summed
// by the same tree whatever N is, so a result does not depend on how many others were reduced with it.
// On return v[j] holds, in lane l with l % 16 == j, the sum of value fold_var<N>(l); the other lanes of the row hold the
// same sum. fold_owner<N>(l): lane l is the one lane that keeps its value (l % 16 < registers left).
template <int N>
__device__ __forceinline__ int fold_var(uint32_t lane) {
  if (N == 1) return 0;
  if (N == 2) return lane >> 5;
  return 4 * (lane & 15) + 2 * ((lane >> 4) & 1) + (lane >> 5);
}
template <int N>
__device__ __forceinline__ bool fold_owner(uint32_t lane) {
  if (N == 1) return lane == 0;
  if (N == 2) return (lane & 31) == 0;
  return (lane & 15) < N / 4;
}
template <int N>
__device__ __forceinline__ float fold_sum(float (&v)[N], uint32_t lane) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16, "fold_sum: 1, 2, 4, 8 or 16 values");
  auto add32 = [](float a, float b) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
  };
  auto add16 = [](float a, float b) {
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
  };
  constexpr int N1 = N >= 2 ? N / 2 : 1, N2 = N >= 4 ? N / 4 : 1;
#pragma unroll
  for (int j = 0; j < N1; ++j) v[j] = N >= 2 ? add32(v[2 * j], v[2 * j + 1]) : add32(v[0], v[0]);
#pragma unroll
  for (int j = 0; j < N2; ++j) v[j] = N >= 4 ? add16(v[2 * j], v[2 * j + 1]) : add16(v[0], v[0]);
#pragma unroll
  for (int j = 0; j < N2; ++j) {
    v[j] = dpp_add<0x140>(v[j]);  // row_mirror (distance 8: both lanes' rows of eight hold different eights)
    v[j] = dpp_add<0x141>(v[j]);  // row_half_mirror
    v[j] = dpp_add<0x4E>(v[j]);   // quad_perm [2,3,0,1]
    v[j] = dpp_add<0xB1>(v[j]);   // quad_perm [1,0,3,2]
  }
  float r = v[0];
#pragma unroll
  for (int j = 1; j < N2; ++j) r = (lane & 15) == (uint32_t)j ? v[j] : r;
  return r;
}

// ---- the activation layout in LDS ---------------------------------------------------------------------------------------------
// A lane of a wavefront that streams a row holds KL consecutive k per segment of 64 * KL k (KL = 16 for FP8: one
// 16-byte load; 32 for INT4: one 16-byte load; 8, 16 or 32 for BF16: one, two or four 16-byte loads). The activations
// of row m are staged as 16-byte chunks of 8 k so that the lanes of a wavefront read consecutive chunks (no bank
// conflicts): chunk c (of KL / 8) of segment s of lane l sits at chunk index ((s * (KL / 8) + c) * 64 + l) of the row.
template <int KL>
__device__ __forceinline__ int xchunk_index(int q) {  // q: the row's chunk number in k order (k = 8 q)
  constexpr int XC = KL / 8;
  const int seg = q / (64 * XC), r = q % (64 * XC);
  return (seg * XC + r % XC) * 64 + r / XC;
}
// Stage rows x[M][ldx] (bf16, global) into lds [M][K/8 chunks] in the layout above; K a multiple of 8. Chunks past K in
// the last segment are zero-filled up to Kpad (a multiple of 64 * KL).
// COHERENT: read with device-scope coherent loads (data written by other workgroups of the same kernel).
// Eight chunks a thread are loaded before any is written to LDS, so their latencies overlap.
template <bool COHERENT>
__device__ __forceinline__ uint4 load_chunk(const uint16_t* p) {
  if (COHERENT) {
    const uint64_t* q = reinterpret_cast<const uint64_t*>(p);
    const uint64_t a = __hip_atomic_load((const DSGX_GLOBAL uint64_t*)(uintptr_t)q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t b = __hip_atomic_load((const DSGX_GLOBAL uint64_t*)(uintptr_t)(q + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_uint4((uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32));
  }
  const u32x4_t v = *(const DSGX_GLOBAL u32x4_t*)(uintptr_t)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}
template <int KL, bool COHERENT = false>
__device__ __forceinline__ void stage_x(uint4* lds, const uint16_t* x, size_t ldx, int M, int K, int Kpad) {
  const int nq = Kpad / 8, total = M * nq;
  constexpr int U = 8;
  for (int i0 = threadIdx.x; i0 < total; i0 += U * blockDim.x) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * blockDim.x;
      v[u] = make_uint4(0, 0, 0, 0);
      if (i < total) {
        const int m = i / nq, q = i % nq;
        if (8 * q < K) v[u] = load_chunk<COHERENT>(x + (size_t)m * ldx + 8 * q);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * blockDim.x;
      if (i < total) lds[(size_t)(i / nq) * nq + xchunk_index<KL>(i % nq)] = v[u];
    }
  }
}
// The same for `ns` consecutive slots of h (each M rows of K = ldx values) staged back to back: one pass over all of
// them, so that a chunk of slots costs one round trip and not one a slot. base(s) gives slot s's rows.
template <int KL, bool COHERENT, class Base>
__device__ __forceinline__ void stage_slots(uint4* lds, int ns, int M, int K, Base&& base) {
  const int nq = K / 8, per = M * nq, total = ns * per;
  constexpr int U = 8;
  for (int i0 = threadIdx.x; i0 < total; i0 += U * blockDim.x) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * blockDim.x;
      v[u] = make_uint4(0, 0, 0, 0);
      if (i < total) {
        const int s = i / per, r = i % per;
        v[u] = load_chunk<COHERENT>(base(s) + (size_t)(r / nq) * K + 8 * (r % nq));
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * blockDim.x;
      if (i < total) {
        const int s = i / per, r = i % per;
        lds[(size_t)s * per + (size_t)(r / nq) * nq + xchunk_index<KL>(r % nq)] = v[u];
      }
    }
  }
}

// ---- the router's row function (one wavefront a row) ------------------------------------------------------------------------------
// s = 1 / (1 + e^-l) from IEEE operations only, so the CPU and the GPU give the same bits: the reference's
// route_sigmoid (engine/experts/formats.cuh:142-163).
__device__ __forceinline__ float route_sigmoid(float l) {
  const float x = -l;
  if (x > 88.f) return 0.f;
  if (x < -87.f) return 1.f;
  const float n = rintf(x * 1.44269504f);
  float r = fmaf(-n, 0.693145751953125f, x);
  r = fmaf(-n, 1.428606765330187e-06f, r);
  float p = 1.f / 5040;
  p = fmaf(p, r, 1.f / 720);
  p = fmaf(p, r, 1.f / 120);
  p = fmaf(p, r, 1.f / 24);
  p = fmaf(p, r, 1.f / 6);
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.f);
  p = fmaf(p, r, 1.f);
  const float e = ldexpf(p, (int)n);
  return __fdiv_rn(1.f, __fadd_rn(1.f, e));
}
// softplus(l) = log1p(exp(l)) for l <= 20, again from IEEE operations only (the reference's log1pf(expf(l)),
// ds41f-4xgx10-switchless/engine/kernels/common.cuh:281, depends on the math library): exp by the sigmoid's reduction and
// polynomial; log1p(e) = log(u) e / (u - 1) with u = 1 + e; log by u = 2^k (1 + f), sqrt(1/2) < 1 + f < sqrt(2),
// s = f / (2 + f), log(1 + f) = f - f^2/2 + s (f^2/2 + R(s^2)), R the degree-7 minimax of fdlibm's e_logf.c. Every
// operation is written out and rounded on its own, so the host oracle's copy gives the same bits.
__device__ __forceinline__ float route_softplus(float l) {
  if (l < -87.f) l = -87.f;
  const float n = rintf(__fmul_rn(l, 1.44269504f));
  float r = fmaf(-n, 0.693145751953125f, l);
  r = fmaf(-n, 1.428606765330187e-06f, r);
  float p = 1.f / 5040;
  p = fmaf(p, r, 1.f / 720);
  p = fmaf(p, r, 1.f / 120);
  p = fmaf(p, r, 1.f / 24);
  p = fmaf(p, r, 1.f / 6);
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.f);
  p = fmaf(p, r, 1.f);
  const float e = ldexpf(p, (int)n);
  const float u = __fadd_rn(1.f, e);
  if (u == 1.f) return e;
  uint32_t ix = __float_as_uint(u);
  int k = (int)(ix >> 23) - 127;
  ix &= 0x007fffffu;
  const uint32_t i = (ix + (0x95f64u << 3)) & 0x800000u;
  ix |= i ^ 0x3f800000u;
  k += (int)(i >> 23);
  const float f = __fsub_rn(__uint_as_float(ix), 1.f), dk = (float)k;
  const float s_ = __fdiv_rn(f, __fadd_rn(2.f, f)), z = __fmul_rn(s_, s_), w = __fmul_rn(z, z);
  const float t1 = __fmul_rn(w, __fadd_rn(0.40000000596f, __fmul_rn(w, __fadd_rn(0.22222198546f, __fmul_rn(w, 0.15313838422f)))));
  const float t2 = __fmul_rn(z, __fadd_rn(0.66666668653f, __fmul_rn(w, __fadd_rn(0.28571429849f, __fmul_rn(w, __fadd_rn(0.18183572590f, __fmul_rn(w, 0.14798198640f)))))));
  const float R = __fadd_rn(t2, t1), hfsq = __fmul_rn(__fmul_rn(0.5f, f), f);
  const float inner = __fadd_rn(__fmul_rn(s_, __fadd_rn(hfsq, R)), __fmul_rn(dk, 9.0580006145e-06f));
  const float lg = __fsub_rn(__fmul_rn(dk, 0.69313812256f), __fsub_rn(__fsub_rn(hfsq, inner), f));
  return __fmul_rn(lg, __fdiv_rn(e, __fsub_rn(u, 1.f)));
}
__device__ __forceinline__ float route_score(float l, int score_fn) {
  if (score_fn == 0) return route_sigmoid(l);
  return sqrtf(l > 20.f ? l : route_softplus(l));  // DeepSeek's sqrt(softplus); sqrtf is the correctly rounded root (__fsqrt_rn is not)
}
// wave-wide maximum of floats (no NaNs), valid in every lane
template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) { return fmaxf(v, __uint_as_float(dpp_mov<CTRL>(__float_as_uint(v)))); }
__device__ __forceinline__ float wave_max_f32(float v) {
  v = dpp_max<0xB1>(v);
  v = dpp_max<0x4E>(v);
  v = dpp_max<0x141>(v);
  v = dpp_max<0x140>(v);
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// wave-wide minimum of unsigned ints, valid in every lane
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
  v = min(v, dpp_mov<0xB1>(v));
  v = min(v, dpp_mov<0x4E>(v));
  v = min(v, dpp_mov<0x141>(v));
  v = min(v, dpp_mov<0x140>(v));
  auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  v = min(r[0], r[1]);
  r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return min(r[0], r[1]);
}

// wave-wide maximum of unsigned ints, valid in every lane
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, dpp_mov<0xB1>(v));
  v = max(v, dpp_mov<0x4E>(v));
  v = max(v, dpp_mov<0x141>(v));
  v = max(v, dpp_mov<0x140>(v));
  auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  v = max(r[0], r[1]);
  r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return max(r[0], r[1]);
}
// a float's bits as an unsigned int of the same order (no NaNs; -0 does not occur: a score is never negative zero)
__device__ __forceinline__ uint32_t f32_order_bits(float f) {
  const uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// One row by one wavefront: experts e = lane + 64 j, j < NJ (E <= 64 NJ). Lane k < topk gets pick k's expert and
// weight (route_warp of the reference, engine/experts/formats.cuh:207-247, at 64 lanes): descending key (float
// compares), ties to the lower id; the sum in the butterfly order ((p0+p4)+(p2+p6))+((p1+p5)+(p3+p7)), absent places
// skipped. The code runs once a launch on a single wavefront, so its instruction count is its latency:
//  - every lane first sorts its NJ places by (key descending, j ascending) with adjacent exchanges (stable);
//  - a pick is the wave-wide maximum of the lanes' heads; the lane holding it (on a tie, rare, the lowest expert id
//    among the heads that hold it: a lane's own ties are already in id order) pops its list.
constexpr int kRouteRJ = DSGX_MAX_EXPERTS / kWave;
// a row's logits (or the bias; null: zeros) in the lanes' places; E wave-uniform
__device__ __forceinline__ void route_fetch(const float* __restrict__ row, int E, int lane, float (&v)[kRouteRJ]) {
  const int nj = (E + kWave - 1) / kWave;
#pragma unroll
  for (int j = 0; j < kRouteRJ; ++j) {
    const int e = lane + kWave * j;
    v[j] = 0.f;
    if (row && j < nj && e < E) v[j] = row[e];
  }
}
template <int NJ>
__device__ __forceinline__ void route_row_nj(const float (&logit)[kRouteRJ], const float (&bias)[kRouteRJ], int E, int topk, float scale,
                                             int score_fn, int lane, int& id_out, float& w_out) {
  // The keys are compared as unsigned ints of the floats' order (f32_order_bits): the wave-wide maximum is then one
  // instruction a step, a third of the float form's (which re-canonicalises its operands). 0 is below every key.
  constexpr uint32_t kDead = 0u;
  float s[NJ];
  uint32_t key[NJ];
  int jj[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    s[j] = 0.f, key[j] = kDead, jj[j] = j;  // an empty place never wins
    if (lane + kWave * j < E) {
      s[j] = route_score(logit[j], score_fn);
      key[j] = f32_order_bits(__fadd_rn(s[j], bias[j]));
    }
  }
  // odd-even transposition: NJ passes of adjacent exchanges, strictly-greater only (equal keys keep their j order)
#pragma unroll
  for (int pass = 0; pass < NJ; ++pass)
#pragma unroll
    for (int j = pass & 1; j + 1 < NJ; j += 2) {
      const bool sw = key[j + 1] > key[j];
      const uint32_t k0 = key[j];
      const float s0 = s[j];
      const int j0 = jj[j];
      key[j] = sw ? key[j + 1] : k0, s[j] = sw ? s[j + 1] : s0, jj[j] = sw ? jj[j + 1] : j0;
      key[j + 1] = sw ? k0 : key[j + 1], s[j + 1] = sw ? s0 : s[j + 1], jj[j + 1] = sw ? j0 : jj[j + 1];
    }
  // lane k keeps pick k; the loop is not unrolled
  float my_s = 0.f;
  int my_id = 0;
#pragma unroll 1
  for (int k = 0; k < topk; ++k) {
    const uint32_t top = wave_max_u32(key[0]);
    const uint64_t hit = __ballot(key[0] == top);
    int wl = __builtin_ctzll(hit);
    if (hit & (hit - 1)) wl = wave_min_u32(key[0] == top ? (uint32_t)(lane + kWave * jj[0]) : 0xFFFFFFFFu) & (kWave - 1);
    const int id = wl + kWave * __builtin_amdgcn_readlane(jj[0], wl);
    const float sv = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(s[0]), wl));
    if (lane == wl) {
#pragma unroll
      for (int j = 0; j + 1 < NJ; ++j) key[j] = key[j + 1], s[j] = s[j + 1], jj[j] = jj[j + 1];
      key[NJ - 1] = kDead;
    }
    if (lane == k) my_s = sv, my_id = id;
  }
  // lanes 0..7 hold p0..p7 (0 past topk: x + 0 = x): three xor steps are the reference's order of adds
  float sum = my_s;
  sum = __fadd_rn(sum, __shfl_xor(sum, 4));
  sum = __fadd_rn(sum, __shfl_xor(sum, 2));
  sum = __fadd_rn(sum, __shfl_xor(sum, 1));
  sum = __fadd_rn(sum, 1e-20f);
  id_out = my_id, w_out = lane < topk ? __fmul_rn(__fdiv_rn(my_s, sum), scale) : 0.f;
}
__device__ __forceinline__ void route_row(const float (&logit)[kRouteRJ], const float (&bias)[kRouteRJ], int E, int topk, float scale,
                                          int score_fn, int lane, int& id_out, float& w_out) {
  if (E <= 2 * kWave) route_row_nj<2>(logit, bias, E, topk, scale, score_fn, lane, id_out, w_out);
  else if (E <= 4 * kWave) route_row_nj<4>(logit, bias, E, topk, scale, score_fn, lane, id_out, w_out);
  else route_row_nj<kRouteRJ>(logit, bias, E, topk, scale, score_fn, lane, id_out, w_out);
}

// h = bf16(bf16(silu(g)) * u), g and u already bf16 values (engine/experts/decode.cu:110-113 of the reference)
__device__ __forceinline__ uint32_t swiglu_bits(float g, float u) {
  const float sl = bf16_round(__fdiv_rn(g, __fadd_rn(1.f, expf(-g))));
  return f32_to_bf16_bits(__fmul_rn(sl, u));
}

// The same with the hardware's exponential and reciprocal (each within 1 ulp) in place of expf() and the IEEE division:
// silu before its rounding to bf16 is within a few f32 ulp of the exact value (the reference's own expf() is specified to
// 2 ulp), so the bf16 it rounds to differs from swiglu_bits' once in ~10^4 values, by one bf16 step. For the prefill
// GEMMs' epilogues, where the exact form's ~20 extra instructions a value are a tenth of the kernel.
__device__ __forceinline__ uint32_t swiglu_fast_bits(float g, float u) {
  const float e = __builtin_amdgcn_exp2f(__fmul_rn(g, -1.44269504088896341f));
  const float sl = bf16_round(__fmul_rn(g, __builtin_amdgcn_rcpf(__fadd_rn(1.f, e))));
  return f32_to_bf16_bits(__fmul_rn(sl, u));
}
// v / d by d's reciprocal (r = rcp(d), within 1 ulp) and one correction step: the quotient rounded to nearest for every v
// and d met here (normal numbers far from the format's ends; the IEEE sequence spends twice the instructions on scaling
// for the ends). Checked against the division bit for bit in tests.
__device__ __forceinline__ float div_by(float v, float d, float r) {
  const float q = __fmul_rn(v, r);
  return fmaf(fmaf(-q, d, v), r, q);
}

}  // namespace dsgx
