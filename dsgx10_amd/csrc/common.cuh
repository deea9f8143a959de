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
__device__ __forceinline__ void i4x8_to_bf16(uint32_t w, float s, float nzs, uint32_t (&o)[4]) {
  const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;  // lo: values 0,2,4,6; hi: 1,3,5,7
  o[0] = pack_bf16(fmaf((float)(lo & 0xFFu), s, nzs), fmaf((float)(hi & 0xFFu), s, nzs));
  o[1] = pack_bf16(fmaf((float)((lo >> 8) & 0xFFu), s, nzs), fmaf((float)((hi >> 8) & 0xFFu), s, nzs));
  o[2] = pack_bf16(fmaf((float)((lo >> 16) & 0xFFu), s, nzs), fmaf((float)((hi >> 16) & 0xFFu), s, nzs));
  o[3] = pack_bf16(fmaf((float)(lo >> 24), s, nzs), fmaf((float)(hi >> 24), s, nzs));
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
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
  auto step = [](uint64_t x, uint32_t olo, uint32_t ohi) {
    const uint64_t o = ((uint64_t)ohi << 32) | olo;
    return o > x ? o : x;
  };
  v = step(v, dpp_mov<0xB1>((uint32_t)v), dpp_mov<0xB1>((uint32_t)(v >> 32)));
  v = step(v, dpp_mov<0x4E>((uint32_t)v), dpp_mov<0x4E>((uint32_t)(v >> 32)));
  v = step(v, dpp_mov<0x141>((uint32_t)v), dpp_mov<0x141>((uint32_t)(v >> 32)));
  v = step(v, dpp_mov<0x140>((uint32_t)v), dpp_mov<0x140>((uint32_t)(v >> 32)));
  {
    auto lo = __builtin_amdgcn_permlane16_swap((uint32_t)v, (uint32_t)v, false, false);
    auto hi = __builtin_amdgcn_permlane16_swap((uint32_t)(v >> 32), (uint32_t)(v >> 32), false, false);
    const uint64_t a = ((uint64_t)hi[0] << 32) | lo[0], b = ((uint64_t)hi[1] << 32) | lo[1];
    v = a > b ? a : b;
  }
  {
    auto lo = __builtin_amdgcn_permlane32_swap((uint32_t)v, (uint32_t)v, false, false);
    auto hi = __builtin_amdgcn_permlane32_swap((uint32_t)(v >> 32), (uint32_t)(v >> 32), false, false);
    const uint64_t a = ((uint64_t)hi[0] << 32) | lo[0], b = ((uint64_t)hi[1] << 32) | lo[1];
    v = a > b ? a : b;
  }
  return v;
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
__device__ __forceinline__ float route_score(float l, int score_fn) {
  if (score_fn == 0) return route_sigmoid(l);
  return sqrtf(l > 20.f ? l : log1pf(expf(l)));  // DeepSeek's sqrt(softplus): libm-dependent, not promised bit-exact
}
// One row by one wavefront: experts e = lane + 64 j, j < 8 (E <= 512). Lane k < topk gets pick k's expert and weight
// (route_warp of the reference, engine/experts/formats.cuh:207-247, at 64 lanes): descending key, ties to the lower
// id; the sum in the butterfly order over eight places ((p0+p4)+(p2+p6))+((p1+p5)+(p3+p7)), absent places skipped.
// The (key, id) order is one unsigned 64-bit order: the key's bits made monotone (sign flipped for positive, all
// flipped for negative floats) above the complemented id, so each pick is one wave-wide integer maximum.
__device__ __forceinline__ void route_row(const float* __restrict__ logits_row, const float* __restrict__ bias, int E, int topk,
                                          float scale, int score_fn, int lane, int& id_out, float& w_out) {
  constexpr int RJ = DSGX_MAX_EXPERTS / kWave;
  float s[RJ];
  uint64_t key[RJ];
  const int nj = (E + kWave - 1) / kWave;
#pragma unroll
  for (int j = 0; j < RJ; ++j) {
    const int e = lane + kWave * j;
    s[j] = 0.f, key[j] = 0;  // an empty place: below every real key
    if (j < nj && e < E) {
      s[j] = route_score(logits_row[e], score_fn);
      const uint32_t kb = __float_as_uint(__fadd_rn(s[j], bias ? bias[e] : 0.f));
      const uint32_t mono = kb ^ ((kb >> 31) ? 0xFFFFFFFFu : 0x80000000u);
      key[j] = ((uint64_t)mono << 32) | (uint32_t)(~e);
    }
  }
  float picked[DSGX_MAX_TOPK];
  int ids[DSGX_MAX_TOPK];
#pragma unroll
  for (int k = 0; k < DSGX_MAX_TOPK; ++k) {
    picked[k] = 0.f, ids[k] = 0;
    if (k >= topk) continue;
    uint64_t best = 0;
#pragma unroll
    for (int j = 0; j < RJ; ++j)
      if (j < nj && key[j] > best) best = key[j];
    best = wave_max_u64(best);
    const int be = (int)(~(uint32_t)best);
    ids[k] = be;
    float sv = 0.f;
#pragma unroll
    for (int j = 0; j < RJ; ++j)
      if (j < nj && lane + kWave * j == be) sv = s[j], key[j] = 0;
    picked[k] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(sv), __builtin_amdgcn_readfirstlane(be & (kWave - 1))));
  }
  auto add = [](float a, float b, bool hb) { return hb ? __fadd_rn(a, b) : a; };
  const float a04 = add(picked[0], picked[4], 4 < topk), a26 = add(picked[2], picked[6], 6 < topk);
  const float a15 = add(picked[1], picked[5], 5 < topk), a37 = add(picked[3], picked[7], 7 < topk);
  const float sum = __fadd_rn(add(add(a04, a26, 2 < topk), add(a15, a37, 3 < topk), 1 < topk), 1e-20f);
  id_out = 0, w_out = 0.f;
#pragma unroll
  for (int k = 0; k < DSGX_MAX_TOPK; ++k)
    if (lane == k && k < topk) id_out = ids[k], w_out = __fmul_rn(__fdiv_rn(picked[k], sum), scale);
}

// h = bf16(bf16(silu(g)) * u), g and u already bf16 values (engine/experts/decode.cu:110-113 of the reference)
__device__ __forceinline__ uint32_t swiglu_bits(float g, float u) {
  const float sl = bf16_round(__fdiv_rn(g, __fadd_rn(1.f, expf(-g))));
  return f32_to_bf16_bits(__fmul_rn(sl, u));
}

}  // namespace dsgx
