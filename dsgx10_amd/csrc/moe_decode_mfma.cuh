// Decode variant 1 (dsgx_decode_cfg::up = 1) for FP8-128x128 layers: the expert matmuls on v_mfma_f32_16x16x32_bf16.
// The reference's decode kernels are tensor-core kernels too (engine/experts/decode.cu:307-343, 526-587: one MMA tile
// holds up to 16 activation rows); here a tile is 16 WEIGHT rows as the MFMA's A operand and the step's rows (up to 16,
// zero beyond M) as its B operand, so a row count costs nothing extra and no sum crosses lanes.
//   * a unit = 16 weight rows x all of K; the eight waves of a workgroup split K in eight slices and walk the slice in
//     steps of 64 k (1 KiB: lane l loads 16 bytes of row l / 4, four lanes 64 contiguous bytes of a row), a register ring
//     kD steps ahead; the bytes reach the MFMA's lane order (row l % 16, k part l / 16) through 1 KiB of the wave's LDS;
//   * e4m3 -> bf16 exactly in registers; per 128-k scale block the four MFMAs sum from zero, then
//     acc = fma(S, sum, acc) (the contract of the FP8 paths: decode.cu:269-306);
//   * the waves' slice sums are added in wave order through LDS (one workgroup barrier a unit), then the epilogue.
// gate/up: unit = 8 channels, rows interleaved (g0, u0, g1, u1, ...), so that g and u of a channel meet in one lane.
// down: units are (slot, 16 output rows), cut into equal contiguous ranges a workgroup; the complete dots go to memory
// as f32 [slot][M][H] and k_down_combine chains them in slot order (as after k_down_part).
// Every output depends on its own activation row only: a row's bits do not depend on the rows beside it.
#pragma once
#include "moe_decode_impl.cuh"

namespace dsgx {

typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
constexpr int kMfD = 4;           // ring depth in steps
constexpr int kMfPad = 64;        // bytes between activation rows in LDS beyond their length (bank spread)
constexpr int kMfThreads = 512;   // eight waves a workgroup, one workgroup a CU
constexpr int kMfWaves = kMfThreads / 64;

// K is cut into slices of whole 128-k scale blocks, one a wave (waves beyond the slices idle: small K only)
__host__ __device__ inline int mf_slices(int K) { return K / 128 < kMfWaves ? K / 128 : kMfWaves; }
__host__ __device__ inline size_t mf_rows_bytes(int M, int K) { return (size_t)M * ((size_t)K * 2 + kMfPad) + 64; }
// + two steps' weights a wave + the waves' slice sums of two units (the lanes of positions < M only: 4 M x 16 bytes a wave)
__host__ __device__ inline size_t mf_lds_bytes(int M, int K) { return mf_rows_bytes(M, K) + kMfWaves * 2048 + 2 * kMfWaves * 64 * M; }

// M rows of K bf16 (row m at src + m * ld) to LDS with the padded stride; 64 zero bytes after them
__device__ __forceinline__ void mf_stage_rows(uint8_t* lds, const uint16_t* src, size_t ld, int M, int K) {
  const int nq = K / 8, total = M * nq;
  const size_t rs = (size_t)K * 2 + kMfPad;
  for (int i0 = threadIdx.x; i0 < total; i0 += 4 * blockDim.x) {
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = min(i0 + u * (int)blockDim.x, total - 1);
      v[u] = load_chunk<false>(src + (size_t)(i / nq) * ld + 8 * (i % nq));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * blockDim.x;
      if (i < total) *reinterpret_cast<uint4*>(lds + (size_t)(i / nq) * rs + 16 * (i % nq)) = v[u];
    }
  }
  if (threadIdx.x < 4) *reinterpret_cast<uint4*>(lds + (size_t)M * rs + 16 * threadIdx.x) = make_uint4(0, 0, 0, 0);
}

// What a lane needs to walk units: set per unit by the caller's `open`
struct MfUnit {
  const uint8_t* wp;  // the lane's 16 bytes of the unit's first step: row l / 8 (and 8 rows on), piece l % 8, this wave's K slice
  size_t half;        // bytes from row l / 8 to row 8 + l / 8
  const float* sp;    // the first step's scale of the unit's even rows (lanes 0, 2, ...) or odd rows (lanes 1, 3, ...)
};

// The core: `nu` units of `steps` steps each; a step is one 128-k scale block of the unit's 16 rows (2 KiB: two loads,
// each eight rows x 128 contiguous bytes, eight lanes a row). open(u) -> MfUnit; done(u, sum) is called by one wave
// (they take turns) with the unit's complete sums (v4f: rows 4 (l / 16) + q, position l % 16). k0: the first k of this
// wave's slice; ns: the slices (= the waves that work). Every wave of the workgroup calls this with the same nu.
template <int M, class Open, class Done>
__device__ __forceinline__ void mf_stream(uint8_t* smem, size_t rows_bytes, int K, int k0, int ns, int nu, int steps, Open&& open, Done&& done) {
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6));
  float* red = reinterpret_cast<float*>(smem + rows_bytes + kMfWaves * 2048);
  auto finish = [&](int u) {  // after the unit's barrier: one wave adds the slices' sums in wave order
    if (wave == u % ns) {
      v4f_t sum = {0.f, 0.f, 0.f, 0.f};
      const int pos = lane & 15, part4 = lane >> 4;
      if (pos < M)
        for (int w = 0; w < ns; ++w) sum += *reinterpret_cast<const v4f_t*>(red + (((size_t)(u & 1) * kMfWaves + w) * 4 * M + part4 * M + pos) * 4);
      done(u, sum);
    }
  };
  if (wave >= ns) {  // (no slice: only the barriers)
    for (int u = 0; u < nu; ++u) __syncthreads();
    return;
  }
  const int r8 = lane >> 3, q = lane & 7, r16 = lane & 15, part = lane >> 4;
  uint8_t* W = smem + rows_bytes + wave * 2048;  // one step's weights: 16 rows x 128 bytes
  const size_t rs = (size_t)K * 2 + kMfPad;
  // LDS offsets. A row's eight 16-byte pieces are exchanged by (row / 2) % 8: the MFMA-order reads of 8 bytes (16 lanes:
  // 16 rows, one k part) then touch every bank once, and the row-major writes stay whole 128-byte rows.
  int wr_off[2], rd_off[4];
#pragma unroll
  for (int h = 0; h < 2; ++h) wr_off[h] = (8 * h + r8) * 128 + ((q ^ (((8 * h + r8) >> 1) & 7)) * 16);
#pragma unroll
  for (int j = 0; j < 4; ++j) rd_off[j] = r16 * 128 + (((2 * j + (part >> 1)) ^ ((r16 >> 1) & 7)) * 16) + 8 * (part & 1);
  const bool live = r16 < M;  // positions beyond the step's rows read the zero bytes
  const uint32_t xb = live ? (uint32_t)(r16 * rs) + (uint32_t)(k0 + 8 * part) * 2 : (uint32_t)(M * rs);
  const uint32_t xk = live ? 2u : 0u;

  struct Entry {
    u32x4_t a, b;  // rows l / 8 and 8 + l / 8
    float s;       // the block's scale (even lanes: of the even rows; odd lanes: of the odd rows)
  };
  Entry ring[kMfD];
  int lu = 0, lstep = 0, cu = 0, cstep = 0;
  MfUnit cur = open(0);
  v4f_t acc = {0.f, 0.f, 0.f, 0.f};
  auto load = [&](Entry& e) {
    const uint8_t* p = pin_after(cur.wp + (size_t)lstep * 128, acc[0]);
    e.a = ldg_stream(p);
    e.b = ldg_stream(p + cur.half);
    e.s = *(const DSGX_GLOBAL float*)(uintptr_t)(cur.sp + lstep);
    if (++lstep == steps) {
      lstep = 0;
      if (++lu < nu) cur = open(lu);  // (past the end the ring re-reads the last unit: unused)
    }
  };
  auto compute = [&](const Entry& e) {
    *reinterpret_cast<u32x4_t*>(W + wr_off[0]) = keep_whole(e.a);
    *reinterpret_cast<u32x4_t*>(W + wr_off[1]) = keep_whole(e.b);
    v4f_t part_sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint2 wq = *reinterpret_cast<const uint2*>(W + rd_off[j]);
      uint32_t o[4];
      fp8x8_to_bf16(wq.x, wq.y, o);
      const u32x4_t av = u32x4_t{o[0], o[1], o[2], o[3]};
      const u32x4_t bv = *reinterpret_cast<const u32x4_t*>(smem + xb + xk * (uint32_t)(cstep * 128 + 32 * j));
      part_sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, av), __builtin_bit_cast(v8bf_t, bv), part_sum, 0, 0, 0);
    }
    // the 128-k block is complete: the scaled add (even rows of the unit: lane 0's scale, odd rows: lane 1's)
    const float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, e.s), 0));
    const float s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, e.s), 1));
    acc[0] = fmaf(s0, part_sum[0], acc[0]), acc[1] = fmaf(s1, part_sum[1], acc[1]);
    acc[2] = fmaf(s0, part_sum[2], acc[2]), acc[3] = fmaf(s1, part_sum[3], acc[3]);
    if (++cstep < steps) return;
    cstep = 0;
    // the unit is complete in this wave's slice: the slices' sums through LDS, added in wave order by one wave
    if (live) *reinterpret_cast<v4f_t*>(red + (((size_t)(cu & 1) * kMfWaves + wave) * 4 * M + part * M + r16) * 4) = acc;
    acc = v4f_t{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    finish(cu);
    ++cu;
  };
#pragma unroll
  for (int d = 0; d < kMfD; ++d) load(ring[d]);
  const int total = nu * steps;
  for (int t = 0; t < total; t += kMfD) {
#pragma unroll
    for (int d = 0; d < kMfD; ++d) {
      if (t + d < total) compute(ring[d]);
      load(ring[d]);
    }
  }
}

template <int M, bool SH>
__device__ __forceinline__ void mf_setup(Step<M>& S, const DecodeArgs& a) {
  constexpr int NR = resolver_waves<M>();
  const int wave = uni((int)(threadIdx.x >> 6)), nw = blockDim.x >> 6;
  ResolveRegs rr;
  if (wave >= nw - NR) resolve_fetch(S, a, wave - (nw - NR), NR, rr);
  prep<DSGX_FMT_FP8_B128, SH ? DSGX_FMT_FP8_B128 : 0, M>(S, a);
  __syncthreads();
  if (wave >= nw - NR) resolve<DSGX_FMT_FP8_B128, SH ? DSGX_FMT_FP8_B128 : 0, M>(S, a, wave - (nw - NR), NR, rr);
  __syncthreads();
}

template <int M, bool SH>
__global__ void __launch_bounds__(kMfThreads) k_up_mfma(DecodeArgs a) {
  extern __shared__ uint8_t mf_smem[];
  __shared__ Step<M> S;
  mf_setup<M, SH>(S, a);
  const int H = a.L.H, I = a.L.I;
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6));
  mf_stage_rows(mf_smem, a.x, H, M, H);
  __syncthreads();
  const int nsl = (SH ? 1 : 0) + uni(S.n), tiles = I / 8, g = blockIdx.x, G = gridDim.x;
  const int tpw = uni(g < tiles ? (tiles - g + G - 1) / G : 0);  // this workgroup's tiles a slot
  const int ns = mf_slices(H), KS = H / ns, k0 = min(wave, ns - 1) * KS;
  const int r8 = lane >> 3, p8 = lane & 7;
  auto open = [&](int u) {
    const int sl = uni(u / tpw), t = g + (u - sl * tpw) * G;
    const Slot& T = S.slots[sl];
    const uint8_t* gw = T.g.w;
    const uint8_t* uw = T.u.w;
    const uint8_t* gs = T.g.s;
    const uint8_t* us = T.u.s;
    // rows of the unit: 2 c and 2 c + 1 are gate and up of channel 8 t + c; this lane loads rows l / 8 and 8 + l / 8
    MfUnit q;
    q.wp = ((r8 & 1) ? uw : gw) + (size_t)(8 * t + (r8 >> 1)) * H + k0 + p8 * 16;
    q.half = (size_t)4 * H;  // row 8 + r is gate / up (the same parity) of channel 4 further
    q.sp = reinterpret_cast<const float*>((lane & 1) ? us : gs) + (size_t)((8 * t) >> 7) * (H >> 7) + (k0 >> 7);
    return q;
  };
  auto done = [&](int u, v4f_t sum) {
    const int sl = uni(u / tpw), t = g + (u - sl * tpw) * G, pos = lane & 15, part = lane >> 4;
    if (pos >= M) return;
    const Slot& T = S.slots[sl];
    const float sg = T.g.s2, su = T.u.s2;
    const uint32_t h0 = swiglu_bits(bf16_round(__fmul_rn(sum[0], sg)), bf16_round(__fmul_rn(sum[1], su)));
    const uint32_t h1 = swiglu_bits(bf16_round(__fmul_rn(sum[2], sg)), bf16_round(__fmul_rn(sum[3], su)));
    uint16_t* dst = a.h + ((size_t)T.hslot * M + pos) * I + 8 * t + 2 * part;
    __hip_atomic_store((DSGX_GLOBAL uint32_t*)(uintptr_t)dst, h0 | (h1 << 16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  if (tpw > 0) mf_stream<M>(mf_smem, mf_rows_bytes(M, H), H, k0, ns, nsl * tpw, KS / 128, open, done);
}

template <int M, bool SH>
__global__ void __launch_bounds__(kMfThreads) k_down_mfma(DecodeArgs a) {
  extern __shared__ uint8_t mf_smem[];
  __shared__ Step<M> S;
  mf_setup<M, SH>(S, a);
  constexpr int nsh = SH ? 1 : 0;
  const int H = a.L.H, I = a.L.I;
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6));
  const int nrouted = uni(S.n), nsl = nsh + nrouted;
  if (blockIdx.x == 0) {  // the slot table for k_down_combine
    if (threadIdx.x == 0) reinterpret_cast<int*>(a.fac)[0] = nrouted;
    for (int i = threadIdx.x; i < nrouted * M; i += blockDim.x)
      a.fac[8 + (i / M) * 8 + i % M] = __fmul_rn(S.slots[nsh + i / M].d.s2, S.wslot[i / M][i % M]);
  }
  const int tps = H / 16;  // tiles a slot
  const long total = (long)nsl * tps;
  const int u_lo = (int)(total * blockIdx.x / gridDim.x), u_hi = (int)(total * (blockIdx.x + 1) / gridDim.x);
  const int ns = mf_slices(I), KS = I / ns, k0 = min(wave, ns - 1) * KS;
  const int r8 = lane >> 3, p8 = lane & 7;
  for (int sl = u_lo / tps; sl * tps < u_hi; ++sl) {  // (the same for every wave of the workgroup)
    const int ta = max(u_lo, sl * tps) - sl * tps, tb = min(u_hi, (sl + 1) * tps) - sl * tps;
    const Slot& T = S.slots[sl];
    __syncthreads();
    mf_stage_rows(mf_smem, a.h + (size_t)T.hslot * M * I, I, M, I);
    __syncthreads();
    if (tb <= ta) continue;
    const uint8_t* dw = T.d.w;
    const uint8_t* ds = T.d.s;
    float* out = a.dpart + (size_t)sl * M * H;
    auto open = [&](int u) {
      const int t = ta + u;
      MfUnit q;
      q.wp = dw + (size_t)(16 * t + r8) * I + k0 + p8 * 16;
      q.half = (size_t)8 * I;
      q.sp = reinterpret_cast<const float*>(ds) + (size_t)((16 * t) >> 7) * (I >> 7) + (k0 >> 7);
      return q;
    };
    auto done = [&](int u, v4f_t sum) {
      const int t = ta + u, pos = lane & 15, part = lane >> 4;
      if (pos < M) *reinterpret_cast<v4f_t*>(out + (size_t)pos * H + 16 * t + 4 * part) = sum;
    };
    mf_stream<M>(mf_smem, mf_rows_bytes(M, I), I, k0, ns, tb - ta, KS / 128, open, done);
  }
}

template <bool SH>
int launch_decode_mfma_m(const DecodeArgs& a, int parts, hipStream_t st);

template <int M, bool SH>
int launch_decode_mfma(const DecodeArgs& a, int parts, hipStream_t st) {
  const int H = a.L.H, I = a.L.I, cus = num_cus_cached();
  if (H % 128 || I % 128 || H % mf_slices(H) || (H / mf_slices(H)) % 128 || (I / mf_slices(I)) % 128)
    return fail(DSGX_EINVAL, "moe_decode (variant 1): hidden %d, intermediate %d (slices of whole 128-k blocks)", H, I);
  if (parts & 1) {
    auto kern = k_up_mfma<M, SH>;
    const size_t lds = mf_lds_bytes(M, H);
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(kMfThreads), lds, st, a);
    DSGX_HIP(hipGetLastError());
  }
  if (parts & 2) {
    auto kern = k_down_mfma<M, SH>;
    const size_t lds = mf_lds_bytes(M, I);
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(kMfThreads), lds, st, a);
    hipLaunchKernelGGL((k_down_combine<M, SH>), dim3((M * H + 255) / 256), dim3(256), 0, st, a);
    DSGX_HIP(hipGetLastError());
  }
  return DSGX_OK;
}

template <bool SH>
int launch_decode_mfma_m(const DecodeArgs& a, int parts, hipStream_t st) {
  switch (a.M) {
    case 1: return launch_decode_mfma<1, SH>(a, parts, st);
    case 2: return launch_decode_mfma<2, SH>(a, parts, st);
    case 3: return launch_decode_mfma<3, SH>(a, parts, st);
    case 4: return launch_decode_mfma<4, SH>(a, parts, st);
    case 5: return launch_decode_mfma<5, SH>(a, parts, st);
    case 6: return launch_decode_mfma<6, SH>(a, parts, st);
    case 7: return launch_decode_mfma<7, SH>(a, parts, st);
    case 8: return launch_decode_mfma<8, SH>(a, parts, st);
  }
  return fail(DSGX_EUNSUPPORTED, "moe_decode (variant 1): %d rows", a.M);
}

}  // namespace dsgx
