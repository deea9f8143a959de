// The grouped GEMMs of DeepSeek's prefill MoE (dsk::moe_prefill, ds41f-4xgx10-switchless/engine/kernels/dsk.h:268-295;
// arithmetic engine/kernels/moe.cu:519-534, 974-981 and ref/inference/model.py:841-851): MXFP4 routed experts and the FP8
// shared expert against rows given as act_quant(x) (e4m3 with a ue8m0 scale per 32 values), on gfx950's block-scaled
// matrix instruction v_mfma_scale_f32_16x16x128_f8f6f4: a lane holds 32 k of one row of each operand and ONE E8M0 scale
// byte, the instruction scales every 32 consecutive k - exactly the formats' scale group - so weights (e2m1 or e4m3),
// activations and both scale tensors go to the instruction as stored - no conversion, no scaled adds on the vector unit -
// and the accumulators run through K inside the matrix unit.
//
// The tiling, the LDS staging by global_load_lds (lane-permuted sources so that the fragment reads are conflict-free),
// the hand-counted waits and the workgroup -> (tile, row group) map are those of pf_gemm_fp8.cuh; what differs:
//   * a weight row of a 128-k block is 64 bytes (e2m1) - four lanes a row, piece q of row r at slot q ^ (r / 4 % 4);
//   * the scales travel with the block: 4 bytes a weight row and 4 a position, read back a byte a lane (ds_read_u8);
//   * UP's epilogue is DeepSeek's: gate, up rounded to bf16, up clamped to +-limit and gate from above, silu(gate) * up
//     times the position's routing weight (none for the shared expert), rounded to bf16, then quantised per 32 channels
//     (ue8m0) for the down projection; DOWN rounds each position's outputs to bf16 (the reference's per-pick rounding).
#pragma once
#include "pf_gemm_fp8.cuh"

namespace dsgx {
namespace pfmx {

using pf8::dma16;
using pf8::dma4;
using pf8::kThreads;
using pf8::kWgRows;
using pf8::swz;
using pf8::v4f_t;
using pf8::v8i_t;
using pf8::wait_loads;

template <int WP, int WF>
struct Shape {
  static constexpr bool F4 = WF == DSGX_FMT_MXFP4_G32;
  static constexpr int kPos = 128 * WP, kSub = 8 * WP, WR = 8 / WP, RA = 2 * WP;
  static constexpr int kRowB = F4 ? 64 : 128;       // bytes of a weight row in a 128-k block
  static constexpr int kStageW = kWgRows * kRowB;
  static constexpr int kStageX = kPos * 128;
  static constexpr int kStageWS = kWgRows * 4;      // the weight rows' four scale bytes of the block
  static constexpr int kStageXS = kPos * 4;         // the positions'
  static constexpr int kStageBytes = kStageW + kStageX + kStageWS + kStageXS;
  static constexpr int kStages = 3 * kStageBytes <= 160 * 1024 ? 3 : 2;
  static constexpr int kLoads = (F4 ? 2 : 4) + 2 * WP + 2;  // a wave's loads a turn: weights, activations, the two scale words
  static constexpr int kLds = kStages * kStageBytes;        // (the epilogues reuse it: UP kPos x 256 B, DOWN 8 x 2 WP KiB)
};

struct Args {
  const uint8_t* aq;   // activations, e4m3 [rows][K]
  const uint8_t* as;   // their ue8m0 scales [rows][K / 32]
  const int* gather;   // position -> activation row (null: the position itself)
  const int* tile_e;   // the tile list (null: the shared expert on rows [0, nrows))
  const int* tile_m0;
  const int* ntiles;
  const int* off;
  int nrows;
  int H, I;
  const uint8_t *wa, *sa, *wb, *sb;  // UP: gate (w1), up (w3); DOWN: w2 in wa / sa. Expert e at + e * wstride / sstride.
  size_t wstride, sstride;
  const float* posw;   // UP, routed: the positions' routing weights (null: the shared expert, no weight)
  float limit;
  uint16_t* h;         // UP: h bf16 [position][I] (before its quantisation)
  uint8_t* hq;         // UP: h as e4m3 [position][I]
  uint8_t* hs;         // UP: its ue8m0 scales [position][I / 32]
  uint16_t* d;         // DOWN: bf16 [position][H]
};

__device__ __forceinline__ int sw4(int r) { return (r >> 2) & 3; }
// 128-byte rows (activations, e4m3 weights) lie in LDS in pf_gemm_fp8.cuh's layout, whose fragment reads (a lane's two
// neighbouring slots 2 part, 2 part + 1, swizzled by row) run without bank conflicts; what differs is WHICH 16 bytes of the
// row a slot holds: the block-scaled instruction wants bytes 16 part ... and 64 + 16 part ... in a lane, so logical piece
// x holds the row's piece x / 2 + 4 (x % 2). (Reading pieces part and 4 + part of rows stored in natural order instead
// costs every second LDS cycle to bank conflicts - measured.)
__device__ __forceinline__ int pc8(int x) { return (x >> 1) + 4 * (x & 1); }

template <int CBSZ>
__device__ __forceinline__ v4f_t mfma_mx(v8i_t a, v8i_t b, v4f_t c, int sa, int sb) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, CBSZ, 0, 0, sa, 0, sb);
}

// DIAG (diagnostic builds only; results are then wrong): 1 no loads after the first stages, 4 no workgroup barrier in the
// loop, 8 no MFMAs, 16 no fragment reads after the first turn, 32 two blocks only, 64 no epilogue
template <bool UP, int WP, int WF, int DIAG = 0>
__device__ __forceinline__ void gemm_tile(const Args& g, uint8_t* smem, int e, int m0, int mend, int ns) {
  using S = Shape<WP, WF>;
  constexpr bool F4 = S::F4;
  constexpr int CBSZ = F4 ? 4 : 0;
  const int K = UP ? g.H : g.I, KB = K / 128, G = K / 32;
  if (mend > m0 + S::kPos) mend = m0 + S::kPos;
  const size_t eo = (e < 0 || (DIAG & 128)) ? 0 : (size_t)e;  // (diagnostic 128: every tile reads expert 0's weights)
  const uint8_t *wa = g.wa + eo * g.wstride, *sa = g.sa + eo * g.sstride;
  const uint8_t *wb = UP ? g.wb + eo * g.wstride : wa, *sb = UP ? g.sb + eo * g.sstride : sa;
  const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6), r16 = lane & 15, part = lane >> 4;
  const int rg = wave % S::WR, pg = wave / S::WR;
  const int c0 = ns * (kWgRows / 2), r0 = ns * kWgRows;
  auto tile_row = [&](int i, const uint8_t*& wbase, const uint8_t*& sbase) {  // first weight row of 16-row tile i, its tensors
    if (UP) {
      wbase = (i & 1) ? wb : wa, sbase = (i & 1) ? sb : sa;
      return c0 + 16 * (i >> 1);
    }
    wbase = wa, sbase = sa;
    return r0 + 16 * i;
  };
  const int nmt = uni(min(S::kSub, (mend - m0 + 15) / 16));
  const int nj = uni(nmt > pg ? (nmt - pg + WP - 1) / WP : 0);

  // ---- what this lane fetches ----
  // weights: the wave brings tiles 2 wave, 2 wave + 1. e2m1: one instruction a tile, lane -> row lane / 4, piece
  // (lane % 4) ^ sw4(row); e4m3: two instructions a tile (rows 0-7, 8-15), lane -> row lane / 8, piece (lane % 8) ^ swz(row)
  const uint8_t* pw[2][2];
  const uint8_t* pws;  // lanes 0-31: the scale word of row lane % 16 of tile 2 wave + lane / 16
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const uint8_t *wbase, *sbase;
    const int row = tile_row(2 * wave + t, wbase, sbase);
    if (F4) {
      const int r = lane >> 2;
      pw[t][0] = wbase + (size_t)(row + r) * (K / 2) + 16 * ((lane & 3) ^ sw4(r));
      pw[t][1] = pw[t][0];
    } else {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int r = 8 * hh + (lane >> 3);
        pw[t][hh] = wbase + (size_t)(row + r) * K + 16 * pc8((lane & 7) ^ swz(r));
      }
    }
    if (((lane >> 4) & 1) == t) pws = sbase + (size_t)(F4 ? row + r16 : (row + r16) / 32) * G;
  }
  const int lr = lane >> 3, lq = lane & 7;
  const uint8_t* px[WP][2];
#pragma unroll
  for (int t = 0; t < WP; ++t)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int r = 8 * hh + lr;
      int pos = m0 + 16 * (WP * wave + t) + r;
      if (pos >= mend) pos = mend - 1;
      px[t][hh] = g.aq + (size_t)((DIAG & 256) ? pos & 255 : g.gather ? g.gather[pos] : pos) * K + 16 * pc8(lq ^ swz(r));  // (diagnostic 256: 256 hot rows)
    }
  const uint8_t* pxs;  // lanes 0 .. 16 WP - 1: the scale word of position 16 WP wave + lane
  {
    int pos = m0 + 16 * WP * wave + (lane & (16 * WP - 1));
    if (pos >= mend) pos = mend - 1;
    pxs = g.as + (size_t)(g.gather ? g.gather[pos] : pos) * G;
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
  // load number i (0 .. kLoads - 1) of block kb: the two scale words, the activations (L2 hits mostly), the weights last: a
  // wave's loads return in issue order, so a load that waits for HBM holds back every later one of its wave and the
  // cache's miss slots with them (weights first: 7% slower, measured). A turn issues them one at a time between its MFMAs (issue_some), so that the
  // texture unit works through a block's 50 KB while the matrix unit runs instead of in front of it: issued together after
  // the barrier they cost every wave the time the unit takes to accept them all (measured: a third of a turn).
  auto issue_one = [&](int kb, int i) {
    const int kc = kb < KB ? kb : KB - 1;
    const uint32_t st = lds0 + (uint32_t)(kb % S::kStages) * S::kStageBytes;
    const uint32_t wbase = st + (uint32_t)wave * (2 * 16 * S::kRowB), xbase = st + S::kStageW + (uint32_t)wave * (2048 * WP);
    if (i == 0) {
      if (lane < 16 * WP) dma4(reinterpret_cast<const float*>(pxs + 4 * kc), uni(st + S::kStageW + S::kStageX + S::kStageWS + (uint32_t)wave * (64 * WP)));
    } else if (i == 1) {
      if (lane < 32) dma4(reinterpret_cast<const float*>(pws + 4 * kc), uni(st + S::kStageW + S::kStageX + (uint32_t)wave * 128));
    } else if (i < 2 + 2 * WP) {
      const int q = i - 2;
      dma16(px[q >> 1][q & 1] + (size_t)kc * 128, uni(xbase + (q >> 1) * 2048 + (q & 1) * 1024));
    } else {
      const int q = i - 2 - 2 * WP;
      if (F4) dma16(pw[q][0] + (size_t)kc * 64, uni(wbase + q * 1024));
      else dma16(pw[q >> 1][q & 1] + (size_t)kc * 128, uni(wbase + (q >> 1) * 2048 + (q & 1) * 1024));
    }
  };
  auto issue = [&](int kb) {
#pragma unroll
    for (int i = 0; i < S::kLoads; ++i) issue_one(kb, i);
  };
#pragma unroll
  for (int s = 0; s + 1 < S::kStages; ++s) issue(s);

  // fragment reads. The instruction numbers an 8-bit operand's k as 64 h + 16 part + i (h: the lane's first or second four
  // registers, i: the byte) and a 4-bit operand's as 32 part + i, and takes the scale of k block g = k / 32 from the lanes
  // of part g (measured with one-hot operands): so activations and e4m3 weights give lane (row r16, part) the 16-byte
  // pieces part and 4 + part of its row's 128 bytes (LDS slots 2 part and 2 part + 1, see pc8), e2m1 weights piece part of
  // the row's 64, and every operand's scale byte `part` of the row's four goes to the lanes of that part.
  const int rd0 = (r16 >> 3) * 1024 + (r16 & 7) * 128 + ((2 * part) ^ swz(r16)) * 16;
  const int rd1 = (r16 >> 3) * 1024 + (r16 & 7) * 128 + ((2 * part + 1) ^ swz(r16)) * 16;
  const int rd4 = r16 * 64 + (part ^ sw4(r16)) * 16;
  auto frag8 = [&](const uint8_t* t) {
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(t + rd0), hi = *reinterpret_cast<const u32x4_t*>(t + rd1);
    return v8i_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };
  auto frag4 = [&](const uint8_t* t) {
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(t + rd4);
    return v8i_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, 0, 0, 0, 0};
  };
  const int rds = r16 * 4;         // the lane's row's scale word within a 16-row (16-position) tile's 64 bytes; its byte: `part`
  const int rsh = 8 * part;

  v4f_t acc[S::RA][8];
#pragma unroll
  for (int t = 0; t < S::RA; ++t)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[t][j] = v4f_t{0.f, 0.f, 0.f, 0.f};

  auto run = [&](auto nj_c) {
    constexpr int NJ = decltype(nj_c)::value;
    for (int kb = 0; kb < ((DIAG & 32) ? 2 : KB); ++kb) {
      wait_loads<(S::kStages - 2) * S::kLoads>();
      if (!(DIAG & 4)) __syncthreads();
      if (!(DIAG & 1) && NJ == 0) issue(kb + S::kStages - 1);
      if (NJ == 0) continue;
      // loads i with i * NJ / kLoads == j go out after the fragment reads of 16-position tile j
      auto issue_some = [&](int j) {
        if (DIAG & 1) return;
#pragma unroll
        for (int i = 0; i < S::kLoads; ++i)
          if (i * (NJ > 0 ? NJ : 1) / S::kLoads == j) issue_one(kb + S::kStages - 1, i);
      };
      const uint8_t* st = smem + (size_t)(((DIAG & 16) ? 0 : kb) % S::kStages) * S::kStageBytes;
      const uint8_t* W = st + S::RA * rg * (16 * S::kRowB);
      const uint8_t* X = st + S::kStageW + pg * 2048;
      const uint8_t* WS = st + S::kStageW + S::kStageX + S::RA * rg * 64 + rds;
      const uint8_t* XS = st + S::kStageW + S::kStageX + S::kStageWS + pg * 64 + rds;
      v8i_t fa[S::RA];
      int fs[S::RA];
#pragma unroll
      for (int t = 0; t < S::RA; ++t) {
        fa[t] = F4 ? frag4(W + t * 1024) : frag8(W + t * 2048);
        fs[t] = (*reinterpret_cast<const uint32_t*>(WS + t * 64) >> rsh) & 0xFFu;
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const v8i_t fb = frag8(X + j * (2048 * WP));
        const int xsb = (*reinterpret_cast<const uint32_t*>(XS + j * (64 * WP)) >> rsh) & 0xFFu;
        issue_some(j);
#pragma unroll
        for (int t = 0; t < S::RA; ++t) {
          if (DIAG & 8) acc[t][j][0] += __builtin_bit_cast(float, fa[t][0] ^ fb[1] ^ fs[t] ^ xsb), acc[t][j][2] += __builtin_bit_cast(float, fa[t][3] ^ fb[6]);
          else acc[t][j] = mfma_mx<CBSZ>(fa[t], fb, acc[t][j], fs[t], xsb);
        }
      }
    }
  };
  switch (nj) {
    case 0: run(std::integral_constant<int, 0>{}); break;
    case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    case 4: run(std::integral_constant<int, 4>{}); break;
    case 5: run(std::integral_constant<int, 5>{}); break;
    case 6: run(std::integral_constant<int, 6>{}); break;
    case 7: run(std::integral_constant<int, 7>{}); break;
    default: run(std::integral_constant<int, 8>{}); break;
  }
  wait_loads<0>();
  __syncthreads();
  if (DIAG & 64) {
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < S::RA; ++t)
#pragma unroll
      for (int j = 0; j < 8; ++j) sum += acc[t][j][0] + acc[t][j][1] + acc[t][j][2] + acc[t][j][3];
    if (sum == 12345.678f) reinterpret_cast<float*>(UP ? (void*)g.h : (void*)g.d)[tid] = sum;
    return;
  }

  // register q of lane l is weight row 4 (l / 16) + q of the 16-row tile, position l % 16 of the 16 positions
  if (UP) {
    const int I = g.I;
    const float lim = g.limit;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j >= nj) break;
      const int p = 16 * (pg + WP * j) + r16;
      const float wv = (g.posw && m0 + p < mend) ? g.posw[m0 + p] : 1.f;
#pragma unroll
      for (int b = 0; b < S::RA / 2; ++b) {
        uint32_t hb[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float gt = bf16_round(acc[2 * b][j][q]), up = bf16_round(acc[2 * b + 1][j][q]);
          up = fminf(fmaxf(up, -lim), lim);
          gt = fminf(gt, lim);
          float hv = __fmul_rn(__fdiv_rn(gt, __fadd_rn(1.f, expf(-gt))), up);
          if (g.posw) hv = __fmul_rn(wv, hv);
          hb[q] = f32_to_bf16_bits(hv);
        }
        const int ch = 16 * (S::RA / 2 * rg + b) + 4 * part;
        const int piece = (ch >> 3) ^ (p & 15);
        *reinterpret_cast<uint2*>(smem + p * 256 + piece * 16 + (ch & 4) * 2) = make_uint2(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16));
      }
    }
    __syncthreads();
    // 16 lanes a position, 8 channels a lane: a scale group (32 channels) is 4 lanes. The scale byte is the exponent of
    // max(amax, 1e-4) / 448 rounded up to a power of two (ds41f engine/kernels/common.cuh:53-66); codes e4m3(h * 2^(127 - e)).
    const int l16 = tid & 15;
    for (int p = tid >> 4; p < 16 * nmt; p += kThreads / 16) {
      const int pos = m0 + p;
      const u32x4_t hv = *reinterpret_cast<const u32x4_t*>(smem + p * 256 + (l16 ^ (p & 15)) * 16);
      float v[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[2 * i] = bf16_bits_to_f32(hv[i] & 0xFFFFu), v[2 * i + 1] = bf16_bits_to_f32(hv[i] >> 16);
      float amax = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
      amax = dpp_max<0xB1>(amax);
      amax = dpp_max<0x4E>(amax);
      const uint32_t bb = __float_as_uint(__fmul_rn(fmaxf(amax, 1e-4f), 1.0f / 448.0f));
      const uint32_t eb = ((bb >> 23) & 0xFFu) + ((bb & 0x7FFFFFu) != 0 ? 1u : 0u);
      const float inv = __uint_as_float((254u - eb) << 23);
      float qv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) qv[i] = fminf(448.f, fmaxf(-448.f, __fmul_rn(v[i], inv)));
      uint32_t o0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[0], qv[1], 0, false), o1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4], qv[5], 0, false);
      o0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[2], qv[3], o0, true), o1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[6], qv[7], o1, true);
      if (pos < mend) {
        *reinterpret_cast<u32x4_t*>(g.h + (size_t)pos * I + c0 + 8 * l16) = hv;
        *reinterpret_cast<uint2*>(g.hq + (size_t)pos * I + c0 + 8 * l16) = make_uint2(o0, o1);
        if ((l16 & 3) == 0) g.hs[(size_t)pos * (I / 32) + c0 / 32 + (l16 >> 2)] = (uint8_t)eb;
      }
    }
  } else {
    // a 16-position tile of the wave at a time through its own piece of LDS: written as held (4 consecutive rows of one
    // position = 8 bytes of bf16), read back as whole rows (32 WP rows = 64 WP bytes a position), 4 WP lanes a position
    const int H = g.H;
    constexpr int RB = 64 * WP, PC = RB / 16;  // bytes and 16-byte pieces of a position's rows of this wave
    uint8_t* my = smem + wave * (1024 * WP);
    const int row0 = r0 + 16 * S::RA * rg;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j >= nj) break;
#pragma unroll
      for (int t = 0; t < S::RA; ++t) {
        const uint32_t lo = f32_to_bf16_bits(acc[t][j][0]) | (f32_to_bf16_bits(acc[t][j][1]) << 16);
        const uint32_t hi = f32_to_bf16_bits(acc[t][j][2]) | (f32_to_bf16_bits(acc[t][j][3]) << 16);
        const int c = 2 * t + (part >> 1);  // the 16-byte piece: rows 16 t + 4 part ... are bytes 32 t + 8 part ...
        *reinterpret_cast<uint2*>(my + r16 * RB + ((c ^ r16) & (PC - 1)) * 16 + (part & 1) * 8) = make_uint2(lo, hi);
      }
#pragma unroll
      for (int i = 0; i < (16 * PC + 63) / 64; ++i) {
        const int idx = i * 64 + lane, p = idx / PC, c = idx % PC;
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(my + p * RB + ((c ^ p) & (PC - 1)) * 16);
        const int pos = m0 + 16 * (pg + WP * j) + p;
        if (pos < mend) *reinterpret_cast<u32x4_t*>(g.d + (size_t)pos * H + row0 + 8 * c) = v;
      }
    }
  }
}

// The shared expert (tile_e null: tiles of 256 rows over [0, nrows)).
template <bool UP, int WF, int DIAG = 0>
__global__ void __launch_bounds__(kThreads) k_gemm(Args g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int NS = UP ? g.I / (kWgRows / 2) : g.H / kWgRows;
  int tile, ns;
  pf8::task_of<true>(NS, tile, ns);
  if (ns >= NS) return;
  const int m0 = tile * Shape<2, WF>::kPos, mend = g.nrows;
  if (m0 >= mend) return;
  gemm_tile<UP, 2, WF, DIAG>(g, smem, -1, m0, mend, ns);
}
// The routed experts' list of both tile shapes (bit 30 of tile_e: a 256-position tile), an expert's tiles next to each other.
template <bool UP, int WF, int DIAG = 0>
__global__ void __launch_bounds__(kThreads) k_gemm_mixed(Args g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int NS = UP ? g.I / (kWgRows / 2) : g.H / kWgRows;
  int tile, ns;
  pf8::task_of<false>(NS, tile, ns);
  if (ns >= NS || tile >= *g.ntiles) return;
  const int te = g.tile_e[tile], e = te & 0xFFFF;
  const int m0 = g.off[e] + g.tile_m0[tile], mend = g.off[e + 1];
  if ((DIAG & 512) && !(te >> 30)) return;  // (diagnostic: the 256-position tiles only / the remainders only)
  if ((DIAG & 1024) && (te >> 30)) return;
  if (te >> 30) gemm_tile<UP, 2, WF, DIAG>(g, smem, e, m0, mend, ns);
  else gemm_tile<UP, 1, WF, DIAG>(g, smem, e, m0, mend, ns);
}

}  // namespace pfmx
}  // namespace dsgx
