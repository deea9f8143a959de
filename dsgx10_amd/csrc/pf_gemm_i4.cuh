// The grouped GEMMs of the prefill step for INT4 (group 32) experts with bf16 activations - the altar-1 contract
// (altar1-4xgx10-switchless/engine/experts/prefill.cu:337-352, 772-831 of the reference): a weight is the bf16 value
// W = bf16((u - u_z) s), products are summed in f32 by v_mfma_f32_16x16x32_bf16, whose accumulators the MFMA carries across K.
//
// The structure is pf_gemm_fp8.cuh's: a workgroup (8 waves) computes up to 128 positions against 256 weight rows (UP: 128
// channels, gate and up), a wave 32 rows x every position; both operands and the weights' scales and zero points go from
// memory straight into a stage of LDS (global_load_lds, three stages of one 128-k block, hand-counted waits, one workgroup
// barrier a block), a turn's loads are issued one at a time between its MFMAs. What is its own:
//   * a weight row of a block is 64 bytes of packed nibbles (four lanes a row, piece q of row r at slot q ^ (r / 4 % 4));
//     lane (row, part) reads ONE piece = the 32 values of one scale group, its bf16 scale and its zero-point word, decodes
//     them in registers (the decode kernels' routine: one rounding of the exact product) into the A fragments of four MFMAs;
//     MFMA j takes the lane's values 8 j .. 8 j + 7, i.e. k = 32 part + 8 j + [0, 8), and the activation fragment of MFMA j
//     holds the same k (the permutation of k inside a block is invisible to the sums);
//   * an activation row of a block is 256 bytes of bf16: sixteen 16-byte pieces, piece c of position r at slot c ^ r, four
//     instructions a 16-position tile; a lane's piece for MFMA j is 4 part + j;
//   * a block's weights are decoded a turn ahead, between the MFMAs of the block before: vector unit and matrix unit run
//     beside each other.
// The k order of the sums - block after block, inside a block the four MFMAs j = 0 .. 3 - is k_pf_gemm16's, so the bits
// are the ones that kernel gave.
#pragma once
#include "pf_gemm_fp8.cuh"

namespace dsgx {
namespace pfi4 {

using pf8::dma16;
using pf8::dma4;
using pf8::kThreads;
using pf8::kWgRows;
using pf8::v4f_t;
using pf8::wait_loads;
typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));

constexpr int kStageW = kWgRows * 64;        // 16 KiB of nibbles
constexpr int kStageS = kWgRows * 8;         // four bf16 scales a row
constexpr int kStageZ = (kWgRows / 8) * 16;  // four zero-point words a group of eight rows
// A tile's shape by its positions: 128 (three stages), or 64 for the tiles that hold no more rows (four stages). What a
// turn waits for is the trip to HBM of a block's 18.5 KB of weights, scales and zero points, not their rate (9 GB/s a CU):
// with three stages a block has one turn to land (it is decoded a turn ahead), with four it has two. Most tiles of a
// chunk of 2048 rows are such tiles (the median bucket holds 34 rows).
template <int POS>
struct Shape {
  static constexpr int kPos = POS;
  static constexpr int kSub = POS / 16;                  // its 16-position tiles: waves 0 .. kSub - 1 bring one each
  static constexpr int kStageX = POS * 256;              // bf16 rows of the block
  static constexpr int kStageBytes = kStageW + kStageX + kStageS + kStageZ;  // 51,712 | 35,328
  static constexpr int kStages = POS == 128 ? 3 : 4;
  static constexpr int kLds = kStages * kStageBytes;     // (the epilogues reuse it: UP POS x 256 B, DOWN 8 x 2 KiB)
};
constexpr int kLoads = 2 + 4 + 1 + 1;        // a wave's loads a turn: two weight tiles, one activation tile (four pieces of 4 rows), scales, zero points
constexpr int kLds = Shape<128>::kLds > Shape<64>::kLds ? Shape<128>::kLds : Shape<64>::kLds;

struct Args {
  const uint16_t* x;   // activations bf16 [rows][K]
  const int* gather;   // position -> activation row (null: the position itself)
  const int* tile_e;   // 128-position tiles: expert, first position inside the expert's bucket
  const int* tile_m0;
  const int* ntiles;
  const int* off;
  dsgx_layer_w L;
  uint16_t* h;         // UP: h bf16 [position][I]
  float* d;            // DOWN: f32 [position][H]
};

__device__ __forceinline__ int sw4(int r) { return (r >> 2) & 3; }

template <bool UP, int POS>
__device__ __forceinline__ void gemm_tile(const Args& g, uint8_t* smem, int e, int m0, int mend, int ns) {
  using S = Shape<POS>;
  constexpr int kPos = S::kPos, kStageX = S::kStageX, kStageBytes = S::kStageBytes, kStages = S::kStages;
  const int K = UP ? g.L.H : g.L.I, N = UP ? g.L.I : g.L.H, KB = K / 128, G = K / 32;
  if (mend > m0 + kPos) mend = m0 + kPos;
  const dsgx_mat_desc* dsc = g.L.desc + (size_t)e * 3;
  const size_t soff = ((size_t)N * K / 2 + 255) / 256 * 256, zoff = soff + ((size_t)N * G * 2 + 255) / 256 * 256;
  const uint8_t* ma = g.L.pool + dsc[UP ? 0 : 2].off;   // UP: gate; DOWN: down
  const uint8_t* mb = UP ? g.L.pool + dsc[1].off : ma;  // UP: up
  const float s2a = UP ? dsc[0].s2 : 1.f, s2b = UP ? dsc[1].s2 : 1.f;
  const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6), r16 = lane & 15, part = lane >> 4;
  const int c0 = ns * (kWgRows / 2), r0 = ns * kWgRows;
  // the wave's two 16-row tiles: UP the gate rows and the up rows of channels c0 + 16 wave ...; DOWN rows r0 + 32 wave + 16 t ...
  auto tile_row = [&](int t, const uint8_t*& base) {
    base = (UP && t) ? mb : ma;
    return UP ? c0 + 16 * wave : r0 + 32 * wave + 16 * t;
  };
  const int nmt = uni(min(S::kSub, (mend - m0 + 15) / 16));
  const bool brings_x = wave < S::kSub;  // (a wave's loads a turn: kLoads, or kLoads - 4)

  // ---- what this lane fetches ----
  const uint8_t* pw[2];   // weights: row lane / 4 of tile t, piece (lane % 4) ^ sw4(row)
  const uint8_t* psc;     // scales: lane -> (tile lane / 32, row lane / 2 % 16, half lane % 2): 4 bytes = two groups' bf16
  const uint8_t* pzp;     // lanes 0-15: zero points: (tile lane / 8, octet lane / 4 % 2, group lane % 4): one word
  {
    const uint8_t* base;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int row = tile_row(t, base), r = lane >> 2;
      pw[t] = base + (size_t)(row + r) * (K / 2) + 16 * ((lane & 3) ^ sw4(r));
    }
    const int ts = lane >> 5, rs = (lane >> 1) & 15;
    const int rows = tile_row(ts, base);
    psc = base + soff + ((size_t)(rows + rs) * G) * 2 + 4 * (lane & 1);
    const int tz = (lane >> 3) & 1, oz = (lane >> 2) & 1;
    const int rowz = tile_row(tz, base);
    pzp = base + zoff + ((size_t)((rowz >> 3) + oz) * G + (lane & 3)) * 4;
  }
  const uint8_t* px[4];   // activations: the wave brings 16-position tile `wave`; instruction i: position 4 i + lane / 16, piece (lane % 16) ^ position
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * i + (lane >> 4);
    int pos = m0 + 16 * wave + r;
    if (pos >= mend) pos = mend - 1;  // a ragged tile re-reads its last row (never stored)
    px[i] = reinterpret_cast<const uint8_t*>(g.x) + (size_t)(g.gather ? g.gather[pos] : pos) * K * 2 + 16 * ((lane & 15) ^ r);
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
  // load number i of block kb (clamped past the end: the last block again, into a stage nobody reads): the small ones first,
  // then the activations (L2 hits mostly), the weights last (a wave's loads return in issue order: the ones that wait for HBM
  // hold back every later one)
  auto issue_one = [&](int kb, int i) {
    const int kc = kb < KB ? kb : KB - 1;
    const uint32_t st = lds0 + (uint32_t)(kb % kStages) * kStageBytes;
    if (i == 0) {
      dma4(reinterpret_cast<const float*>(psc + (size_t)kc * 8), uni(st + kStageW + kStageX + (uint32_t)wave * 256));
    } else if (i == 1) {
      if (lane < 16) dma4(reinterpret_cast<const float*>(pzp + (size_t)kc * 16), uni(st + kStageW + kStageX + kStageS + (uint32_t)wave * 64));
    } else if (i < 6) {
      if (brings_x) dma16(px[i - 2] + (size_t)kc * 256, uni(st + kStageW + (uint32_t)wave * 4096 + (i - 2) * 1024));
    } else {
      dma16(pw[i - 6] + (size_t)kc * 64, uni(st + (uint32_t)wave * 2048 + (i - 6) * 1024));
    }
  };
#pragma unroll
  for (int s = 0; s + 1 < kStages; ++s)
#pragma unroll
    for (int i = 0; i < kLoads; ++i) issue_one(s, i);

  // fragment reads
  const int rdw = r16 * 64 + (part ^ sw4(r16)) * 16;  // the lane's 32 nibbles: row r16, group `part` of the block
  const int rds = r16 * 8 + part * 2;                 // its bf16 scale
  const int rdz = (r16 >> 3) * 16 + part * 4;         // its zero-point word (the row's nibble: r16 % 8)
  const uint32_t zsh = 4 * (r16 & 7);
  int rdx[4];                                         // the activation piece of MFMA j: 4 part + j of position r16
#pragma unroll
  for (int j = 0; j < 4; ++j) rdx[j] = r16 * 256 + (((4 * part + j) ^ r16) & 15) * 16;

  v4f_t acc[2][8];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[t][j] = v4f_t{0.f, 0.f, 0.f, 0.f};

  // A block's weights are decoded a turn ahead, a piece (one MFMA's fragment) at a time between the MFMAs of the turn before:
  // the decode is vector-unit work and the MFMAs run beside it. (Decoded in front of its own MFMAs it stood in their way: both
  // waves of a SIMD reach it together behind the barrier: 1.39 -> 1.1 ms for gate/up.) Turn kb therefore needs block kb + 1
  // landed: with three stages it waits for every load issued so far and issues block kb + 2's; with four, block kb + 2 may
  // still be in flight and it issues block kb + 3's.
  u32x4_t raw[2];
  float sc[2], nzs[2];
  auto open_block = [&](int kb) {  // the lane's raw words, scale and -(zero point * scale) of the wave's two tiles of block kb
    const uint8_t* st = smem + (size_t)(kb % kStages) * kStageBytes;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      raw[t] = *reinterpret_cast<const u32x4_t*>(st + wave * 2048 + t * 1024 + rdw);
      sc[t] = bf16_bits_to_f32(*reinterpret_cast<const uint16_t*>(st + kStageW + kStageX + wave * 256 + t * 128 + rds));
      nzs[t] = -((float)((*reinterpret_cast<const uint32_t*>(st + kStageW + kStageX + kStageS + wave * 64 + t * 32 + rdz) >> zsh) & 15u) * sc[t]);
    }
  };
  auto piece = [&](u32x4_t (&fa)[2][4], int pc) {  // piece pc = 4 t + j of the opened block
    const int t = pc >> 2, j = pc & 3;
    uint32_t o[4];
    i4x8_to_bf16(j == 0 ? raw[t].x : j == 1 ? raw[t].y : j == 2 ? raw[t].z : raw[t].w, sc[t], nzs[t], o);
    fa[t][j] = u32x4_t{o[0], o[1], o[2], o[3]};
  };
  auto run = [&](auto nj_c) {
    constexpr int NJ = decltype(nj_c)::value;
    u32x4_t fa[2][4], fn[2][4];
    // block 0 has landed (the later ones of the first stages may be in flight)
    if (brings_x) wait_loads<(kStages - 2) * kLoads>();
    else wait_loads<(kStages - 2) * (kLoads - 4)>();
    __syncthreads();
    open_block(0);
#pragma unroll
    for (int pc = 0; pc < 8; ++pc) piece(fa, pc);
    auto turn = [&](int kb, u32x4_t (&fa)[2][4], u32x4_t (&fn)[2][4]) {
      // block kb + 1 has landed (four stages: block kb + 2 may be in flight)
      if (brings_x) wait_loads<(kStages - 3) * kLoads>();
      else wait_loads<(kStages - 3) * (kLoads - 4)>();
      __syncthreads();
      open_block(kb + 1);
      const uint8_t* X = smem + (size_t)(kb % kStages) * kStageBytes + kStageW;
#pragma unroll
      for (int mt = 0; mt < 8; ++mt) {
        // (the turn's loads between its MFMAs; a ragged tile issues what is left behind its last 16-position tile)
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
          if (NJ > 0 ? (mt < NJ && i * NJ / kLoads == mt) : mt == 0) issue_one(kb + kStages - 1, i);
        piece(fn, mt);
        if (mt >= NJ) continue;
        u32x4_t fb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) fb[j] = *reinterpret_cast<const u32x4_t*>(X + mt * 4096 + rdx[j]);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < 2; ++t)
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, fa[t][j]), __builtin_bit_cast(v8bf_t, fb[j]), acc[t][mt], 0, 0, 0);
      }
    };
    for (int kb = 0; kb < KB; kb += 2) {  // (two turns a pass: the two fragment buffers swap roles without copies)
      turn(kb, fa, fn);
      if (kb + 1 < KB) turn(kb + 1, fn, fa);
    }
  };
  switch (nmt) {
    case 0: run(std::integral_constant<int, 0>{}); break;
    case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    default:
      if constexpr (S::kSub == 4) {
        run(std::integral_constant<int, 4>{});
      } else {
        switch (nmt) {
          case 4: run(std::integral_constant<int, 4>{}); break;
          case 5: run(std::integral_constant<int, 5>{}); break;
          case 6: run(std::integral_constant<int, 6>{}); break;
          case 7: run(std::integral_constant<int, 7>{}); break;
          default: run(std::integral_constant<int, 8>{}); break;
        }
      }
      break;
  }
  wait_loads<0>();
  __syncthreads();

  // register q of lane l is weight row 4 (l / 16) + q of the 16-row tile, position l % 16 of the 16 positions
  if (UP) {
    // h = bf16(bf16(silu(bf16 g)) * bf16 u) of the workgroup's 128 channels into an LDS tile [position][256 bytes] (16-byte
    // pieces exchanged by position: writes and reads spread over the banks), then whole lines to memory, 16 lanes a position
    const int I = g.L.I;
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
      if (mt >= nmt) break;
      const int p = 16 * mt + r16;
      uint32_t hb[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        hb[q] = swiglu_bits(bf16_round(__fmul_rn(acc[0][mt][q], s2a)), bf16_round(__fmul_rn(acc[1][mt][q], s2b)));
      const int ch = 16 * wave + 4 * part;
      const int piece = (ch >> 3) ^ (p & 15);
      *reinterpret_cast<uint2*>(smem + p * 256 + piece * 16 + (ch & 4) * 2) = make_uint2(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16));
    }
    __syncthreads();
    const int l16 = tid & 15;
    for (int p = tid >> 4; p < 16 * nmt; p += kThreads / 16) {
      const int pos = m0 + p;
      const u32x4_t hv = *reinterpret_cast<const u32x4_t*>(smem + p * 256 + (l16 ^ (p & 15)) * 16);
      if (pos < mend) *reinterpret_cast<u32x4_t*>(g.h + (size_t)pos * I + c0 + 8 * l16) = hv;
    }
  } else {
    // a 16-position tile at a time through the wave's own 2 KiB: written as held (four rows of a position: 16 bytes), read back
    // as whole rows (32 rows = 128 bytes a position, 8 lanes a position)
    const int H = g.L.H;
    uint8_t* my = smem + wave * 2048;
    const int row0 = r0 + 32 * wave;
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
      if (mt >= nmt) break;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int c = 4 * t + part;
        *reinterpret_cast<v4f_t*>(my + r16 * 128 + ((c ^ r16) & 7) * 16) = acc[t][mt];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int idx = i * 64 + lane, p = idx >> 3, c = idx & 7;
        const v4f_t v = *reinterpret_cast<const v4f_t*>(my + p * 128 + ((c ^ p) & 7) * 16);
        const int pos = m0 + 16 * mt + p;
        if (pos < mend) *reinterpret_cast<v4f_t*>(g.d + (size_t)pos * H + row0 + 4 * c) = v;
      }
    }
  }
}

template <bool UP>
__global__ void __launch_bounds__(kThreads) k_gemm(Args g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int NS = UP ? g.L.I / (kWgRows / 2) : g.L.H / kWgRows;
  int tile, ns;
  pf8::task_of<false>(NS, tile, ns);
  if (ns >= NS || tile >= *g.ntiles) return;
  const int e = g.tile_e[tile];
  const int m0 = g.off[e] + g.tile_m0[tile], mend = g.off[e + 1];
  if (mend - m0 <= 64) gemm_tile<UP, 64>(g, smem, e, m0, mend, ns);
  else gemm_tile<UP, 128>(g, smem, e, m0, mend, ns);
}

}  // namespace pfi4
}  // namespace dsgx
