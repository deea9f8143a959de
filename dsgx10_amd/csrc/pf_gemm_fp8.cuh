// The FP8 x FP8 grouped GEMM of the prefill step (gate/up + SwiGLU, and down), DeepSeek's block-scaled contract
// (ds41f-4xgx10-switchless/ref/torchref/kernel.py:105-125, ref/inference/kernel.py:207-274 of the reference): per 128-k
// block the e4m3 x e4m3 products summed in f32 from zero, then acc = fma(x_scale * w_scale, partial, acc).
//
// A workgroup (8 waves) computes one tile of positions against 256 weight rows (UP: 128 channels, gate and up), in one
// of two shapes (template parameter WP):
//   WP 1  up to 128 positions; a wave owns 32 weight rows and every position; three LDS stages of one 128-k block;
//   WP 2  up to 256 positions; the waves form 4 row groups x 2 position groups, a wave owns 64 weight rows and every
//         second 16-position tile; two LDS stages. For the shared expert and for experts that hold many rows: half the
//         bytes from L2 a flop, and an expert's weights are read half as often.
// Weights are the MFMA's A operand, so a lane's four accumulators of a 16 x 16 tile belong to ONE position and the
// block's combined scale is one value a lane.
//
// Both operands go from memory straight into LDS (global_load_lds_dwordx4: no registers, no LDS store instructions).
// Such a load puts lane l's 16 bytes at (base) + 16 l, so the LDS layout is chosen by what each lane fetches: a 16-row
// tile is two instructions of eight rows, eight consecutive lanes fetch the eight 16-byte pieces of one row's 128 bytes
// (one full line of the caches) in the order piece = q ^ swz(row), swz(r) = (r % 8) ^ (r / 8), which leaves piece c of
// row r at slot 8 r + (c ^ swz(r)): the MFMA-order reads (consecutive lanes = consecutive rows, one piece) then touch
// different bank groups, whether the LDS serves 8 lanes (128 bytes) or 16 lanes (256 bytes) a clock: swz is one-to-one
// on rows 0-7, on rows 8-15, on the even rows and on the odd rows (measured: no bank conflicts).
// The loads are written as inline assembly with the waits counted by hand (the compiler would otherwise wait for every
// outstanding load before each LDS read): a fixed number of loads a wave and turn, so vmcnt(that number x blocks still
// allowed in flight) = "the block of this turn has landed".
//
// The number of live 16-position tiles of a wave (ragged tiles: most experts of a chunk hold fewer rows than a tile) is
// a template parameter of the loop: a turn is straight-line code, the MFMAs take the constant 0 as their addend, and
// tiles past the end cost nothing.
//
// Epilogues go through LDS so that every store instruction writes whole 128-byte lines (a lane's accumulators are four
// consecutive weight rows of one position: stored directly, each line would be written in pieces by several
// instructions, which the memory system pays for several times over). UP also quantises h for the down projection
// (act_quant over the workgroup's 128 channels = one scale block) on the way out.
#pragma once
#include <type_traits>

#include "abi_internal.h"
#include "common.cuh"

namespace dsgx {
namespace pf8 {

typedef int v8i_t __attribute__((ext_vector_type(8)));
typedef float v4f_t __attribute__((ext_vector_type(4)));

constexpr int kWgRows = 256;      // weight rows a workgroup (UP: 128 channels)
constexpr int kThreads = 512;

template <int WP>
struct Shape {
  static constexpr int kPos = 128 * WP;            // positions of a tile
  static constexpr int kSub = 8 * WP;              // its 16-position tiles
  static constexpr int WR = 8 / WP;                // row groups of waves
  static constexpr int RA = 2 * WP;                // 16-row tiles a wave
  static constexpr int kStages = WP == 1 ? 3 : 2;
  static constexpr int kStageW = kWgRows * 128;    // sixteen 16-row tiles of 2 KiB
  static constexpr int kStageX = kPos * 128;
  static constexpr int kStageBytes = kStageW + kStageX + kPos * 4;  // + the positions' scales of the block
  static constexpr int kLoads = 5 + 2 * WP;        // a wave's loads a turn: 4 weight, 2 WP activation, 1 scale
  static constexpr int kLds = kStages * kStageBytes;  // (the epilogues reuse it: UP kPos x 256 B, DOWN 8 x 2 WP KiB)
};

struct Args {
  const uint8_t* aq;   // activations, e4m3 [rows][K]
  const float* as;     // their scales [rows][K / 128]
  const int* gather;   // position -> activation row (null: the position itself)
  const int* tile_e;   // the tile list (null: one pseudo-expert -1 holding rows [0, nrows): the shared expert)
  const int* tile_m0;
  const int* ntiles;
  const int* off;
  int nrows;           // shared expert: T
  int fast_act;        // UP: SwiGLU by the hardware's exp2 / rcp instead of expf() and the IEEE division
  dsgx_layer_w L;
  uint16_t* h;         // UP: h bf16 [position][I]
  uint8_t* hq;         // UP: h quantised, e4m3 [position][I]
  float* hs;           // UP: its scales [position][I / 128]
  float* d;            // DOWN: f32 [position][H]
#ifdef DSGX_PF_TRACE
  unsigned long long* trace;  // (diagnostic build: thread 0's wall-clock stamps, 8 a workgroup)
#endif
};
#ifdef DSGX_PF_TRACE
#define PF_STAMP(g, k) do { if ((g).trace && threadIdx.x == 0) (g).trace[(size_t)blockIdx.x * 8 + (k)] = wall_clock64(); } while (0)
#else
#define PF_STAMP(g, k) do { } while (0)
#endif

// Workgroup -> (position tile, group of weight rows): blocks of kMapTiles consecutive tiles x kMapNs row groups get 32
// consecutive workgroup numbers of ONE XCD (numbers x, x + 8, x + 16, ...), so that what they share (a tile's
// activations, an expert's weights) is fetched into that XCD's L2 once. 8 tiles x 4 row groups measured best at the
// benchmark's chunk (routed 2.83 ms against 2.875 with 4 x 8, 2.85 with 16 x 2, 2.97 with 2 x 16 or 32 x 1: what pays
// is an expert's weights shared between its neighbouring tiles, more than a tile's activations between row groups).
constexpr int kMapTiles = 8, kMapNs = 4, kXcds = 8;
__host__ __device__ inline unsigned grid_of(int tiles, int NS) {
  const int blocks = ((tiles + kMapTiles - 1) / kMapTiles) * ((NS + kMapNs - 1) / kMapNs);
  return (unsigned)((blocks + kXcds - 1) / kXcds) * kXcds * (kMapTiles * kMapNs);
}
// TILE_MINOR: neighbouring workgroup numbers are neighbouring tiles of one row group (the dense GEMM of the shared expert,
// where every tile streams the same weights: 0.241 against 0.250 ms at 8192 rows); else the row groups of one tile (the
// routed experts' list: 1.63 against 1.75 ms for gate/up).
template <bool TILE_MINOR>
__device__ __forceinline__ void task_of(int NS, int& tile, int& ns) {
  const int x = blockIdx.x % kXcds, j = blockIdx.x / kXcds;
  const int b = (j / (kMapTiles * kMapNs)) * kXcds + x, i = j % (kMapTiles * kMapNs);
  const int NG = (NS + kMapNs - 1) / kMapNs;
  tile = (b / NG) * kMapTiles + (TILE_MINOR ? i % kMapTiles : i / kMapNs);
  ns = (b % NG) * kMapNs + (TILE_MINOR ? i / kMapTiles : i % kMapNs);
}

// lane l's 16 bytes from `src` to LDS at lds_base + 16 l (lds_base wave-uniform)
__device__ __forceinline__ void dma16(const uint8_t* src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(src) : "memory");
}
// the active lanes' 4 bytes to lds_base + 4 l
__device__ __forceinline__ void dma4(const float* src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_base), "v"(src) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ int swz(int r) { return (r & 7) ^ (r >> 3); }

// DIAG (diagnostic builds only; results are then wrong): 1 no loads after the first stages, 2 the MFMAs accumulate by
// themselves (no scaled adds on the vector unit), 4 no workgroup barrier in the loop, 8 no MFMAs, 16 no fragment reads
// after the first turn, 128 the weight loads / 256 the activation loads re-read block 0 (cached) after the first stages
// one tile: expert e (-1: the shared expert), rows [m0, mend) of the activations' positions, row group ns
template <bool UP, int WP, int DIAG>
__device__ __forceinline__ void gemm_tile(const Args& g, uint8_t* smem, int e, int m0, int mend, int ns) {
  using S = Shape<WP>;
  const int K = UP ? g.L.H : g.L.I, KB = K / 128;
  if (mend > m0 + S::kPos) mend = m0 + S::kPos;  // (the tile's own rows)
  const uint8_t *wa, *wb;  // UP: gate, up; DOWN: down twice
  const float *sa, *sb;
  float s2a = 1.f, s2b = 1.f;
  const size_t NK = (size_t)g.L.H * g.L.I;
  if (e < 0) {
    if (UP) wa = g.L.sh.g, sa = g.L.sh.gs, wb = g.L.sh.u, sb = g.L.sh.us;
    else wa = wb = g.L.sh.d, sa = sb = g.L.sh.ds;
  } else {
    const dsgx_mat_desc* d = g.L.desc + (size_t)e * 3;
    if (UP) wa = g.L.pool + d[0].off, wb = g.L.pool + d[1].off, s2a = d[0].s2, s2b = d[1].s2;
    else wa = wb = g.L.pool + d[2].off;
    sa = reinterpret_cast<const float*>(wa + (NK + 255) / 256 * 256);
    sb = reinterpret_cast<const float*>(wb + (NK + 255) / 256 * 256);
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6), r16 = lane & 15, part = lane >> 4;
  const int rg = wave % S::WR, pg = wave / S::WR;  // the wave's row group and position group
  // The workgroup's sixteen 16-row tiles. UP: tile 2 c is the gate rows, tile 2 c + 1 the up rows of channels
  // c0 + 16 c ... (so a wave's tiles come in gate/up pairs of the same channels); DOWN: tile i is rows r0 + 16 i ...
  const int c0 = ns * (kWgRows / 2), r0 = ns * kWgRows;
  auto tile_row = [&](int i, const uint8_t*& base) {  // first weight row of tile i and its matrix
    if (UP) {
      base = (i & 1) ? wb : wa;
      return c0 + 16 * (i >> 1);
    }
    base = wa;
    return r0 + 16 * i;
  };
  const int nmt = uni(min(S::kSub, (mend - m0 + 15) / 16));  // the tile's 16-position tiles that hold rows
  const int nj = uni(nmt > pg ? (nmt - pg + WP - 1) / WP : 0);  // this wave's: pg, pg + WP, ...

  // ---- what this lane fetches: row lr = lane / 8 of an 8-row half, piece (lane % 8) ^ swz(row of the 16) ----
  const int lr = lane >> 3, lq = lane & 7;
  const uint8_t* pw[2][2];  // the two weight tiles this wave brings (2 wave, 2 wave + 1), their halves (rows 0-7, 8-15)
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const uint8_t* base;
    const int row = tile_row(2 * wave + t, base);
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int r = 8 * hh + lr;
      pw[t][hh] = base + (size_t)(row + r) * K + 16 * (lq ^ swz(r));
    }
  }
  const uint8_t* px[WP][2];  // the WP 16-position tiles this wave brings (WP wave, ...)
#pragma unroll
  for (int t = 0; t < WP; ++t)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int r = 8 * hh + lr;
      int pos = m0 + 16 * (WP * wave + t) + r;
      if (pos >= mend) pos = mend - 1;  // a ragged tile re-reads its last row (never stored)
      px[t][hh] = g.aq + (size_t)(g.gather ? g.gather[pos] : pos) * K + 16 * (lq ^ swz(r));
    }
  const float* pxs;  // lanes 0 .. 16 WP - 1: the scale of position 16 WP wave + lane
  {
    int pos = m0 + 16 * WP * wave + (lane & (16 * WP - 1));
    if (pos >= mend) pos = mend - 1;
    pxs = g.as + (size_t)(g.gather ? g.gather[pos] : pos) * KB;
  }
  // (the dynamic segment's address inside LDS: the pointer in the LDS address space is that 32-bit offset)
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
  // the 16-position tiles this wave brings that hold rows: a ragged tile's other slots are neither fetched nor read (a
  // remainder of a few rows otherwise spends a third of its loads on them; gate/up 1.6% and down 0.8% faster at the
  // benchmark's chunk; the same change in the INT4 and MXFP4 kernels, whose loads sit between their MFMAs, gained nothing
  // and is not in them). A wave's loads a turn are then 4, or 4 + 2 nx + 1, which its waits count.
  const int nx = uni(min(WP, max(0, nmt - WP * wave)));
  auto issue = [&](int kb) {  // block kb (clamped: past the end the last block again, into a stage nobody reads) -> its stage
    const int kc = kb < KB ? kb : KB - 1;
    const uint32_t st = lds0 + (uint32_t)(kb % S::kStages) * S::kStageBytes;
    const uint32_t wbase = st + (uint32_t)wave * 4096, xbase = st + S::kStageW + (uint32_t)wave * (2048 * WP);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) dma16(pw[t][hh] + (size_t)(((DIAG & 128) && kb >= S::kStages) ? 0 : kc) * 128, uni(wbase + t * 2048 + hh * 1024));
#pragma unroll
    for (int t = 0; t < WP; ++t) {
      if (t >= nx) break;  // (a ragged tile: nobody reads the 16-position tiles past its end)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) dma16(px[t][hh] + (size_t)(((DIAG & 256) && kb >= S::kStages) ? 0 : kc) * 128, uni(xbase + t * 2048 + hh * 1024));
    }
    if (nx > 0 && lane < 16 * WP) dma4(pxs + kc, uni(st + S::kStageW + S::kStageX + (uint32_t)wave * (64 * WP)));
  };
  // The wave's weight scales: lane l holds those of block l; one value
  // a 16-row tile pair (UP: gate and up; DOWN: all of a wave's rows lie in one 128-row block). They are loaded with
  // ordinary loads and WAITED FOR before any of the loads above is issued (the compiler's own wait for them would
  // otherwise count those as well and drain the pipeline). Rows of up to 64 blocks (8192 k), which the host checks.
  const int srow = (UP ? c0 : r0 + 16 * S::RA * rg) / 128;
  const float* swa = sa + (size_t)srow * KB;
  const float* swb = UP ? sb + (size_t)srow * KB : swa;
  float wsa_l, wsb_l;
  auto load_ws = [&](int kb0) {
    const int kc = min(kb0 + lane, KB - 1);
    wsa_l = swa[kc], wsb_l = swb[kc];
    asm volatile("" : "+v"(wsa_l), "+v"(wsb_l));  // (uses that make the compiler place its wait here)
  };
  PF_STAMP(g, 2);
  load_ws(0);
  PF_STAMP(g, 3);
#pragma unroll
  for (int s = 0; s + 1 < S::kStages; ++s) issue(s);

  // fragment reads: lane (row r16, part) takes pieces 2 part and 2 part + 1 of its row (32 consecutive k)
  const int rd0 = (r16 >> 3) * 1024 + (r16 & 7) * 128 + ((2 * part) ^ swz(r16)) * 16;
  const int rd1 = (r16 >> 3) * 1024 + (r16 & 7) * 128 + ((2 * part + 1) ^ swz(r16)) * 16;
  auto frag = [&](const uint8_t* t) {
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(t + rd0), hi = *reinterpret_cast<const u32x4_t*>(t + rd1);
    return v8i_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };

  v4f_t acc[S::RA][8];
#pragma unroll
  for (int t = 0; t < S::RA; ++t)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[t][j] = v4f_t{0.f, 0.f, 0.f, 0.f};

  auto run = [&](auto nj_c) {
    constexpr int NJ = decltype(nj_c)::value;
    for (int kb = 0; kb < ((DIAG & 32) ? 2 : KB); ++kb) {
      // this wave's loads of block kb have landed (later blocks may be in flight); after the barrier everyone's have, and
      // everyone is done reading the stage of block kb - 1, which the loads of block kb + kStages - 1 now overwrite
      if (S::kStages == 2) wait_loads<0>();
      else if (nx == WP) wait_loads<(S::kStages - 2) * S::kLoads>();
      else if (nx == 0) wait_loads<(S::kStages - 2) * 4>();
      else wait_loads<(S::kStages - 2) * (5 + 2 * (WP - 1))>();  // (WP 2 with one live tile; two stages wait for all anyway)
      if (!(DIAG & 4)) __syncthreads();
      if (kb == 0) PF_STAMP(g, 4);
      if (!(DIAG & 1)) issue(kb + S::kStages - 1);
      if (NJ == 0) continue;
      const float wsa = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wsa_l), kb & 63));
      const float wsb = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wsb_l), kb & 63));
      const uint8_t* st = smem + (size_t)(((DIAG & 16) ? 0 : kb) % S::kStages) * S::kStageBytes;
      const uint8_t* W = st + S::RA * rg * 2048;
      const uint8_t* X = st + S::kStageW + pg * 2048;
      const float* XS = reinterpret_cast<const float*>(st + S::kStageW + S::kStageX) + 16 * pg;
      v8i_t fa[S::RA];
#pragma unroll
      for (int t = 0; t < S::RA; ++t) fa[t] = frag(W + t * 2048);
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const v8i_t fb = frag(X + j * (2048 * WP));
        const float xv = XS[16 * WP * j + r16];
        const float s0 = __fmul_rn(xv, wsa), s1 = __fmul_rn(xv, wsb);
#pragma unroll
        for (int t = 0; t < S::RA; ++t) {
          if (DIAG & 2) {
            acc[t][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa[t], fb, acc[t][j], 0, 0, 0, 0, 0, 0);
            continue;
          }
          v4f_t p;
          if (DIAG & 8) p = v4f_t{__builtin_bit_cast(float, fa[t][0] ^ fb[0]), __builtin_bit_cast(float, fa[t][1] ^ fb[3]), __builtin_bit_cast(float, fa[t][4] ^ fb[4]), __builtin_bit_cast(float, fa[t][7] ^ fb[7])};
          else p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa[t], fb, v4f_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
          const float sc = (UP && (t & 1)) ? s1 : s0;
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[t][j][q] = fmaf(sc, p[q], acc[t][j][q]);
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
  wait_loads<0>();   // the trailing loads into unused stages: nothing may still be landing in LDS from here on
  __syncthreads();   // ... in any wave's part of it: the epilogues reuse the stages
  PF_STAMP(g, 5);
  if (DIAG & 64) {   // (diagnostic: no epilogue; one store keeps the sums alive)
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
    // h = bf16(bf16(silu(bf16 g)) * bf16 u) for the workgroup's 128 channels of every position into an LDS tile
    // [position][256 bytes], 16-byte pieces exchanged by position so that writes and reads spread over the banks; then 16
    // lanes a position: h to memory as whole lines, act_quant over the 128 channels (the scale block of the down
    // projection: amax clamped at 1e-4, scale = amax * f32(1 / 448), e4m3 codes of h / scale clamped to +-448).
    const int I = g.L.I;
    const bool fast = uni(g.fast_act) != 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j >= nj) break;
      const int p = 16 * (pg + WP * j) + r16;  // position within the tile
#pragma unroll
      for (int b = 0; b < S::RA / 2; ++b) {
        uint32_t hb[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float gv = bf16_round(__fmul_rn(acc[2 * b][j][q], s2a)), uv = bf16_round(__fmul_rn(acc[2 * b + 1][j][q], s2b));
          hb[q] = fast ? swiglu_fast_bits(gv, uv) : swiglu_bits(gv, uv);
        }
        const int ch = 16 * (S::RA / 2 * rg + b) + 4 * part;  // first of the lane's four channels (of the workgroup's 128)
        const int piece = (ch >> 3) ^ (p & 15);
        *reinterpret_cast<uint2*>(smem + p * 256 + piece * 16 + (ch & 4) * 2) = make_uint2(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16));
      }
    }
    __syncthreads();
    const int l16 = tid & 15;
    for (int p = tid >> 4; p < 16 * nmt; p += kThreads / 16) {  // (whole rows of 16 lanes take the same turns)
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
      amax = dpp_max<0x141>(amax);
      amax = dpp_max<0x140>(amax);
      amax = fmaxf(amax, 1e-4f);
      const float sc = __fmul_rn(amax, 1.0f / 448.0f), rsc = __builtin_amdgcn_rcpf(sc);
      float qv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) qv[i] = fminf(448.f, fmaxf(-448.f, div_by(v[i], sc, rsc)));
      uint32_t o0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[0], qv[1], 0, false), o1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4], qv[5], 0, false);
      o0 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[2], qv[3], o0, true), o1 = __builtin_amdgcn_cvt_pk_fp8_f32(qv[6], qv[7], o1, true);
      if (pos < mend) {
        *reinterpret_cast<u32x4_t*>(g.h + (size_t)pos * I + c0 + 8 * l16) = hv;
        *reinterpret_cast<uint2*>(g.hq + (size_t)pos * I + c0 + 8 * l16) = make_uint2(o0, o1);
        if (l16 == 0) g.hs[(size_t)pos * (I / 128) + ns] = sc;
      }
    }
  } else {
    // the wave's 16 positions x 32 WP rows of one 16-position tile at a time through its own piece of LDS (2 WP KiB):
    // written as held, read back as whole rows, 8 WP lanes a position
    const int H = g.L.H;
    constexpr int RB = 128 * WP;  // bytes of a position's rows of this wave
    uint8_t* my = smem + wave * (2048 * WP);
    const int row0 = r0 + 16 * S::RA * rg;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j >= nj) break;
#pragma unroll
      for (int t = 0; t < S::RA; ++t) {
        const int c = 4 * t + part;  // the 16-byte piece: rows 16 t + 4 part ...
        *reinterpret_cast<v4f_t*>(my + r16 * RB + ((c & ~7) | ((c ^ r16) & 7)) * 16) = acc[t][j];
      }
#pragma unroll
      for (int i = 0; i < 2 * WP; ++i) {
        const int idx = i * 64 + lane, p = idx / (8 * WP), c = idx % (8 * WP);
        const v4f_t v = *reinterpret_cast<const v4f_t*>(my + p * RB + ((c & ~7) | ((c ^ p) & 7)) * 16);
        const int pos = m0 + 16 * (pg + WP * j) + p;
        if (pos < mend) *reinterpret_cast<v4f_t*>(g.d + (size_t)pos * H + row0 + 4 * c) = v;
      }
    }
  }
  PF_STAMP(g, 6);
}

// The shared expert (tile_e null: tiles of Shape<WP>::kPos rows over [0, nrows)) or one list of tiles of one shape.
template <bool UP, int WP, int DIAG = 0>
__global__ void __launch_bounds__(kThreads) k_gemm(Args g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int NS = UP ? g.L.I / (kWgRows / 2) : g.L.H / kWgRows;
  int tile, ns;
  task_of<true>(NS, tile, ns);
  if (ns >= NS) return;
  int e = -1, m0 = tile * Shape<WP>::kPos, mend = g.nrows;
  if (g.tile_e) {
    if (tile >= *g.ntiles) return;
    e = g.tile_e[tile] & 0xFFFF;
    const int o = g.off[e];
    m0 = o + g.tile_m0[tile], mend = g.off[e + 1];
  } else if (m0 >= mend) {
    return;
  }
  gemm_tile<UP, WP, DIAG>(g, smem, e, m0, mend, ns);
}
// The routed experts' list of both shapes (bit 30 of tile_e: a 256-position tile), an expert's tiles next to each other.
template <bool UP, int DIAG = 0>
__global__ void __launch_bounds__(kThreads) k_gemm_mixed(Args g) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int NS = UP ? g.L.I / (kWgRows / 2) : g.L.H / kWgRows;
  int tile, ns;
  PF_STAMP(g, 0);
  task_of<false>(NS, tile, ns);
  if (ns >= NS || tile >= *g.ntiles) return;
  const int te = g.tile_e[tile], e = te & 0xFFFF;
  const int m0 = g.off[e] + g.tile_m0[tile], mend = g.off[e + 1];
  if (m0 >= 0) PF_STAMP(g, 1);
#ifdef DSGX_PF_TRACE
  if (g.trace && threadIdx.x == 0) g.trace[(size_t)blockIdx.x * 8 + 7] = ((te >> 30) ? 0x10000 : 0) | min(mend - m0, (te >> 30) ? 256 : 128);
#endif
  if (te >> 30) gemm_tile<UP, 2, DIAG>(g, smem, e, m0, mend, ns);
  else gemm_tile<UP, 1, DIAG>(g, smem, e, m0, mend, ns);
}

}  // namespace pf8
}  // namespace dsgx
