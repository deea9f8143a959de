// The prefill expert step for a chunk of T token rows: the gfx950 counterpart of the reference's gx::moe_prefill
// (altar1-4xgx10-switchless/engine/experts/prefill.cu:94-150 bucketing, :337-352 / :772-972 the grouped GEMMs and the
// combine, :1056-1116 the host sequence), with DeepSeek's FP8 activation contract (ds41f-4xgx10-switchless/ref/
// torchref/kernel.py:56-125: activations quantised per row and 128 k to e4m3 with an f32 scale; per 128-k block the
// e4m3 x e4m3 products are summed in f32 from zero and added as fma(x_scale * w_scale, partial, acc)).
//
// Phases (dsgx_prefill_cfg::phases):
//   1  bucket   picks counted per expert, offsets scanned, rows scattered into expert buckets in token order, the 128-row
//               tiles listed, each row's picks sorted by expert id (rpos, re, and the combine's factor s2_down * w)
//   2  up       x quantised; one grouped GEMM over the tiles: gate and up together, h = bf16(silu(bf16 g) * bf16 u)
//   4  down     h quantised; grouped GEMM, each pick's f32 result row kept (d)
//   8  combine  yr[t] = sum over the row's picks in expert-id order of fma(s2 * w, d, acc) (decode.cu:526-566's order)
//   16 shared   the fused FP8 shared expert on all T rows with the same two GEMMs -> ys
// The FP8-activation GEMMs run on v_mfma_f32_16x16x128_f8f6f4 (one instruction a 128-k scale block), the bf16-activation
// ones on v_mfma_f32_16x16x32_bf16: weights are the A operand (rows n), activations the B operand, so a lane's four
// accumulators of a 16 x 16 tile belong to ONE token row and the block's combined scale is one value a lane.
#include <cstdlib>

#include "abi_internal.h"
#include "common.cuh"
#include "pf_gemm_fp8.cuh"
#include "pf_gemm_mx.cuh"
#include "pf_gemm_i4.cuh"

#ifdef DSGX_TRACE
extern "C" unsigned long long* dsgx_trace_buf();
#endif
namespace dsgx {
namespace {

typedef int v8i_t __attribute__((ext_vector_type(8)));
typedef float v16f_t __attribute__((ext_vector_type(16)));

// D (32 x 32, f32) += A (32 x 64, e4m3) B^T (32 x 64, e4m3): v_mfma_f32_32x32x64_f8f6f4. A lane holds 32 consecutive k
// of one row of A and of one row of B: row lane % 32, k = 32 (lane / 32) ... + 31, as eight dwords. The result's
// register r of lane l is D[8 (r / 4) + 4 (l / 32) + r % 4][l % 32].
__device__ __forceinline__ v16f_t mfma_fp8(v8i_t a, v8i_t b, v16f_t c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);  // (both scales 0: the unscaled form)
}

typedef float v4f_t __attribute__((ext_vector_type(4)));
// D (16 x 16, f32) += A (16 x 128, e4m3) B^T (16 x 128, e4m3): v_mfma_f32_16x16x128_f8f6f4. A lane holds 32 k of one row
// of A and of one row of B (row lane % 16, k-part lane / 16: which 32 k of the 128 a part holds does not matter as long
// as A and B agree). The result's register r of lane l is D[4 (l / 16) + r][l % 16].
__device__ __forceinline__ v4f_t mfma_fp8_k128(v8i_t a, v8i_t b, v4f_t c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
// the probe of the 16 x 16 x 128 form: a lane's 32 bytes are the 16 bytes at part * 16 and those at 64 + part * 16 of
// its row (the k order the prefill kernels use, so that four lanes read 64 contiguous bytes of a row an instruction)
__global__ void __launch_bounds__(64) k_probe_mfma_fp8_k128(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ raw) {
  const int l = threadIdx.x, row = l % 16, part = l / 16;
  auto frag = [&](const uint8_t* M) {
    const uint4 lo = *reinterpret_cast<const uint4*>(M + row * 128 + part * 16), hi = *reinterpret_cast<const uint4*>(M + row * 128 + 64 + part * 16);
    return v8i_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };
  v4f_t c = {};
  c = mfma_fp8_k128(frag(A), frag(B), c);
#pragma unroll
  for (int r = 0; r < 4; ++r) raw[l * 16 + r] = c[r];
}

__global__ void __launch_bounds__(64) k_probe_mfma_fp8(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, float* __restrict__ raw) {
  const int l = threadIdx.x;
  const v8i_t a = *reinterpret_cast<const v8i_t*>(A + (l % 32) * 64 + (l / 32) * 32);
  const v8i_t b = *reinterpret_cast<const v8i_t*>(B + (l % 32) * 64 + (l / 32) * 32);
  v16f_t c = {};
  c = mfma_fp8(a, b, c);
#pragma unroll
  for (int r = 0; r < 16; ++r) raw[l * 16 + r] = c[r];
}

// ---- the workspace -------------------------------------------------------------------------------------------------------
constexpr int kDefaultTileOrder = 0;  // dsgx_prefill_cfg::tile_order = -1
constexpr int kTile = 128;  // rows of a tile (token positions) and weight rows a workgroup
constexpr int kRowBlock = 128;  // token rows a workgroup of the bucketing kernels
struct PfLayout {
  size_t cnt, off, ntiles, tile_e, tile_m0, perm, pickpos, posw, rpos, re, rk, xq, xs, h, hq, hs, hsh, hshq, hshs, d, bcnt, boff, bmask, total;
  size_t nbig, big_e, big_m0, nsmall, small_e, small_m0;  // the FP8 kernels' lists: 256-position tiles, and the experts' remainders
  size_t nmix, mix_e, mix_m0;                             // ... and the two merged, in expert order
  size_t ord_e, ord_m0;                                   // ... and merged with the experts by falling count, remainders spread evenly
  int P, max_tiles, max_big;
};
PfLayout pf_layout(const dsgx_layer_w* L, int T) {
  PfLayout o{};
  const size_t H = L->H, I = L->I, E = L->E, P = (size_t)T * L->topk;
  o.P = (int)P;
  o.max_tiles = (int)(P / kTile + E);
  size_t at = 0;
  auto take = [&](size_t bytes) { const size_t a = at; at += align256(bytes); return a; };
  o.cnt = take(E * 4), o.off = take((E + 1) * 4), o.ntiles = take(4);
  o.tile_e = take((size_t)o.max_tiles * 4), o.tile_m0 = take((size_t)o.max_tiles * 4);
  o.max_big = (int)(P / 256 + E);
  o.nbig = take(4), o.big_e = take((size_t)o.max_big * 4), o.big_m0 = take((size_t)o.max_big * 4);
  o.nsmall = take(4), o.small_e = take(E * 4), o.small_m0 = take(E * 4);
  o.nmix = take(4), o.mix_e = take((size_t)(o.max_big + E) * 4), o.mix_m0 = take((size_t)(o.max_big + E) * 4);
  o.ord_e = take((size_t)(o.max_big + E) * 4), o.ord_m0 = take((size_t)(o.max_big + E) * 4);
  o.perm = take(P * 4), o.pickpos = take(P * 4), o.posw = take(P * 4), o.rpos = take(P * 4), o.re = take(P * 4), o.rk = take(P * 4);
  o.xq = take((size_t)T * H), o.xs = take((size_t)T * (H / 128) * 4);
  o.h = take(P * I * 2), o.hq = take(P * I), o.hs = take(P * (I / 128) * 4);
  o.hsh = take((size_t)T * I * 2), o.hshq = take((size_t)T * I), o.hshs = take((size_t)T * (I / 128) * 4);
  o.d = take(P * H * 4);
  const size_t NB = ((size_t)T + kRowBlock - 1) / kRowBlock;  // the bucketing's row blocks
  o.bcnt = take(NB * E * 4), o.boff = take(NB * E * 4), o.bmask = take(NB * E * 16);
  o.total = at;
  return o;
}

// ---- bucketing -----------------------------------------------------------------------------------------------------------
// Positions inside an expert's bucket follow the picks' order (row-major over [T][topk]); a row picks an expert at most
// once, so that is the order of the rows. Three launches:
//   k_pf_mask   a workgroup a block of 128 rows: for every expert the 128-bit mask of the block's rows that picked it
//               (LDS atomics), stored with its population count;
//   k_pf_scan   one workgroup, a thread an expert: the blocks' counts summed in block order (each block's offset inside
//               the bucket), the buckets' offsets and the list of 128-row tiles in expert order by two scans;
//   k_pf_place  a workgroup a block, a thread a pick: position = bucket offset + block offset + rows of the block below
//               this one in the expert's mask; and, per row, its picks in expert-id order (ids are distinct in a row):
//               expert, bucket position, the combine's factor s2 * w.
__global__ void __launch_bounds__(256) k_pf_mask(const int* __restrict__ idx, int T, int topk, int E, int* __restrict__ bcnt,
                                                 uint32_t* __restrict__ bmask) {
  __shared__ uint32_t mask[DSGX_MAX_EXPERTS * 4];
  const int b = blockIdx.x, t0 = b * kRowBlock, rows = min(kRowBlock, T - t0);
  for (int i = threadIdx.x; i < E * 4; i += blockDim.x) mask[i] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < rows * topk; i += blockDim.x) {
    const int r = i / topk, e = idx[(size_t)t0 * topk + i];
    atomicOr(&mask[e * 4 + (r >> 5)], 1u << (r & 31));
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    const uint4 m = *reinterpret_cast<const uint4*>(&mask[e * 4]);
    bcnt[(size_t)b * E + e] = __popc(m.x) + __popc(m.y) + __popc(m.z) + __popc(m.w);
    *reinterpret_cast<uint4*>(&bmask[((size_t)b * E + e) * 4]) = m;
  }
}
// The FP8 kernels' two lists: an expert of c rows gives c / 256 tiles of 256 positions, one more if over 128 rows are left,
// else (if any are left) one tile of up to 128 positions.
struct TileLists {
  int *ntiles, *tile_e, *tile_m0;     // all rows in 128-position tiles
  int *nbig, *big_e, *big_m0;         // 256-position tiles
  int *nsmall, *small_e, *small_m0;   // the remainders of up to 128 positions
  int *nmix, *mix_e, *mix_m0;         // both, in expert order (expert | 1 << 30 for a 256-position tile)
  int *ord_e, *ord_m0;                // both (nmix of them), the experts by falling count (see k_pf_scan)
};
__global__ void __launch_bounds__(DSGX_MAX_EXPERTS) k_pf_scan(const int* __restrict__ bcnt, int NB, int E, int* __restrict__ boff,
                                                              int* __restrict__ cnt, int* __restrict__ off, TileLists tl, int order) {
  __shared__ int sa[DSGX_MAX_EXPERTS], sb[DSGX_MAX_EXPERTS], sc[DSGX_MAX_EXPERTS], sd[DSGX_MAX_EXPERTS];
  const int e = threadIdx.x;
  int c = 0;
  if (e < E) {
    int b = 0;
    for (; b + 8 <= NB; b += 8) {  // (eight blocks' counts requested together: the loop is one round trip a pass)
      int v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = bcnt[(size_t)(b + i) * E + e];
#pragma unroll
      for (int i = 0; i < 8; ++i) boff[(size_t)(b + i) * E + e] = c, c += v[i];
    }
    for (; b < NB; ++b) {
      const int v = bcnt[(size_t)b * E + e];
      boff[(size_t)b * E + e] = c;
      c += v;
    }
  }
  const int nt = (c + kTile - 1) / kTile;
  const int rem = c % 256, nbig = c / 256 + (rem > 128 ? 1 : 0), nsmall = rem > 0 && rem <= 128 ? 1 : 0;
  sa[e] = e < E ? c : 0, sb[e] = e < E ? nt : 0, sc[e] = e < E ? nbig : 0, sd[e] = e < E ? nsmall : 0;
  __syncthreads();
  for (int d = 1; d < DSGX_MAX_EXPERTS; d <<= 1) {  // inclusive scans of the counts and of the tile counts
    const int va = e >= d ? sa[e - d] : 0, vb = e >= d ? sb[e - d] : 0, vc = e >= d ? sc[e - d] : 0, vd = e >= d ? sd[e - d] : 0;
    __syncthreads();
    sa[e] += va, sb[e] += vb, sc[e] += vc, sd[e] += vd;
    __syncthreads();
  }
  if (e < E) {
    cnt[e] = c;
    off[e] = sa[e] - c;
    if (e == E - 1) off[E] = sa[e], *tl.ntiles = sb[e], *tl.nbig = sc[e], *tl.nsmall = sd[e];
    const int t0 = sb[e] - nt;
    for (int i = 0; i < nt; ++i) tl.tile_e[t0 + i] = e, tl.tile_m0[t0 + i] = i * kTile;
    const int b0 = sc[e] - nbig;
    for (int i = 0; i < nbig; ++i) tl.big_e[b0 + i] = e, tl.big_m0[b0 + i] = i * 256;
    if (nsmall) tl.small_e[sd[e] - 1] = e, tl.small_m0[sd[e] - 1] = (c / 256) * 256;
  }
  __syncthreads();
  const int nb = sc[DSGX_MAX_EXPERTS - 1], nsm = sd[DSGX_MAX_EXPERTS - 1];
  // The merged list, in expert order: an expert's 256-position tiles, then its remainder. Neighbours in the list run at
  // about the same time on one XCD (pf8::task_of), so part of what an expert's tiles stream, each in full, comes out of
  // that XCD's L2: 12% fewer bytes from HBM for gate/up, 19% for down, than with the remainders spread evenly among the
  // big tiles (measured; the time differs by 1% only: the stream is not what bounds these launches).
  if (e < E) {
    const int p0 = (sc[e] - nbig) + (sd[e] - nsmall);
    for (int i = 0; i < nbig; ++i) tl.mix_e[p0 + i] = e | (1 << 30), tl.mix_m0[p0 + i] = i * 256;
    if (nsmall) tl.mix_e[p0 + nbig] = e, tl.mix_m0[p0 + nbig] = (c / 256) * 256;
    if (!order) {  // (the second list is always a valid one: a later call may name it whatever this call was told)
      for (int i = 0; i < nbig; ++i) tl.ord_e[p0 + i] = e | (1 << 30), tl.ord_m0[p0 + i] = i * 256;
      if (nsmall) tl.ord_e[p0 + nbig] = e, tl.ord_m0[p0 + nbig] = (c / 256) * 256;
    }
  }
  if (e == 0) *tl.nmix = nb + nsm;
  // The same tiles in the order of the reference's prefill_tuning tord (ds41f-4xgx10-switchless/engine/kernels/prefill.cu:
  // 658-668: the most-picked experts' tiles with those of the least-picked between them): the experts by falling count
  // (ties by id), their 256-position tiles as one list B and their remainders as one list S, merged so that both lists
  // run out together (B's tile k at key (k + 1/2) / |B|, S's tile j at (j + 1/2) / |S|, by rising key, B first on a tie).
  // A 256-position tile is bound by the matrix unit and a remainder by the weight stream, so at any time the chip runs
  // a mix of the two. The order of the sums does not depend on the list's order.
  if (!order) return;  // (the same for every thread)
  __syncthreads();
  sa[e] = e < E ? c : -1;
  __syncthreads();
  int rank = 0, rank2 = 0;  // by falling count; by falling remainder (order 2's list of remainders)
  {
    const int ce = e < E ? c : -1, re = (e < E && nsmall) ? rem : -1;
    for (int j = 0; j < DSGX_MAX_EXPERTS; ++j) {
      const int cj = sa[j];
      const int rj = (cj >= 0 && cj % 256 > 0 && cj % 256 <= 128) ? cj % 256 : -1;
      rank += (cj > ce) || (cj == ce && j < e);
      rank2 += (rj > re) || (rj == re && j < e);
    }
  }
  __syncthreads();
  sb[rank] = e < E ? nbig : 0, sd[order == 2 ? rank2 : rank] = e < E ? nsmall : 0;
  __syncthreads();
  for (int d = 1; d < DSGX_MAX_EXPERTS; d <<= 1) {  // inclusive scans in rank order
    const int vb = e >= d ? sb[e - d] : 0, vd = e >= d ? sd[e - d] : 0;
    __syncthreads();
    sb[e] += vb, sd[e] += vd;
    __syncthreads();
  }
  if (e < E) {
    const long long NB_ = nb, NS_ = nsm;
    const int k0 = sb[rank] - nbig, j0 = sd[order == 2 ? rank2 : rank] - nsmall;
    for (int i = 0; i < nbig; ++i) {
      const long long k = k0 + i;
      long long before = NS_ ? ((2 * k + 1) * NS_ + NB_ - 1) / (2 * NB_) : 0;  // S tiles of a key below this one's
      if (before > NS_) before = NS_;
      if (order == 2) before = 0;  // every 256-position tile before every remainder
      tl.ord_e[k + before] = e | (1 << 30), tl.ord_m0[k + before] = i * 256;
    }
    if (nsmall) {
      const long long j = j0;
      long long before = NB_ ? ((2 * j + 1) * NB_ + NS_) / (2 * NS_) : 0;      // B tiles of a key up to this one's
      if (before > NB_ || order == 2) before = NB_;
      tl.ord_e[j + before] = e, tl.ord_m0[j + before] = (c / 256) * 256;
    }
  }
}
__global__ void __launch_bounds__(256) k_pf_place(const int* __restrict__ idx, const float* __restrict__ w, int T, int topk, int E,
                                                  const int* __restrict__ off, const int* __restrict__ boff,
                                                  const uint32_t* __restrict__ bmask, const dsgx_mat_desc* __restrict__ desc,
                                                  int* __restrict__ perm, int* __restrict__ pickpos, int* __restrict__ rpos,
                                                  int* __restrict__ re, float* __restrict__ rk, float* __restrict__ posw) {
  __shared__ uint32_t mask[DSGX_MAX_EXPERTS * 4];
  __shared__ int base[DSGX_MAX_EXPERTS];
  const int b = blockIdx.x, t0 = b * kRowBlock, rows = min(kRowBlock, T - t0);
  for (int i = threadIdx.x; i < E * 4; i += blockDim.x) mask[i] = bmask[(size_t)b * E * 4 + i];
  for (int e = threadIdx.x; e < E; e += blockDim.x) base[e] = off[e] + boff[(size_t)b * E + e];
  __syncthreads();
  for (int i = threadIdx.x; i < rows * topk; i += blockDim.x) {
    const int r = i / topk, k = i % topk, t = t0 + r, e = idx[(size_t)t * topk + k];
    int below = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t m = mask[e * 4 + q];
      below += q < (r >> 5) ? __popc(m) : q == (r >> 5) ? __popc(m & ((1u << (r & 31)) - 1)) : 0;
    }
    const int pos = base[e] + below;
    perm[pos] = t, pickpos[(size_t)t * topk + k] = pos;
    int rank = 0;
    for (int j = 0; j < topk; ++j) rank += idx[(size_t)t * topk + j] < e;
    const size_t o = (size_t)t * topk + rank;
    const float wv = w[(size_t)t * topk + k];
    re[o] = e, rpos[o] = pos, rk[o] = desc ? __fmul_rn(desc[(size_t)e * 3 + 2].s2, wv) : wv;
    if (posw) posw[pos] = wv;  // (DeepSeek's layers apply the routing weight to h, position by position)
  }
}

// ---- the grouped GEMMs ---------------------------------------------------------------------------------------------------
// FP8 activations (e4m3 MFMA): pf_gemm_fp8.cuh. bf16 activations (bf16 MFMA): k_pf_gemm16 below.
constexpr int kWgRows = 256;                     // weight rows a workgroup (UP: 128 channels)
constexpr int kGemmThreads = 512;

// Workgroup -> (position tile, group of weight rows). Workgroups go to the eight XCDs round robin by their number, and
// each XCD has an L2 of its own: what two workgroups share is read from memory once only if they run on the same XCD at
// about the same time. So the tasks are cut into blocks of kMapTiles consecutive tiles (mostly one expert's: tiles are in
// expert order) x kMapNs row groups, and a block's 32 tasks get 32 consecutive workgroup numbers OF ONE XCD (numbers
// x, x + 8, x + 16, ...): they start together and walk K together, a weight line is then fetched by one of the
// kMapTiles workgroups that use it and an activation line by one of kMapNs, the others hit L2 (measured: 115 GB/s a CU
// from L2, 28 from beyond).
constexpr int kMapTiles = 4, kMapNs = 8, kXcds = 8;
__host__ __device__ inline unsigned pf_grid(int tiles, int NS) {
  const int blocks = ((tiles + kMapTiles - 1) / kMapTiles) * ((NS + kMapNs - 1) / kMapNs);
  return (unsigned)((blocks + kXcds - 1) / kXcds) * kXcds * (kMapTiles * kMapNs);
}
__device__ __forceinline__ void pf_task(int NS, int& tile, int& ns) {
  const int x = blockIdx.x % kXcds, j = blockIdx.x / kXcds;
  const int b = (j / (kMapTiles * kMapNs)) * kXcds + x, i = j % (kMapTiles * kMapNs);
  const int NG = (NS + kMapNs - 1) / kMapNs;
  tile = (b / NG) * kMapTiles + i / kMapNs;
  ns = (b % NG) * kMapNs + i % kMapNs;
}

// ---- the grouped GEMM with bf16 activations (INT4 layers, and their BF16 shared expert) -----------------------------
// The same streaming structure for the altar-1 contract (engine/experts/prefill.cu:337-352, 772-831): activations stay
// bf16, a weight is the bf16 value W = bf16((u - u_z) s) (INT4; decoded in registers by the decode kernels' routine) or
// the stored bf16 (the shared expert), products are summed in f32 by v_mfma_f32_16x16x32_bf16, whose accumulators the
// MFMA itself carries across K (no per-block scale here: the scales are inside W).
// A 128-k block is four MFMAs (j = 0..3) a 16-row tile. INT4: a lane's 16 bytes are the 32 values of ONE scale group:
// lane (row, part) holds k = 32 part + 8 j + [0, 8) for MFMA j (four lanes a row: 64 contiguous bytes an instruction),
// one scale and one zero-point word a lane and block. BF16: k = 32 j + 8 part + [0, 8), one 16-byte load an MFMA.
// The activation panel in LDS is in fragment order for the same k map: piece (tile mt, j, lane) at 16 ((4 mt + j) 64 + lane).
typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
constexpr int kPanel16 = kTile * 256;  // bytes of one bf16 activation panel (128 positions x 128 k)
constexpr int kStages16 = 3;

struct Gemm16Args {
  const uint16_t* x;   // activations bf16 [rows][K]
  const int* gather;   // position -> activation row (null: the position itself)
  const int* tile_e;   // (null: the shared expert on rows [0, nrows))
  const int* tile_m0;
  const int* ntiles;
  const int* off;
  int nrows;
  dsgx_layer_w L;
  uint16_t* h;         // UP: h bf16 [position][I]
  float* d;            // DOWN: f32 [position][H]
};

// WF: the weights' format (DSGX_FMT_INT4_G32: the routed experts; DSGX_FMT_BF16: the shared expert, gate/up interleaved;
// DSGX_FMT_FP8_B128: e4m3 experts or shared expert with bf16 activations, the reference engine's own prefill contract
// for FP8 weights, prefill.cu:337-352: per 128-k block the bf16 x bf16 products summed from zero, acc = fma(S, sum, acc))
template <bool UP, int WF>
__global__ void __launch_bounds__(kGemmThreads) k_pf_gemm16(Gemm16Args g) {
  extern __shared__ uint8_t smem[];
  constexpr bool I4 = WF == DSGX_FMT_INT4_G32, F8 = WF == DSGX_FMT_FP8_B128;
  const int K = UP ? g.L.H : g.L.I, N = UP ? g.L.I : g.L.H, KB = K / 128;
  const int NS = UP ? g.L.I / (kWgRows / 2) : g.L.H / kWgRows;
  int tile, ns;
  pf_task(NS, tile, ns);
  if (ns >= NS) return;
  int e = -1, m0 = tile * kTile, mend = g.nrows;
  if (g.tile_e) {
    if (tile >= *g.ntiles) return;
    e = g.tile_e[tile];
    const int o = g.off[e];
    m0 = o + g.tile_m0[tile], mend = g.off[e + 1];
  } else if (m0 >= mend) {
    return;
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6), r16 = lane & 15, part = lane >> 4;
  // loads are issued with lane l on row l / 4, piece l % 4 (four consecutive lanes read 64 contiguous bytes), weights are
  // then moved to the MFMA's lane order (row l % 16, part l / 16) by a cross-lane permute, activations by their LDS slot
  const int lrow = lane >> 2, lq = lane & 3;
  const int perm_addr = 4 * (4 * r16 + part);
  const int nmt = uni(min(8, (mend - m0 + 15) / 16));  // the tile's 16-position tiles that hold rows
  const int n0 = UP ? ns * (kWgRows / 2) + 16 * wave : ns * kWgRows + 32 * wave;  // UP: first channel; DOWN: first row
  // the lane's weight row of each of the wave's two tiles
  const uint8_t* pw[2];
  const uint8_t* ps[2] = {nullptr, nullptr};
  const uint8_t* pz[2] = {nullptr, nullptr};
  uint32_t zsh[2] = {0, 0};
  float s2a = 1.f, s2b = 1.f;
  if (I4) {
    const dsgx_mat_desc* d = g.L.desc + (size_t)e * 3;
    const int G = K / 32;
    const size_t soff = ((size_t)N * K / 2 + 255) / 256 * 256, zoff = soff + ((size_t)N * G * 2 + 255) / 256 * 256;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const uint8_t* base = g.L.pool + d[UP ? t : 2].off;
      const int ln = UP ? n0 + lrow : n0 + 16 * t + lrow;  // the row this lane loads codes of
      const int n = UP ? n0 + r16 : n0 + 16 * t + r16;       // the row it holds after the permute (scales: loaded as held)
      pw[t] = base + (size_t)ln * (K / 2) + lq * 16;
      ps[t] = base + soff + ((size_t)n * G + part) * 2;
      pz[t] = base + zoff + ((size_t)(n >> 3) * G + part) * 4;
      zsh[t] = 4 * (n & 7);
    }
    if (UP) s2a = d[0].s2, s2b = d[1].s2;
  } else if (F8) {
    const uint8_t *wa, *wb;
    const float *sa, *sb;
    if (e < 0) {
      if (UP) wa = g.L.sh.g, sa = g.L.sh.gs, wb = g.L.sh.u, sb = g.L.sh.us;
      else wa = wb = g.L.sh.d, sa = sb = g.L.sh.ds;
    } else {
      const dsgx_mat_desc* d = g.L.desc + (size_t)e * 3;
      if (UP) wa = g.L.pool + d[0].off, wb = g.L.pool + d[1].off, s2a = d[0].s2, s2b = d[1].s2;
      else wa = wb = g.L.pool + d[2].off;
      const size_t NK = (size_t)g.L.H * g.L.I;
      sa = reinterpret_cast<const float*>(wa + (NK + 255) / 256 * 256);
      sb = reinterpret_cast<const float*>(wb + (NK + 255) / 256 * 256);
    }
    pw[0] = wa + (size_t)(n0 + lrow) * K + lq * 16;
    pw[1] = (UP ? wb + (size_t)(n0 + lrow) * K : wa + (size_t)(n0 + 16 + lrow) * K) + lq * 16;
    ps[0] = reinterpret_cast<const uint8_t*>(sa + (size_t)(n0 / 128) * KB);  // the tiles' scale rows (32 rows: one 128-row block)
    ps[1] = UP ? reinterpret_cast<const uint8_t*>(sb + (size_t)(n0 / 128) * KB) : ps[0];
  } else {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      // shared expert: gate row c is row 2 c of bgu, up row c is row 2 c + 1; down rows plain
      const size_t row = UP ? 2 * (size_t)(n0 + lrow) + t : (size_t)(n0 + 16 * t + lrow);
      pw[t] = reinterpret_cast<const uint8_t*>(UP ? g.L.sh.bgu : g.L.sh.bd) + row * K * 2 + lq * 16;
    }
  }
  // activation staging: wave w brings the 16 positions 16 w ..., the lane the four 16-byte pieces of its fragments
  const uint8_t* px;
  {
    int pos = m0 + 16 * wave + lrow;
    if (pos >= mend) pos = mend - 1;
    px = reinterpret_cast<const uint8_t*>(g.x) + (size_t)(g.gather ? g.gather[pos] : pos) * K * 2 + lq * 16;
  }
  // Activation load i of a lane is the 16-byte piece c = 4 i + lq of its row's block (k = 8 c ...): the piece of MFMA j,
  // part p with c = 4 p + j (INT4 map: k = 32 p + 8 j) or c = 4 j + p (BF16 map: k = 32 j + 8 p).
  // FP8 map: a lane's 32 codes are the 16 at 16 p and the 16 at 64 + 16 p of the block: k = 64 (j / 2) + 16 p + 8 (j % 2), c = k / 8.
  auto slot_of = [&](int i) {
    const int c = 4 * i + lq;
    const int j = I4 ? c & 3 : F8 ? 2 * (c >> 3) + (c & 1) : c >> 2, p = I4 ? c >> 2 : F8 ? (c >> 1) & 3 : c & 3;
    return ((4 * wave + j) * 64 + p * 16 + lrow) * 16;
  };

  v4f_t acc[2][8];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) acc[t][mt] = v4f_t{};

  constexpr int kRing16 = I4 || F8 ? 3 : 2;
  struct WRegs {
    u32x4_t v[I4 ? 1 : F8 ? 2 : 4];
    uint32_t s, z;
  };
  // FP8: the wave's weight scales, lane l holding those of block kb0 + l for the 64 blocks from kb0 (a load inside the
  // turn would be a wait for every load before it)
  float ws_l[2] = {1.f, 1.f};
  auto load_ws = [&](int kb0) {
    if (F8) {
      const int kc = min(kb0 + lane, KB - 1);
      ws_l[0] = reinterpret_cast<const float*>(ps[0])[kc], ws_l[1] = reinterpret_cast<const float*>(ps[1])[kc];
    }
  };
  load_ws(0);
  WRegs ra[kRing16][2];
  auto load_a = [&](int slot, int kb) {
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (I4) {
        const uint8_t* p = pin_after(pw[t] + (size_t)kc * 64, acc[t][0][0]);
        ra[slot][t].v[0] = ldg_stream(p);
        ra[slot][t].s = ldg_u16(ps[t] + (size_t)kc * 8);
        ra[slot][t].z = ldg_u32(pz[t] + (size_t)kc * 16);
      } else if (F8) {
        const uint8_t* p = pin_after(pw[t] + (size_t)kc * 128, acc[t][0][0]);
        ra[slot][t].v[0] = *reinterpret_cast<const DSGX_GLOBAL u32x4_t*>((uintptr_t)p);
        ra[slot][t].v[F8 ? 1 : 0] = *reinterpret_cast<const DSGX_GLOBAL u32x4_t*>((uintptr_t)(p + 64));
      } else {
        const uint8_t* p = pin_after(pw[t] + (size_t)kc * 256, acc[t][0][0]);
#pragma unroll
        for (int j = 0; j < 4; ++j) ra[slot][t].v[I4 || F8 ? 0 : j] = ldg_stream(p + 64 * j);
      }
    }
  };
  // The activations of a block wait kHold16 turns in registers between their loads and their LDS writes (the memory
  // latency is several turns long, and a wait for one load is a wait for every load issued before it).
  constexpr int kHold16 = F8 ? 2 : 3;
  struct XRegs16 {
    u32x4_t v[4];
  };
  auto fetch_x = [&](XRegs16& r, int kb) {
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int j = 0; j < 4; ++j) r.v[j] = *reinterpret_cast<const u32x4_t*>(px + (size_t)kc * 256 + 64 * j);
  };
  auto stash_x = [&](const XRegs16& r, int stage) {
    uint8_t* B = smem + (size_t)stage * kPanel16;
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4_t*>(B + slot_of(j)) = r.v[j];
  };
  auto compute = [&](int slot, int stage, int kb) {
    const uint8_t* B = smem + (size_t)stage * kPanel16;
    float wsc[2] = {1.f, 1.f};
    if (F8) {
      if ((kb & 63) == 0 && kb > 0) load_ws(kb);
#pragma unroll
      for (int t = 0; t < 2; ++t) wsc[t] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ws_l[t]), kb & 63));
    }
    // the wave's two A tiles of the block as bf16 fragments
    u32x4_t fa[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (I4) {
        const float sc = bf16_bits_to_f32(ra[slot][t].s);
        const float nzs = -((float)((ra[slot][t].z >> zsh[t]) & 15u) * sc);
        auto mv = [&](uint32_t v) { return (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)v); };
        const u32x4_t wl = keep_whole(ra[slot][t].v[0]);
        const u32x4_t w = u32x4_t{mv(wl.x), mv(wl.y), mv(wl.z), mv(wl.w)};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t o[4];
          i4x8_to_bf16(j == 0 ? w.x : j == 1 ? w.y : j == 2 ? w.z : w.w, sc, nzs, o);
          fa[t][j] = u32x4_t{o[0], o[1], o[2], o[3]};
        }
      } else if (F8) {
        auto mv = [&](uint32_t v) { return (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)v); };
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const u32x4_t wl = keep_whole(ra[slot][t].v[F8 ? h : 0]);
          const u32x4_t w = u32x4_t{mv(wl.x), mv(wl.y), mv(wl.z), mv(wl.w)};
          uint32_t o[4];
          fp8x8_to_bf16(w.x, w.y, o);
          fa[t][2 * h] = u32x4_t{o[0], o[1], o[2], o[3]};
          fp8x8_to_bf16(w.z, w.w, o);
          fa[t][2 * h + 1] = u32x4_t{o[0], o[1], o[2], o[3]};
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          auto mv = [&](uint32_t v) { return (uint32_t)__builtin_amdgcn_ds_bpermute(perm_addr, (int)v); };
          const u32x4_t wl = keep_whole(ra[slot][t].v[I4 || F8 ? 0 : j]);
          fa[t][j] = u32x4_t{mv(wl.x), mv(wl.y), mv(wl.z), mv(wl.w)};
        }
      }
    }
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
      if (mt >= nmt) break;  // (a ragged tile's 16-position tiles past its end: most experts hold fewer than 128 rows)
      u32x4_t fb[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) fb[j] = *reinterpret_cast<const u32x4_t*>(B + ((4 * mt + j) * 64 + lane) * 16);
      if (F8) {  // the block's sum from zero, then the scaled add
        v4f_t p[2] = {v4f_t{}, v4f_t{}};
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < 2; ++t)
            p[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, fa[t][j]), __builtin_bit_cast(v8bf_t, fb[j]), p[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[t][mt][q] = fmaf(wsc[t], p[t][q], acc[t][mt][q]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < 2; ++t)
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, fa[t][j]), __builtin_bit_cast(v8bf_t, fb[j]),
                                                                 acc[t][mt], 0, 0, 0);
      }
    }
  };
  // prologue
#pragma unroll
  for (int d = 0; d < kRing16; ++d) load_a(d, d);
  XRegs16 rx[kHold16];
  {
    XRegs16 t0, t1;
    fetch_x(t0, 0), fetch_x(t1, 1);
#pragma unroll
    for (int v = 0; v < kHold16; ++v) fetch_x(rx[v], 2 + v);
    stash_x(t0, 0), stash_x(t1, 1);
  }
  __syncthreads();
  // turn kb: the activations of block kb + 2 (loaded kHold16 turns ago; set kb % kHold16) go to their stage (last read a
  // turn ago) and the loads of block kb + 2 + kHold16 are issued in their place; compute block kb; the weight loads of
  // block kb + ring issued in its place. (Unrolled over a common multiple of the rotations.)
  constexpr int kUnroll = 6;
  static_assert(kUnroll % kRing16 == 0 && kUnroll % kStages16 == 0 && kUnroll % kHold16 == 0, "unroll");
  for (int kb0 = 0; kb0 < KB; kb0 += kUnroll) {
#pragma unroll
    for (int v = 0; v < kUnroll; ++v) {
      const int kb = kb0 + v;
      if (kb >= KB) break;
      stash_x(rx[v % kHold16], (v + 2) % kStages16);
      fetch_x(rx[v % kHold16], kb + 2 + kHold16);
      compute(v % kRing16, v % kStages16, kb);
      load_a(v % kRing16, kb + kRing16);
      __syncthreads();
    }
  }
  // epilogue: register q of lane l is weight row 4 (l / 16) + q of the 16-row tile, position l % 16 of the 16 positions
  if (UP) {
    const int I = g.L.I;
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
      const int pos = m0 + 16 * mt + r16;
      if (pos >= mend) continue;
      uint32_t hb[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        hb[q] = swiglu_bits(bf16_round(__fmul_rn(acc[0][mt][q], s2a)), bf16_round(__fmul_rn(acc[1][mt][q], s2b)));
      *reinterpret_cast<uint2*>(g.h + (size_t)pos * I + n0 + 4 * part) = make_uint2(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16));
    }
  } else {
    const int H = g.L.H;
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
      const int pos = m0 + 16 * mt + r16;
      if (pos >= mend) continue;
#pragma unroll
      for (int t = 0; t < 2; ++t)
        *reinterpret_cast<float4*>(g.d + (size_t)pos * H + n0 + 16 * t + 4 * part) = make_float4(acc[t][mt][0], acc[t][mt][1], acc[t][mt][2], acc[t][mt][3]);
    }
  }
}

// yr[t][n] over the row's picks in expert-id order: acc = fma(s2 * w, d, acc); four columns a thread. TOPK > 0: the picks'
// loads are all issued before the first add (the adds keep their order); 0: any top-k, one pick after the other
template <int TOPK>
__global__ void __launch_bounds__(256) k_pf_combine(const float* __restrict__ d, const int* __restrict__ rpos, const float* __restrict__ rk,
                                                    int T, int H, int topk, float* __restrict__ yr) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per = H / 4;
  if (i >= (size_t)T * per) return;
  const int t = (int)(i / per), n = (int)(i % per) * 4;
  float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
  if (TOPK > 0) {
    float k[TOPK > 0 ? TOPK : 1];
    pf8::v4f_t v[TOPK > 0 ? TOPK : 1];
#pragma unroll
    for (int r = 0; r < TOPK; ++r) {
      k[r] = rk[t * TOPK + r];
      v[r] = __builtin_nontemporal_load(reinterpret_cast<const pf8::v4f_t*>(d + (size_t)rpos[t * TOPK + r] * H + n));
    }
#pragma unroll
    for (int r = 0; r < TOPK; ++r) a.x = fmaf(k[r], v[r][0], a.x), a.y = fmaf(k[r], v[r][1], a.y), a.z = fmaf(k[r], v[r][2], a.z), a.w = fmaf(k[r], v[r][3], a.w);
  } else {
    for (int r = 0; r < topk; ++r) {
      const float k = rk[t * topk + r];
      const float4 v = *reinterpret_cast<const float4*>(d + (size_t)rpos[t * topk + r] * H + n);
      a.x = fmaf(k, v.x, a.x), a.y = fmaf(k, v.y, a.y), a.z = fmaf(k, v.z, a.z), a.w = fmaf(k, v.w, a.w);
    }
  }
  *reinterpret_cast<float4*>(yr + (size_t)t * H + n) = a;
}
static void launch_pf_combine(const float* d, const int* rpos, const float* rk, int T, int H, int topk, float* yr, hipStream_t st) {
  const size_t n = (size_t)T * (H / 4);
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (topk == 8) hipLaunchKernelGGL(k_pf_combine<8>, grid, block, 0, st, d, rpos, rk, T, H, topk, yr);
  else hipLaunchKernelGGL(k_pf_combine<0>, grid, block, 0, st, d, rpos, rk, T, H, topk, yr);
}

// DeepSeek's combine (ds41f engine/kernels/moe.cu:974-981): y[t] = the f32 sum, in expert-id order, of the picks' outputs
// (each already rounded to bf16 by the down GEMM), then the shared expert's; eight columns a thread. TOPK > 0: every
// row is requested before the first add (the adds keep their order); 0: any top-k, one row after the other
template <int TOPK>
__global__ void __launch_bounds__(256) k_pfmx_combine(const uint16_t* __restrict__ d, const uint16_t* __restrict__ dsh, const int* __restrict__ rpos,
                                                      int T, int H, int topk, float* __restrict__ y) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per = H / 8;
  if (i >= (size_t)T * per) return;
  const int t = (int)(i / per), n = (int)(i % per) * 8;
  float a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  auto add = [&](const u32x4_t v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) a[2 * j] = __fadd_rn(a[2 * j], bf16_bits_to_f32(v[j] & 0xFFFFu)), a[2 * j + 1] = __fadd_rn(a[2 * j + 1], bf16_bits_to_f32(v[j] >> 16));
  };
  if (TOPK > 0) {
    u32x4_t v[TOPK > 0 ? TOPK + 1 : 1];
#pragma unroll
    for (int r = 0; r < TOPK; ++r) v[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(d + (size_t)rpos[t * TOPK + r] * H + n));
    if (dsh) v[TOPK] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(dsh + (size_t)t * H + n));
#pragma unroll
    for (int r = 0; r < TOPK; ++r) add(v[r]);
    if (dsh) add(v[TOPK]);
  } else {
    for (int r = 0; r < topk; ++r) add(*reinterpret_cast<const u32x4_t*>(d + (size_t)rpos[t * topk + r] * H + n));
    if (dsh) add(*reinterpret_cast<const u32x4_t*>(dsh + (size_t)t * H + n));
  }
  float4* o = reinterpret_cast<float4*>(y + (size_t)t * H + n);
  o[0] = make_float4(a[0], a[1], a[2], a[3]), o[1] = make_float4(a[4], a[5], a[6], a[7]);
}

// one v_mfma_scale_f32_16x16x128_f8f6f4: A [16 rows][128 k] as e2m1 pairs (64 bytes a row) or e4m3, B [16][128] e4m3, a
// ue8m0 byte per row and 32 k for each (SA, SB [16][4]); out[a row][b row]. Operands as the kernels of pf_gemm_mx.cuh
// hand them over: an 8-bit row's bytes 16 part ... and 64 + 16 part ..., a 4-bit row's bytes 16 part ..., scale byte `part`.
template <int CBSZ>
__global__ void __launch_bounds__(64) k_probe_mfma_scaled(const uint8_t* __restrict__ A, const uint8_t* __restrict__ SA, const uint8_t* __restrict__ B,
                                                          const uint8_t* __restrict__ SB, const float* __restrict__ C, float* __restrict__ out) {
  const int l = threadIdx.x, row = l % 16, part = l / 16;
  pf8::v8i_t a = {0, 0, 0, 0, 0, 0, 0, 0}, b;
  if (CBSZ == 4) {
    const uint4 lo = *reinterpret_cast<const uint4*>(A + row * 64 + part * 16);
    a = pf8::v8i_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, 0, 0, 0, 0};
  } else {
    const uint4 lo = *reinterpret_cast<const uint4*>(A + row * 128 + part * 16), hi = *reinterpret_cast<const uint4*>(A + row * 128 + 64 + part * 16);
    a = pf8::v8i_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  }
  {
    const uint4 lo = *reinterpret_cast<const uint4*>(B + row * 128 + part * 16), hi = *reinterpret_cast<const uint4*>(B + row * 128 + 64 + part * 16);
    b = pf8::v8i_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  }
  pf8::v4f_t c = {0.f, 0.f, 0.f, 0.f};
  if (C) {
#pragma unroll
    for (int q = 0; q < 4; ++q) c[q] = C[(4 * part + q) * 16 + row];
  }
  c = pfmx::mfma_mx<CBSZ>(a, b, c, SA[row * 4 + part], SB[row * 4 + part]);
#pragma unroll
  for (int q = 0; q < 4; ++q) out[(4 * part + q) * 16 + row] = c[q];
}

// one v_mfma_f32_16x16x32_bf16: A [16][32], B [16][32] bf16 bits (a lane of part p holds k = 8 p .. 8 p + 7 of its row), C [16][16]
__global__ void __launch_bounds__(64) k_probe_mfma_bf16(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, const float* __restrict__ C,
                                                        float* __restrict__ out) {
  typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
  const int l = threadIdx.x, row = l % 16, part = l / 16;
  const uint4 a = *reinterpret_cast<const uint4*>(A + row * 32 + part * 8), b = *reinterpret_cast<const uint4*>(B + row * 32 + part * 8);
  pf8::v4f_t c = {0.f, 0.f, 0.f, 0.f};
  if (C) {
#pragma unroll
    for (int q = 0; q < 4; ++q) c[q] = C[(4 * part + q) * 16 + row];
  }
  c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, a), __builtin_bit_cast(v8bf_t, b), c, 0, 0, 0);
#pragma unroll
  for (int q = 0; q < 4; ++q) out[(4 * part + q) * 16 + row] = c[q];
}

bool layer_has_fp8_shared(const dsgx_layer_w* L) { return L->sh.g && L->sh.u && L->sh.d && L->sh.gs && L->sh.us && L->sh.ds; }

}  // namespace
}  // namespace dsgx

using namespace dsgx;

extern "C" {

// raw[lane][r]: the accumulator registers of one e4m3 MFMA, so that a test can pin the operand and result layouts the
// prefill kernels assume. form 0: v_mfma_f32_32x32x64 over A [32][64], B [32][64]; form 1: v_mfma_f32_16x16x128 over
// A [16][128], B [16][128] (codes, k contiguous; 16 floats a lane, form 1 fills the first four).
int dsgx_probe_mfma_fp8(const void* A, const void* B, float* raw, int form, void* stream) {
  if (!A || !B || !raw || form < 0 || form > 1) return fail(DSGX_EINVAL, "probe_mfma_fp8: null argument or form %d", form);
  if (form == 0) hipLaunchKernelGGL(k_probe_mfma_fp8, dim3(1), dim3(64), 0, (hipStream_t)stream, (const uint8_t*)A, (const uint8_t*)B, raw);
  else hipLaunchKernelGGL(k_probe_mfma_fp8_k128, dim3(1), dim3(64), 0, (hipStream_t)stream, (const uint8_t*)A, (const uint8_t*)B, raw);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}

void dsgx_prefill_cfg_default(dsgx_prefill_cfg* c) {
  if (!c) return;
  c->shared = 1;
  c->phases = 31;
  c->act_fp8 = 1;
  c->fast_act = 0;
  c->tile_order = -1;
}

static int prefill_check(const dsgx_layer_w* L, int T, const char* who) {
  if (!L) return fail(DSGX_EINVAL, "%s: null layer", who);
  if (L->fmt != DSGX_FMT_FP8_B128 && L->fmt != DSGX_FMT_INT4_G32)
    return fail(DSGX_EUNSUPPORTED, "%s: FP8_B128 and INT4_G32 layers are built (format %u)", who, L->fmt);
  if (T < 1 || T > DSGX_MAX_CHUNK) return fail(DSGX_EINVAL, "%s: T %d (1..%d)", who, T, DSGX_MAX_CHUNK);
  if (L->H < 256 || L->H % 256 || L->I < 128 || L->I % 128)
    return fail(DSGX_EINVAL, "%s: H %d (a multiple of 256), I %d (a multiple of 128)", who, L->H, L->I);
  if (L->E < 1 || L->E > DSGX_MAX_EXPERTS || L->topk < 1 || L->topk > DSGX_MAX_TOPK || L->topk > L->E)
    return fail(DSGX_EINVAL, "%s: E %d, top-k %d", who, L->E, L->topk);
  return DSGX_OK;
}

size_t dsgx_prefill_ws_bytes(const dsgx_layer_w* L, int T) {
  if (prefill_check(L, T, "prefill_ws_bytes")) return 0;
  return pf_layout(L, T).total;
}

int dsgx_moe_prefill(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int T, void* ws, float* yr, float* ys,
                     void* stream, const dsgx_prefill_cfg* cfg_in) {
  if (int rc = prefill_check(L, T, "moe_prefill")) return rc;
  dsgx_prefill_cfg cfg;
  dsgx_prefill_cfg_default(&cfg);
  if (cfg_in) cfg = *cfg_in;
  if (!x || !idx || !w || !ws || !yr) return fail(DSGX_EINVAL, "moe_prefill: null x, idx, w, ws or yr");
  if (!L->pool || !L->desc) return fail(DSGX_EINVAL, "moe_prefill: layer without pool or descriptors");
  const bool i4 = L->fmt == DSGX_FMT_INT4_G32;
  if (cfg.shared && !i4 && L->sh.bgu) return fail(DSGX_EUNSUPPORTED, "moe_prefill: a BF16 shared expert in an FP8 layer is not built yet");
  if (cfg.shared && i4 && L->sh.g) return fail(DSGX_EUNSUPPORTED, "moe_prefill: an FP8 shared expert in an INT4 layer is not built yet");
  const bool shared = cfg.shared && (i4 ? (L->sh.bgu && L->sh.bd) : layer_has_fp8_shared(L));
  if (shared && !ys) return fail(DSGX_EINVAL, "moe_prefill: the layer has a fused shared expert and ys is null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const PfLayout o = pf_layout(L, T);
  uint8_t* W = static_cast<uint8_t*>(ws);
  auto I32 = [&](size_t off) { return reinterpret_cast<int*>(W + off); };
  auto F32 = [&](size_t off) { return reinterpret_cast<float*>(W + off); };
  const int H = L->H, I = L->I, E = L->E, topk = L->topk, P = o.P;
  int order = cfg.tile_order < 0 ? kDefaultTileOrder : cfg.tile_order;
  if (order > 2) return fail(DSGX_EINVAL, "moe_prefill: tile_order %d (-1, 0, 1, 2)", cfg.tile_order);
  if (i4 || !cfg.act_fp8) order = 0;  // (the bf16-activation kernels walk the 128-position list)

  if (cfg.phases & 1) {
    const int NB = (T + kRowBlock - 1) / kRowBlock;
    uint32_t* bmask = reinterpret_cast<uint32_t*>(W + o.bmask);
    hipLaunchKernelGGL(k_pf_mask, dim3(NB), dim3(256), 0, st, idx, T, topk, E, I32(o.bcnt), bmask);
    const TileLists tl{I32(o.ntiles), I32(o.tile_e), I32(o.tile_m0), I32(o.nbig), I32(o.big_e), I32(o.big_m0), I32(o.nsmall), I32(o.small_e), I32(o.small_m0),
                       I32(o.nmix), I32(o.mix_e), I32(o.mix_m0), I32(o.ord_e), I32(o.ord_m0)};
    hipLaunchKernelGGL(k_pf_scan, dim3(1), dim3(DSGX_MAX_EXPERTS), 0, st, I32(o.bcnt), NB, E, I32(o.boff), I32(o.cnt), I32(o.off), tl, order);
    hipLaunchKernelGGL(k_pf_place, dim3(NB), dim3(256), 0, st, idx, w, T, topk, E, I32(o.off), I32(o.boff), bmask, L->desc, I32(o.perm),
                       I32(o.pickpos), I32(o.rpos), I32(o.re), F32(o.rk), (float*)nullptr);
    DSGX_HIP(hipGetLastError());
  }
  if (i4 || !cfg.act_fp8) {
    // bf16 activations throughout: x -> h (bf16) -> d (f32 a pick) -> combine; the shared expert likewise -> ys.
    // INT4 layers (BF16 shared expert), or FP8 layers under the engine's own contract (act_fp8 = 0; FP8 shared expert)
    const size_t lds16 = (size_t)kStages16 * kPanel16;
    auto k_up = i4 ? k_pf_gemm16<true, DSGX_FMT_INT4_G32> : k_pf_gemm16<true, DSGX_FMT_FP8_B128>;
    auto k_dn = i4 ? k_pf_gemm16<false, DSGX_FMT_INT4_G32> : k_pf_gemm16<false, DSGX_FMT_FP8_B128>;
    auto k_sup = i4 ? k_pf_gemm16<true, DSGX_FMT_BF16> : k_pf_gemm16<true, DSGX_FMT_FP8_B128>;
    auto k_sdn = i4 ? k_pf_gemm16<false, DSGX_FMT_BF16> : k_pf_gemm16<false, DSGX_FMT_FP8_B128>;
    for (const void* k : {(const void*)k_up, (const void*)k_dn, (const void*)k_sup, (const void*)k_sdn})
      if (int rc = allow_dynamic_lds(k, lds16)) return rc;
    Gemm16Args q{};
    q.L = *L;
    q.tile_e = I32(o.tile_e), q.tile_m0 = I32(o.tile_m0), q.ntiles = I32(o.ntiles), q.off = I32(o.off), q.nrows = P;
    // INT4 experts: the LDS-staged kernels of pf_gemm_i4.cuh (DSGX_PF_I4_OLD=1: the register-ring kernel they replaced, same bits)
    const char* old4 = std::getenv("DSGX_PF_I4_OLD");
    const bool new4 = i4 && !(old4 && old4[0] == '1');
    pfi4::Args q4{};
    if (new4) {
      for (const void* k : {(const void*)pfi4::k_gemm<true>, (const void*)pfi4::k_gemm<false>})
        if (int rc = allow_dynamic_lds(k, pfi4::kLds)) return rc;
      q4.L = *L, q4.tile_e = I32(o.tile_e), q4.tile_m0 = I32(o.tile_m0), q4.ntiles = I32(o.ntiles), q4.off = I32(o.off);
    }
    if (cfg.phases & 2) {
      q.x = x, q.gather = I32(o.perm), q.h = reinterpret_cast<uint16_t*>(W + o.h), q.d = nullptr;
      q4.x = q.x, q4.gather = q.gather, q4.h = q.h, q4.d = nullptr;
      if (new4) hipLaunchKernelGGL(pfi4::k_gemm<true>, dim3(pf8::grid_of(o.max_tiles, I / (kWgRows / 2))), dim3(pf8::kThreads), pfi4::kLds, st, q4);
      else hipLaunchKernelGGL(k_up, dim3(pf_grid(o.max_tiles, I / (kWgRows / 2))), dim3(kGemmThreads), lds16, st, q);
    }
    if (cfg.phases & 4) {
      q.x = reinterpret_cast<const uint16_t*>(W + o.h), q.gather = nullptr, q.h = nullptr, q.d = F32(o.d);
      q4.x = q.x, q4.gather = nullptr, q4.h = nullptr, q4.d = q.d;
      if (new4) hipLaunchKernelGGL(pfi4::k_gemm<false>, dim3(pf8::grid_of(o.max_tiles, H / kWgRows)), dim3(pf8::kThreads), pfi4::kLds, st, q4);
      else hipLaunchKernelGGL(k_dn, dim3(pf_grid(o.max_tiles, H / kWgRows)), dim3(kGemmThreads), lds16, st, q);
    }
    if (cfg.phases & 8) {
      launch_pf_combine(F32(o.d), I32(o.rpos), F32(o.rk), T, H, topk, yr, st);
    }
    if ((cfg.phases & 16) && shared) {
      const int tiles = (T + kTile - 1) / kTile;
      q.tile_e = q.tile_m0 = q.ntiles = q.off = nullptr, q.nrows = T;
      q.x = x, q.gather = nullptr, q.h = reinterpret_cast<uint16_t*>(W + o.hsh), q.d = nullptr;
      hipLaunchKernelGGL(k_sup, dim3(pf_grid(tiles, I / (kWgRows / 2))), dim3(kGemmThreads), lds16, st, q);
      q.x = reinterpret_cast<const uint16_t*>(W + o.hsh), q.h = nullptr, q.d = ys;
      hipLaunchKernelGGL(k_sdn, dim3(pf_grid(tiles, H / kWgRows)), dim3(kGemmThreads), lds16, st, q);
    }
    DSGX_HIP(hipGetLastError());
    return DSGX_OK;
  }
  // FP8 activations: x quantised -> gate/up + SwiGLU (h bf16 for the view, and quantised for the down projection in the
  // same kernel) -> down (f32 a pick) -> ordered combine. Every GEMM runs twice: the 256-position tiles, then the
  // experts' remainders of up to 128 positions.
  if (H > 8192 || I > 8192) return fail(DSGX_EUNSUPPORTED, "moe_prefill: FP8 activations: hidden %d, intermediate %d (up to 8192)", H, I);
  void (*k_up)(pf8::Args) = pf8::k_gemm_mixed<true>;    // the routed experts: the merged list of both tile shapes
  void (*k_dn)(pf8::Args) = pf8::k_gemm_mixed<false>;
  void (*k_up2)(pf8::Args) = pf8::k_gemm<true, 2>;      // the shared expert: 256-position tiles
  void (*k_dn2)(pf8::Args) = pf8::k_gemm<false, 2>;
#ifdef DSGX_PF_DIAG
  {  // diagnostic build: DSGX_PF_DIAG=<bits> switches parts of the kernels off (wrong results; for timing only)
    const char* dv = std::getenv("DSGX_PF_DIAG");
    switch (dv ? std::atoi(dv) : 0) {
#define DSGX_DIAG_CASE(n) case n: k_up = pf8::k_gemm_mixed<true, n>, k_dn = pf8::k_gemm_mixed<false, n>, k_up2 = pf8::k_gemm<true, 2, n>, k_dn2 = pf8::k_gemm<false, 2, n>; break;
      DSGX_DIAG_CASE(1) DSGX_DIAG_CASE(2) DSGX_DIAG_CASE(4) DSGX_DIAG_CASE(8) DSGX_DIAG_CASE(16) DSGX_DIAG_CASE(3) DSGX_DIAG_CASE(9) DSGX_DIAG_CASE(25) DSGX_DIAG_CASE(32) DSGX_DIAG_CASE(64) DSGX_DIAG_CASE(128) DSGX_DIAG_CASE(256) DSGX_DIAG_CASE(384)
#undef DSGX_DIAG_CASE
    }
  }
#endif
  constexpr int kLdsMix = pf8::Shape<1>::kLds > pf8::Shape<2>::kLds ? pf8::Shape<1>::kLds : pf8::Shape<2>::kLds;
  for (const void* k : {(const void*)k_up, (const void*)k_dn})
    if (int rc = allow_dynamic_lds(k, kLdsMix)) return rc;
  for (const void* k : {(const void*)k_up2, (const void*)k_dn2})
    if (int rc = allow_dynamic_lds(k, pf8::Shape<2>::kLds)) return rc;
  pf8::Args g{};
  g.L = *L;
  g.fast_act = cfg.fast_act;
#ifdef DSGX_PF_TRACE
  if (const char* tp = std::getenv("DSGX_PF_TRACE_PTR")) g.trace = reinterpret_cast<unsigned long long*>(std::strtoull(tp, nullptr, 0));
#endif
  const int NSU = I / (pf8::kWgRows / 2), NSD = H / pf8::kWgRows;
  const bool mixed = order >= 1;
  g.tile_e = I32(mixed ? o.ord_e : o.mix_e), g.tile_m0 = I32(mixed ? o.ord_m0 : o.mix_m0), g.ntiles = I32(o.nmix), g.off = I32(o.off), g.nrows = P;
  if (cfg.phases & (2 | 16)) {
    if (int rc = dsgx_act_quant(x, T, H, W + o.xq, F32(o.xs), stream)) return rc;
  }
  if (cfg.phases & 2) {
    g.aq = W + o.xq, g.as = F32(o.xs), g.gather = I32(o.perm);
    g.h = reinterpret_cast<uint16_t*>(W + o.h), g.hq = W + o.hq, g.hs = F32(o.hs), g.d = nullptr;
    hipLaunchKernelGGL(k_up, dim3(pf8::grid_of(o.max_big + E, NSU)), dim3(pf8::kThreads), kLdsMix, st, g);
    DSGX_HIP(hipGetLastError());
  }
  if (cfg.phases & 4) {
    g.aq = W + o.hq, g.as = F32(o.hs), g.gather = nullptr;
    g.h = nullptr, g.hq = nullptr, g.hs = nullptr, g.d = F32(o.d);
    hipLaunchKernelGGL(k_dn, dim3(pf8::grid_of(o.max_big + E, NSD)), dim3(pf8::kThreads), kLdsMix, st, g);
    DSGX_HIP(hipGetLastError());
  }
  if (cfg.phases & 8) {
    launch_pf_combine(F32(o.d), I32(o.rpos), F32(o.rk), T, H, topk, yr, st);
    DSGX_HIP(hipGetLastError());
  }
  if ((cfg.phases & 16) && shared) {
    const int tiles = (T + 255) / 256;
    g.tile_e = g.tile_m0 = g.ntiles = g.off = nullptr, g.nrows = T;
    g.aq = W + o.xq, g.as = F32(o.xs), g.gather = nullptr;
    g.h = reinterpret_cast<uint16_t*>(W + o.hsh), g.hq = W + o.hshq, g.hs = F32(o.hshs), g.d = nullptr;
    hipLaunchKernelGGL(k_up2, dim3(pf8::grid_of(tiles, NSU)), dim3(pf8::kThreads), pf8::Shape<2>::kLds, st, g);
    g.aq = W + o.hshq, g.as = F32(o.hshs), g.h = nullptr, g.hq = nullptr, g.hs = nullptr, g.d = ys;
    hipLaunchKernelGGL(k_dn2, dim3(pf8::grid_of(tiles, NSD)), dim3(pf8::kThreads), pf8::Shape<2>::kLds, st, g);
    DSGX_HIP(hipGetLastError());
  }
  return DSGX_OK;
}

int dsgx_prefill_view_get(const dsgx_layer_w* L, void* ws, int T, dsgx_prefill_view* out) {
  if (int rc = prefill_check(L, T, "prefill_view")) return rc;
  if (!ws || !out) return fail(DSGX_EINVAL, "prefill_view: null ws or out");
  const PfLayout o = pf_layout(L, T);
  uint8_t* W = static_cast<uint8_t*>(ws);
  out->rpos = reinterpret_cast<const int*>(W + o.rpos);
  out->re = reinterpret_cast<const int*>(W + o.re);
  out->h = reinterpret_cast<const uint16_t*>(W + o.h);
  out->hsh = reinterpret_cast<const uint16_t*>(W + o.hsh);
  out->off = reinterpret_cast<const int*>(W + o.off);
  out->perm = reinterpret_cast<const int*>(W + o.perm);
  return DSGX_OK;
}

int dsgx_probe_mfma_bf16(const void* A, const void* B, const float* C, float* out, void* stream) {
  if (!A || !B || !out) return fail(DSGX_EINVAL, "probe_mfma_bf16: null argument");
  hipLaunchKernelGGL(k_probe_mfma_bf16, dim3(1), dim3(64), 0, (hipStream_t)stream, (const uint16_t*)A, (const uint16_t*)B, C, out);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}

// one v_dot2_f32_bf16 a thread (the vector-unit kernels' multiply-add: common.cuh's dot2)
__global__ void __launch_bounds__(256) k_probe_dot2(const uint32_t* __restrict__ a, const uint32_t* __restrict__ b, const float* __restrict__ c,
                                                    float* __restrict__ out, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = dot2(a[i], b[i], c[i]);
}
int dsgx_probe_dot2_bf16(const void* a, const void* b, const float* c, float* out, int n, void* stream) {
  if (!a || !b || !c || !out || n <= 0) return fail(DSGX_EINVAL, "probe_dot2_bf16: null argument or n <= 0");
  hipLaunchKernelGGL(k_probe_dot2, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (const uint32_t*)a, (const uint32_t*)b, c, out, n);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}

int dsgx_probe_mfma_scaled(const void* A, const void* SA, const void* B, const void* SB, int a_fp4, const float* C, float* out, void* stream) {
  if (!A || !SA || !B || !SB || !out) return fail(DSGX_EINVAL, "probe_mfma_scaled: null argument");
  const uint8_t *a = (const uint8_t*)A, *sa = (const uint8_t*)SA, *b = (const uint8_t*)B, *sb = (const uint8_t*)SB;
  if (a_fp4) hipLaunchKernelGGL(k_probe_mfma_scaled<4>, dim3(1), dim3(64), 0, (hipStream_t)stream, a, sa, b, sb, C, out);
  else hipLaunchKernelGGL(k_probe_mfma_scaled<0>, dim3(1), dim3(64), 0, (hipStream_t)stream, a, sa, b, sb, C, out);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}

// ---- DeepSeek's prefill MoE (dsk::moe_prefill, ds41f-4xgx10-switchless/engine/kernels/dsk.h:268-295, prefill.cu:1605-1675) ----
void dsgx_dsk_prefill_cfg_default(dsgx_dsk_prefill_cfg* c) {
  if (!c) return;
  c->swiglu_limit = 10.f;
  c->phases = 31;
}
static int dsk_prefill_check(const dsgx_dsk_weights* W, int T, const char* who, dsgx_layer_w* shape) {
  if (!W) return fail(DSGX_EINVAL, "%s: null weights", who);
  if (T < 1 || T > DSGX_MAX_CHUNK) return fail(DSGX_EINVAL, "%s: T %d (1..%d)", who, T, DSGX_MAX_CHUNK);
  if (W->H < 256 || W->H % 256 || W->I < 128 || W->I % 128 || W->H > 16384 || W->I > 16384)
    return fail(DSGX_EINVAL, "%s: H %d (a multiple of 256), I %d (a multiple of 128), both up to 16384", who, W->H, W->I);
  if (W->E < 1 || W->E > DSGX_MAX_EXPERTS || W->topk < 1 || W->topk > DSGX_MAX_TOPK || W->topk > W->E)
    return fail(DSGX_EINVAL, "%s: E %d, top-k %d", who, W->E, W->topk);
  *shape = dsgx_layer_w{};
  shape->H = W->H, shape->I = W->I, shape->E = W->E, shape->topk = W->topk, shape->fmt = DSGX_FMT_MXFP4_G32;
  return DSGX_OK;
}
size_t dsgx_dsk_prefill_ws_bytes(int H, int I, int E, int topk, int T) {
  dsgx_dsk_weights w{};
  w.H = H, w.I = I, w.E = E, w.topk = topk;
  dsgx_layer_w shape;
  if (dsk_prefill_check(&w, T, "dsk_prefill_ws_bytes", &shape)) return 0;
  return pf_layout(&shape, T).total;
}

int dsgx_dsk_moe_prefill(const dsgx_dsk_weights* Wt, const uint8_t* xq, const uint8_t* xs, int T, const int* idx, const float* w, void* ws,
                         float* y, void* stream, const dsgx_dsk_prefill_cfg* cfg_in) {
  dsgx_layer_w shape;
  if (int rc = dsk_prefill_check(Wt, T, "dsk_moe_prefill", &shape)) return rc;
  dsgx_dsk_prefill_cfg cfg;
  dsgx_dsk_prefill_cfg_default(&cfg);
  if (cfg_in) cfg = *cfg_in;
  if (!xq || !xs || !idx || !w || !ws || !y) return fail(DSGX_EINVAL, "dsk_moe_prefill: null xq, xs, idx, w, ws or y");
  if (!Wt->w1 || !Wt->s1 || !Wt->w3 || !Wt->s3 || !Wt->w2 || !Wt->s2) return fail(DSGX_EINVAL, "dsk_moe_prefill: null expert tensor");
  const bool shared = Wt->sh_w1 != nullptr;
  if (shared && (!Wt->sh_s1 || !Wt->sh_w3 || !Wt->sh_s3 || !Wt->sh_w2 || !Wt->sh_s2)) return fail(DSGX_EINVAL, "dsk_moe_prefill: shared expert tensors missing");
  for (const void* p : {(const void*)xq, (const void*)Wt->w1, (const void*)Wt->w3, (const void*)Wt->w2, (const void*)Wt->sh_w1, (const void*)Wt->sh_w3, (const void*)Wt->sh_w2})
    if ((uintptr_t)p % 16) return fail(DSGX_EINVAL, "dsk_moe_prefill: xq and the weight tensors must be 16-byte aligned");
  for (const void* p : {(const void*)xs, (const void*)Wt->s1, (const void*)Wt->s3, (const void*)Wt->s2, (const void*)Wt->sh_s1, (const void*)Wt->sh_s3, (const void*)Wt->sh_s2})
    if ((uintptr_t)p % 4) return fail(DSGX_EINVAL, "dsk_moe_prefill: the scale tensors must be 4-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const PfLayout o = pf_layout(&shape, T);
  uint8_t* W = static_cast<uint8_t*>(ws);
  auto I32 = [&](size_t off) { return reinterpret_cast<int*>(W + off); };
  auto F32 = [&](size_t off) { return reinterpret_cast<float*>(W + off); };
  auto U16 = [&](size_t off) { return reinterpret_cast<uint16_t*>(W + off); };
  const int H = Wt->H, I = Wt->I, E = Wt->E, topk = Wt->topk, P = o.P;
  constexpr int F4 = DSGX_FMT_MXFP4_G32, F8 = DSGX_FMT_FP8_B32E;
  constexpr int kLdsMix = pfmx::Shape<1, F4>::kLds > pfmx::Shape<2, F4>::kLds ? pfmx::Shape<1, F4>::kLds : pfmx::Shape<2, F4>::kLds;
  constexpr int kLdsSh = pfmx::Shape<2, F8>::kLds;
  void (*k_up)(pfmx::Args) = pfmx::k_gemm_mixed<true, F4>;
  void (*k_dn)(pfmx::Args) = pfmx::k_gemm_mixed<false, F4>;
  void (*k_sup)(pfmx::Args) = pfmx::k_gemm<true, F8>;
  void (*k_sdn)(pfmx::Args) = pfmx::k_gemm<false, F8>;
#ifdef DSGX_PF_DIAG
  {  // diagnostic build: DSGX_PF_DIAG=<bits> switches parts of the kernels off (wrong results; for timing only)
    const char* dv = std::getenv("DSGX_PF_DIAG");
    switch (dv ? std::atoi(dv) : 0) {
#define DSGX_DIAG_CASE(n) case n: k_up = pfmx::k_gemm_mixed<true, F4, n>, k_dn = pfmx::k_gemm_mixed<false, F4, n>, k_sup = pfmx::k_gemm<true, F8, n>, k_sdn = pfmx::k_gemm<false, F8, n>; break;
      DSGX_DIAG_CASE(1) DSGX_DIAG_CASE(4) DSGX_DIAG_CASE(8) DSGX_DIAG_CASE(32) DSGX_DIAG_CASE(64) DSGX_DIAG_CASE(128) DSGX_DIAG_CASE(256) DSGX_DIAG_CASE(384) DSGX_DIAG_CASE(512) DSGX_DIAG_CASE(1024) DSGX_DIAG_CASE(513) DSGX_DIAG_CASE(1025) DSGX_DIAG_CASE(1152) DSGX_DIAG_CASE(1280) DSGX_DIAG_CASE(1408) DSGX_DIAG_CASE(1032) DSGX_DIAG_CASE(1088) DSGX_DIAG_CASE(1056)
#undef DSGX_DIAG_CASE
    }
  }
#endif
  for (const void* k : {(const void*)k_up, (const void*)k_dn})
    if (int rc = allow_dynamic_lds(k, kLdsMix)) return rc;
  for (const void* k : {(const void*)k_sup, (const void*)k_sdn})
    if (int rc = allow_dynamic_lds(k, kLdsSh)) return rc;
  const int NSU = I / (pf8::kWgRows / 2), NSD = H / pf8::kWgRows;
  uint16_t* dsh = U16(o.d + align256((size_t)P * H * 2));  // the shared expert's outputs behind the picks', both bf16
  // phases (dsk::MoePCfg, dsk.h:278-282): 1 bucketing, 2 shared expert, 4 routed up, 8 routed down, 16 combine
  if (cfg.phases & 1) {
    const int NB = (T + kRowBlock - 1) / kRowBlock;
    uint32_t* bmask = reinterpret_cast<uint32_t*>(W + o.bmask);
    hipLaunchKernelGGL(k_pf_mask, dim3(NB), dim3(256), 0, st, idx, T, topk, E, I32(o.bcnt), bmask);
    const TileLists tl{I32(o.ntiles), I32(o.tile_e), I32(o.tile_m0), I32(o.nbig), I32(o.big_e), I32(o.big_m0), I32(o.nsmall), I32(o.small_e), I32(o.small_m0),
                       I32(o.nmix), I32(o.mix_e), I32(o.mix_m0), I32(o.ord_e), I32(o.ord_m0)};
    hipLaunchKernelGGL(k_pf_scan, dim3(1), dim3(DSGX_MAX_EXPERTS), 0, st, I32(o.bcnt), NB, E, I32(o.boff), I32(o.cnt), I32(o.off), tl, 0);
    hipLaunchKernelGGL(k_pf_place, dim3(NB), dim3(256), 0, st, idx, w, T, topk, E, I32(o.off), I32(o.boff), bmask, (const dsgx_mat_desc*)nullptr, I32(o.perm),
                       I32(o.pickpos), I32(o.rpos), I32(o.re), F32(o.rk), F32(o.posw));
    DSGX_HIP(hipGetLastError());
  }
  pfmx::Args g{};
  g.H = H, g.I = I, g.limit = cfg.swiglu_limit;
  if ((cfg.phases & 2) && shared) {
    const int tiles = (T + 255) / 256;
    g.tile_e = g.tile_m0 = g.ntiles = g.off = nullptr, g.nrows = T, g.gather = nullptr, g.posw = nullptr, g.wstride = g.sstride = 0;
    g.aq = xq, g.as = xs, g.wa = Wt->sh_w1, g.sa = Wt->sh_s1, g.wb = Wt->sh_w3, g.sb = Wt->sh_s3;
    g.h = U16(o.hsh), g.hq = W + o.hshq, g.hs = W + o.hshs, g.d = nullptr;
    hipLaunchKernelGGL(k_sup, dim3(pf8::grid_of(tiles, NSU)), dim3(pf8::kThreads), kLdsSh, st, g);
    g.aq = W + o.hshq, g.as = W + o.hshs, g.wa = Wt->sh_w2, g.sa = Wt->sh_s2, g.wb = g.sb = nullptr;
    g.h = nullptr, g.hq = g.hs = nullptr, g.d = dsh;
    hipLaunchKernelGGL(k_sdn, dim3(pf8::grid_of(tiles, NSD)), dim3(pf8::kThreads), kLdsSh, st, g);
    DSGX_HIP(hipGetLastError());
  }
  g.tile_e = I32(o.mix_e), g.tile_m0 = I32(o.mix_m0), g.ntiles = I32(o.nmix), g.off = I32(o.off), g.nrows = P;
  auto launch = [&](bool up) {
    hipLaunchKernelGGL(up ? k_up : k_dn, dim3(pf8::grid_of(o.max_big + E, up ? NSU : NSD)), dim3(pf8::kThreads), kLdsMix, st, g);
  };
  if (cfg.phases & 4) {
    g.aq = xq, g.as = xs, g.gather = I32(o.perm), g.posw = F32(o.posw);
    g.wa = Wt->w1, g.sa = Wt->s1, g.wb = Wt->w3, g.sb = Wt->s3, g.wstride = (size_t)I * H / 2, g.sstride = (size_t)I * H / 32;
    g.h = U16(o.h), g.hq = W + o.hq, g.hs = W + o.hs, g.d = nullptr;
    launch(true);
    DSGX_HIP(hipGetLastError());
  }
  if (cfg.phases & 8) {
    g.aq = W + o.hq, g.as = W + o.hs, g.gather = nullptr, g.posw = nullptr;
    g.wa = Wt->w2, g.sa = Wt->s2, g.wb = g.sb = nullptr, g.wstride = (size_t)I * H / 2, g.sstride = (size_t)I * H / 32;
    g.h = nullptr, g.hq = g.hs = nullptr, g.d = U16(o.d);
    launch(false);
    DSGX_HIP(hipGetLastError());
  }
  if (cfg.phases & 16) {
    const size_t n = (size_t)T * (H / 8);
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    const uint16_t* sh = shared ? dsh : (const uint16_t*)nullptr;
    if (topk == 6) hipLaunchKernelGGL(k_pfmx_combine<6>, grid, block, 0, st, U16(o.d), sh, I32(o.rpos), T, H, topk, y);
    else if (topk == 8) hipLaunchKernelGGL(k_pfmx_combine<8>, grid, block, 0, st, U16(o.d), sh, I32(o.rpos), T, H, topk, y);
    else hipLaunchKernelGGL(k_pfmx_combine<0>, grid, block, 0, st, U16(o.d), sh, I32(o.rpos), T, H, topk, y);
    DSGX_HIP(hipGetLastError());
  }
  return DSGX_OK;
}

int dsgx_dsk_prefill_view_get(const dsgx_dsk_weights* Wt, void* ws, int T, dsgx_dsk_prefill_view* out) {
  dsgx_layer_w shape;
  if (int rc = dsk_prefill_check(Wt, T, "dsk_prefill_view", &shape)) return rc;
  if (!ws || !out) return fail(DSGX_EINVAL, "dsk_prefill_view: null ws or out");
  const PfLayout o = pf_layout(&shape, T);
  uint8_t* W = static_cast<uint8_t*>(ws);
  out->rpos = reinterpret_cast<const int*>(W + o.rpos);
  out->re = reinterpret_cast<const int*>(W + o.re);
  out->off = reinterpret_cast<const int*>(W + o.off);
  out->perm = reinterpret_cast<const int*>(W + o.perm);
  out->h = reinterpret_cast<const uint16_t*>(W + o.h);
  out->hsh = reinterpret_cast<const uint16_t*>(W + o.hsh);
  out->hq = W + o.hq, out->hs = W + o.hs;
  out->d = reinterpret_cast<const uint16_t*>(W + o.d);
  out->dsh = reinterpret_cast<const uint16_t*>(W + o.d + align256((size_t)o.P * Wt->H * 2));
  return DSGX_OK;
}

}  // extern "C"
