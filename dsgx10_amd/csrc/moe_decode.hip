// The decode expert step for 1-16 rows: the gfx950 counterpart of the reference's gx::moe_decode
// (altar1-4xgx10-switchless/engine/experts/decode.cu; contract in engine/experts/experts.h:104-147).
//
// Two kernels, as the reference's k_up / k_down:
//  k_up    every (slot, channel pair) of the union of the rows' picks (expert-id order; a fused shared expert first) is a
//          batch of four weight rows (gate c, gate c+1, up c, up c+1) owned by one wavefront, which streams them once,
//          K split over its 64 lanes, dequantises in registers, sums against the M activation rows staged in LDS, adds
//          the lanes' partials with cross-lane shuffles, and writes h = bf16(bf16(silu(bf16 g)) * bf16 u) (decode.cu:366-400).
//  k_down  a wavefront owns RB output rows and walks every slot in expert-id order: per lane acc = fma(s2 * w_row, partial,
//          acc), the routing weight 0 for rows that did not pick the expert, so a row's bits do not depend on the other
//          rows (decode.cu:526-566); the lanes are added once at the end. The fused shared expert's rows go to ys, and
//          with ysum yr += ys (decode.cu:569-581).
// Both kernels size their grid to the chip and use no atomics: results are deterministic and batch-invariant.
// The order of the f32 adds inside a dot product differs from the reference's (not part of its contract).
#include <algorithm>

#include "abi_internal.h"
#include "rowdot.cuh"

namespace dsgx {
namespace {

struct DecodeArgs {
  const uint16_t* x;
  int M;
  const int* idx;
  const float* w;
  const float* logits;  // fused routing (DecodeCfg::logits): idx, w unused
  const float* bias;
  float route_scale;
  int score_fn;
  dsgx_layer_w L;
  uint16_t* h;  // [slot][M][I]
  float* yr;
  float* ys;
  int ysum;
  int shfmt;  // the fused shared expert's format, 0: none
};

// The union of the rows' picks in expert-id order (build_union of the reference, decode.cu:57-106), by every
// workgroup for itself. WT: also the rows' weights per slot.
struct Union {
  int n;
  uint32_t mask[DSGX_MAX_EXPERTS / 32];
  int ri[DSGX_MAX_ROWS * DSGX_MAX_TOPK];
  float rw[DSGX_MAX_ROWS * DSGX_MAX_TOPK];
  int id[DSGX_MAX_UNION];
};
__device__ void build_union(Union& U, const DecodeArgs& a, float (*wslot)[DSGX_MAX_ROWS]) {
  const int tid = threadIdx.x, E = a.L.E, topk = a.L.topk, ne = a.M * topk;
  if (tid < DSGX_MAX_EXPERTS / 32) U.mask[tid] = 0;
  if (wslot)
    for (int i = tid; i < DSGX_MAX_UNION * DSGX_MAX_ROWS; i += blockDim.x) (&wslot[0][0])[i] = 0.f;
  if (a.logits) {  // a wavefront a row, route()'s code
    for (int row = tid >> 6; row < a.M; row += blockDim.x >> 6) {
      int id;
      float w;
      route_row(a.logits + (size_t)row * E, a.bias, E, topk, a.route_scale, a.score_fn, tid & 63, id, w);
      if ((tid & 63) < topk) U.ri[row * topk + (tid & 63)] = id, U.rw[row * topk + (tid & 63)] = w;
    }
  } else {
    for (int i = tid; i < ne; i += blockDim.x) U.ri[i] = a.idx[i], U.rw[i] = a.w[i];
  }
  __syncthreads();
  for (int i = tid; i < ne; i += blockDim.x) atomicOr(&U.mask[U.ri[i] >> 5], 1u << (U.ri[i] & 31));
  __syncthreads();
  for (int i = tid; i < ne; i += blockDim.x) {
    const int e = U.ri[i];
    int r = __popc(U.mask[e >> 5] & ((1u << (e & 31)) - 1));
    for (int j = 0; j < (e >> 5); ++j) r += __popc(U.mask[j]);
    U.id[r] = e;
    if (wslot) wslot[r][i / topk] = U.rw[i];
  }
  if (tid == 0) {
    int n = 0;
    for (int j = 0; j < DSGX_MAX_EXPERTS / 32; ++j) n += __popc(U.mask[j]);
    U.n = n;
  }
  __syncthreads();
}

__device__ __forceinline__ MatDev mat_of(const uint8_t* base, uint32_t fmt, int N, int K, float s2) {
  MatDev m;
  m.w = base, m.s = m.zp = nullptr, m.lrs = m.lks = 7, m.srow = K >> 7, m.s2 = s2;
  if (fmt == DSGX_FMT_FP8_B128) m.s = base + ((size_t)N * K + 255) / 256 * 256;
  else if (fmt == DSGX_FMT_INT4_G32) {
    m.s = base + ((size_t)N * K / 2 + 255) / 256 * 256;
    m.zp = m.s + ((size_t)N * (K / 32) * 2 + 255) / 256 * 256;
  }
  return m;
}
__device__ __forceinline__ MatDev mat_parts(const uint8_t* w, const void* s, int K) {
  MatDev m;
  m.w = w, m.s = static_cast<const uint8_t*>(s), m.zp = nullptr, m.lrs = m.lks = 7, m.srow = K >> 7, m.s2 = 1.f;
  return m;
}

// ---------------------------------------------------------------------------------------------------------------------
// gate/up. F: the format of the slots this body walks. INTER: the matrix is the BF16 shared expert's interleaved
// gate/up (rows 2c gate, 2c + 1 up); else gate and up are two matrices. Wave numbering (gw of GW) is the caller's.
struct UpSlot {
  MatDev g, u;
  int hslot;
};
template <int FMT, int M, bool INTER, int D>
__device__ __forceinline__ void up_body(const DecodeArgs& a, const uint4* xs, const UpSlot* slots, int nsl, int gw, int GW) {
  constexpr int RB = 4;
  const int lane = threadIdx.x & 63, H = a.L.H, I = a.L.I;
  const int nsegk = num_segs<FMT>(H), nq = nsegk * FmtT<FMT>::SEGK / 8;
  const int nb_e = I / 2, nbatch = nsl * nb_e;
  const int nmine = gw < nbatch ? (nbatch - gw + GW - 1) / GW : 0;
  const int nsteps = nmine * nsegk;
  Raw w[D][RB];
  int lj = 0, lseg = 0;
  auto load = [&](Raw (&r)[RB]) {
    const int b = gw + lj * GW, sl = b / nb_e, p = b % nb_e;
    const UpSlot& S = slots[sl];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      if (INTER) load_raw<FMT>(r[i], S.g, 4 * p + i, lseg, lane, H);
      else load_raw<FMT>(r[i], i < 2 ? S.g : S.u, 2 * p + (i & 1), lseg, lane, H);
    }
    if (++lseg == nsegk) lseg = 0, ++lj;
  };
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < nsteps) load(w[d]);
  float acc[RB][M];
  int cj = 0, cseg = 0;
  for (int t0 = 0; t0 < nsteps; t0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int t = t0 + d;
      if (t >= nsteps) break;
      if (cseg == 0) {
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
          for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
      }
      step_dot<FMT, M, RB>(w[d], xs, nq, cseg, lane, acc);
      if (t + D < nsteps) load(w[d]);
      if (++cseg < nsegk) continue;
      cseg = 0;
      const int b = gw + cj * GW, sl = b / nb_e, p = b % nb_e;
      ++cj;
      // lane i * M + m (i: the batch's channel 0 or 1) finishes channel 2p + i of activation row m
      float gv = 0.f, uv = 0.f;
#pragma unroll
      for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) {
          const float v = wave_sum(acc[r][m]);
          const int ch = INTER ? r >> 1 : r & 1;
          const bool up = INTER ? (r & 1) : (r >> 1);
          if (lane == ch * M + m) {
            if (up) uv = v;
            else gv = v;
          }
        }
      if (lane < 2 * M) {
        const UpSlot& S = slots[sl];
        const int i = lane / M, m = lane % M;
        const float gt = bf16_round(__fmul_rn(gv, S.g.s2)), ut = bf16_round(__fmul_rn(uv, INTER ? S.g.s2 : S.u.s2));
        a.h[((size_t)S.hslot * a.M + m) * I + 2 * p + i] = (uint16_t)swiglu_bits(gt, ut);
      }
    }
  }
}

template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(256) k_up(DecodeArgs a, int shared_wgs) {
  extern __shared__ uint4 xs[];
  __shared__ Union U;
  __shared__ UpSlot slots[DSGX_MAX_UNION + 1];
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  const int H = a.L.H, I = a.L.I;
  const int wpb = blockDim.x >> 6;
  if (kMixed && (int)blockIdx.x < shared_wgs) {
    // these workgroups do the BF16 shared expert's interleaved gate/up only
    if (threadIdx.x == 0) {
      slots[0].g = mat_parts(a.L.sh.bgu, nullptr, H);
      slots[0].u = slots[0].g;
      slots[0].hslot = DSGX_SH_SLOT;
    }
    stage_x<FmtT<DSGX_FMT_BF16>::KL>(xs, a.x, H, M, H, num_segs<DSGX_FMT_BF16>(H) * 512);
    __syncthreads();
    if constexpr (kMixed)
      up_body<DSGX_FMT_BF16, M, true, 4>(a, xs, slots, 1, blockIdx.x * wpb + (threadIdx.x >> 6), shared_wgs * wpb);
    return;
  }
  stage_x<FmtT<FMT>::KL>(xs, a.x, H, M, H, num_segs<FMT>(H) * FmtT<FMT>::SEGK);
  build_union(U, a, nullptr);
  const int nsh = (SHFMT != 0 && !kMixed) ? 1 : 0;  // a same-format (FP8) shared expert is slot 0
  const int nsl = nsh + U.n;
  for (int s = threadIdx.x; s < nsl; s += blockDim.x) {
    UpSlot S;
    if (s < nsh) {
      S.g = mat_parts(a.L.sh.g, a.L.sh.gs, H);
      S.u = mat_parts(a.L.sh.u, a.L.sh.us, H);
      S.hslot = DSGX_SH_SLOT;
    } else {
      const dsgx_mat_desc* d = a.L.desc + (size_t)U.id[s - nsh] * 3;
      S.g = mat_of(a.L.pool + d[0].off, FMT, I, H, d[0].s2);
      S.u = mat_of(a.L.pool + d[1].off, FMT, I, H, d[1].s2);
      S.hslot = s - nsh;
    }
    slots[s] = S;
  }
  __syncthreads();
  const int wg0 = kMixed ? shared_wgs : 0;
  up_body<FMT, M, false, 4>(a, xs, slots, nsl, ((int)blockIdx.x - wg0) * wpb + (threadIdx.x >> 6), ((int)gridDim.x - wg0) * wpb);
}

// ---------------------------------------------------------------------------------------------------------------------
// down
struct DownSlot {
  MatDev d;
  int hslot;   // where its h is in the workspace
  int shared;  // its rows go to ys
};
template <int FMT, int SHFMT, int M, int RB, int D>
__global__ void __launch_bounds__(256) k_down(DecodeArgs a, int slots_per_chunk) {
  extern __shared__ uint4 hs[];  // a chunk's h: [slot in chunk][M][I / 8 chunks]
  __shared__ Union U;
  __shared__ float wslot[DSGX_MAX_UNION][DSGX_MAX_ROWS];
  __shared__ DownSlot slots[DSGX_MAX_UNION + 1];
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  const int H = a.L.H, I = a.L.I, lane = threadIdx.x & 63;
  build_union(U, a, wslot);
  const int nsh = SHFMT != 0 ? 1 : 0;
  const int nsl = nsh + U.n;
  for (int s = threadIdx.x; s < nsl; s += blockDim.x) {
    DownSlot S;
    if (s < nsh) {
      S.d = SHFMT == DSGX_FMT_BF16 ? mat_parts(a.L.sh.bd, nullptr, I) : mat_parts(a.L.sh.d, a.L.sh.ds, I);
      S.hslot = DSGX_SH_SLOT, S.shared = 1;
    } else {
      const dsgx_mat_desc* d = a.L.desc + (size_t)U.id[s - nsh] * 3 + 2;
      S.d = mat_of(a.L.pool + d->off, FMT, H, I, d->s2);
      S.hslot = s - nsh, S.shared = 0;
    }
    slots[s] = S;
  }
  __syncthreads();
  const int n0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * RB;  // the wave's rows (past H: idle, but in the barriers)
  const bool live = n0 < H;
  const int nq = I / 8;                           // chunks a row of h
  const int segs_r = num_segs<FMT>(I);            // segments a routed slot
  const int segs_s = nsh ? (SHFMT == DSGX_FMT_BF16 ? num_segs<DSGX_FMT_BF16>(I) : num_segs<DSGX_FMT_FP8_B128>(I)) : 0;
  const int nsteps = live ? segs_s + U.n * segs_r : 0;

  Raw w[D][RB];
  int ls = 0, lseg = 0;
  auto load = [&](Raw (&r)[RB]) {
    const DownSlot& S = slots[ls];
    const bool sh = kMixed && ls < nsh;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      if (sh) load_raw<SHFMT == 0 ? FMT : SHFMT>(r[i], S.d, n0 + i, lseg, lane, I);
      else load_raw<FMT>(r[i], S.d, n0 + i, lseg, lane, I);
    }
    if (++lseg == (ls < nsh ? segs_s : segs_r)) lseg = 0, ++ls;
  };
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < nsteps) load(w[d]);

  float yacc[RB][M], sacc[RB][M], acc[RB][M];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) yacc[r][m] = sacc[r][m] = 0.f;

  int t = 0;  // this wave's step counter
  for (int c0 = 0; c0 < nsl; c0 += slots_per_chunk) {
    const int c1 = min(nsl, c0 + slots_per_chunk);
    // stage the chunk's h rows, each slot in its format's lane order
    __syncthreads();
    for (int s = c0; s < c1; ++s) {
      const uint16_t* hp = a.h + (size_t)slots[s].hslot * a.M * I;
      uint4* dst = hs + (size_t)(s - c0) * M * nq;
      if (kMixed && s < nsh) stage_x<FmtT<SHFMT == 0 ? FMT : SHFMT>::KL>(dst, hp, I, M, I, I);
      else stage_x<FmtT<FMT>::KL>(dst, hp, I, M, I, I);
    }
    __syncthreads();
    if (!live) continue;
    for (int s = c0; s < c1; ++s) {
      const bool sh = s < nsh;
      const int nseg = sh ? segs_s : segs_r;
      const uint4* xs = hs + (size_t)(s - c0) * M * nq;
#pragma unroll
      for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
      for (int seg = 0; seg < nseg; ++seg, ++t) {
        // the ring slot of step t is t % D: dispatch so that the register index is a constant
        bool done = false;
#pragma unroll
        for (int d = 0; d < D; ++d) {
          if (done || (t % D) != d) continue;
          if (kMixed && sh) step_dot<SHFMT == 0 ? FMT : SHFMT, M, RB>(w[d], xs, nq, seg, lane, acc);
          else step_dot<FMT, M, RB>(w[d], xs, nq, seg, lane, acc);
          if (t + D < nsteps) load(w[d]);
          done = true;
        }
      }
      const DownSlot& S = slots[s];
#pragma unroll
      for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) {
          if (sh) sacc[r][m] = acc[r][m];
          else yacc[r][m] = fmaf(__fmul_rn(S.d.s2, wslot[s - nsh][m]), acc[r][m], yacc[r][m]);
        }
    }
  }
  if (!live) return;
  // add the lanes; lane r * M + m keeps output (row n0 + r, activation row m)
  float yv = 0.f, sv = 0.f;
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float v = wave_sum(yacc[r][m]);
      if (lane == r * M + m) yv = v;
      if (SHFMT != 0) {
        const float s = wave_sum(sacc[r][m]);
        if (lane == r * M + m) sv = s;
      }
    }
  if (lane >= RB * M) return;
  const int r = lane / M, m = lane % M;
  const size_t o = (size_t)m * H + n0 + r;
  if (SHFMT != 0) a.ys[o] = sv;
  else if (a.ysum) sv = a.ys[o];
  if (a.ysum) yv = __fadd_rn(yv, sv);
  a.yr[o] = yv;
}

// ---------------------------------------------------------------------------------------------------------------------
template <class K>
int set_lds(K kern, size_t lds) { return allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds); }

template <int FMT, int SHFMT, int M>
int launch_decode(const DecodeArgs& a, int parts, hipStream_t st) {
  const int H = a.L.H, I = a.L.I, cus = num_cus_cached();
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  if (parts & 1) {
    const int segk = FmtT<FMT>::SEGK;
    size_t lds = (size_t)M * ((H + segk - 1) / segk * segk) * 2;
    if (kMixed) lds = std::max(lds, (size_t)M * ((H + 511) / 512 * 512) * 2);
    const int per_cu = lds <= 56 * 1024 ? 2 : 1;
    int grid = cus * per_cu, shared_wgs = 0;
    if (kMixed) {
      // split the workgroups between the BF16 shared expert and the routed experts by their bytes (M * top-k picks at most)
      const double bsh = 2.0 * I * H * 2, bro = (double)std::min(a.M * a.L.topk, a.L.E) * 2.0 * (double)dsgx_mat_bytes(FMT, I, H);
      shared_wgs = (int)(grid * bsh / (bsh + bro) + 0.5);
      shared_wgs = std::max(1, std::min(grid - 1, shared_wgs));
    }
    auto kern = k_up<FMT, SHFMT, M>;
    if (int rc = set_lds(kern, lds)) return rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, a, shared_wgs);
    DSGX_HIP(hipGetLastError());
  }
  if (parts & 2) {
    constexpr int RB = 2;
    // a chunk of slots' h in LDS: at most 64 KiB
    const size_t slot_bytes = (size_t)M * I * 2;
    int spc = (int)((64 * 1024) / slot_bytes);
    if (spc < 1) spc = 1;
    if (spc > DSGX_MAX_UNION + 1) spc = DSGX_MAX_UNION + 1;
    const size_t lds = (size_t)spc * slot_bytes;
    const int waves = (H + RB - 1) / RB, grid = (waves + 3) / 4;
    auto kern = k_down<FMT, SHFMT, M, RB, 4>;
    if (int rc = set_lds(kern, lds)) return rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, a, spc);
    DSGX_HIP(hipGetLastError());
  }
  return DSGX_OK;
}

template <int FMT, int SHFMT>
int launch_decode_m(const DecodeArgs& a, int parts, hipStream_t st) {
  switch (a.M) {
    case 1: return launch_decode<FMT, SHFMT, 1>(a, parts, st);
    case 2: return launch_decode<FMT, SHFMT, 2>(a, parts, st);
    case 3: return launch_decode<FMT, SHFMT, 3>(a, parts, st);
    case 4: return launch_decode<FMT, SHFMT, 4>(a, parts, st);
    case 5: return launch_decode<FMT, SHFMT, 5>(a, parts, st);
    case 6: return launch_decode<FMT, SHFMT, 6>(a, parts, st);
    case 7: return launch_decode<FMT, SHFMT, 7>(a, parts, st);
    case 8: return launch_decode<FMT, SHFMT, 8>(a, parts, st);
  }
  return fail(DSGX_EUNSUPPORTED, "moe_decode: %d rows (1..8 are built; the reference takes up to 16)", a.M);
}

}  // namespace
}  // namespace dsgx

using namespace dsgx;

extern "C" {

void dsgx_decode_cfg_default(dsgx_decode_cfg* c) {
  if (!c) return;
  c->up = c->down = 0;
  c->parts = 3;
  c->ysum = 0;
  c->logits = c->bias = nullptr;
  c->route_scale = 1.f;
  c->score_fn = 0;
  c->post = nullptr;
}

size_t dsgx_decode_ws_bytes(const dsgx_layer_w* L) {
  if (!L || L->I <= 0) return 0;
  return (size_t)(DSGX_MAX_UNION + 1) * DSGX_MAX_ROWS * L->I * 2 + 256;
}

int dsgx_moe_decode(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, void* ws, float* yr, float* ys,
                    void* stream, const dsgx_decode_cfg* cfg) {
  dsgx_decode_cfg c;
  if (cfg) c = *cfg;
  else dsgx_decode_cfg_default(&c);
  // the reference's checks (decode.cu:710-729): it dies, this returns an error
  if (!L || !x || !ws) return fail(DSGX_EINVAL, "moe_decode: null layer, x or workspace");
  if (M < 1 || M > DSGX_MAX_ROWS) return fail(DSGX_EINVAL, "moe_decode: M=%d", M);
  if (!c.logits && (!idx || !w)) return fail(DSGX_EINVAL, "moe_decode: idx and w, or logits");
  if (c.post) return fail(DSGX_EUNSUPPORTED, "moe_decode: posted outputs need the reference's ring; one GPU has none");
  if (c.parts < 1 || c.parts > 3) return fail(DSGX_EINVAL, "moe_decode: parts %d", c.parts);
  if (c.up != 0 || c.down != 0) return fail(DSGX_EINVAL, "moe_decode: up variant %d / down variant %d (only 0 is built)", c.up, c.down);
  if (L->fmt == DSGX_FMT_REF_NVFP4 || L->fmt == DSGX_FMT_REF_INT4 || L->fmt == DSGX_FMT_REF_BF16)
    return fail(DSGX_EFORMAT, "moe_decode: layer expert format %u names a GB10 block tiling; repack to FP8_B128 (16), INT4_G32 (18) or BF16 (19)", L->fmt);
  if (L->fmt != DSGX_FMT_FP8_B128 && L->fmt != DSGX_FMT_INT4_G32 && L->fmt != DSGX_FMT_BF16)
    return fail(DSGX_EFORMAT, "moe_decode: layer expert format %u is not FP8_B128 (16), INT4_G32 (18) or BF16 (19)", L->fmt);
  if (!L->pool || !L->desc) return fail(DSGX_EINVAL, "moe_decode: null pool or descriptors");
  const int H = L->H, I = L->I;
  if (L->E < 1 || L->E > DSGX_MAX_EXPERTS || L->topk < 1 || L->topk > DSGX_MAX_TOPK || L->topk > L->E)
    return fail(DSGX_EINVAL, "moe_decode: E %d, top-k %d", L->E, L->topk);
  const int kmul = L->fmt == DSGX_FMT_INT4_G32 ? 2048 : L->fmt == DSGX_FMT_FP8_B128 ? 1024 : 512;
  if (H < kmul || H % kmul || I < kmul || I % kmul || I % 128 || H % 128)
    return fail(DSGX_EINVAL, "moe_decode: hidden %d, intermediate %d (multiples of %d for this format)", H, I, kmul);
  const bool fp8sh = L->sh.g != nullptr, b16sh = L->sh.bgu != nullptr;
  if (fp8sh && b16sh) return fail(DSGX_EINVAL, "moe_decode: an FP8 and a BF16 shared expert");
  if (fp8sh && (!L->sh.u || !L->sh.d || !L->sh.gs || !L->sh.us || !L->sh.ds)) return fail(DSGX_EINVAL, "moe_decode: the FP8 shared expert needs g, u, d and their scales");
  if (fp8sh && (H % 1024 || I % 1024)) return fail(DSGX_EINVAL, "moe_decode: the FP8 shared expert needs hidden and intermediate multiples of 1024");
  if (b16sh && !L->sh.bd) return fail(DSGX_EINVAL, "moe_decode: the BF16 shared expert needs its down");
  if ((c.parts & 2) && !yr) return fail(DSGX_EINVAL, "moe_decode: null yr");
  if ((fp8sh || b16sh || c.ysum) && (c.parts & 2) && !ys) return fail(DSGX_EINVAL, "moe_decode: ys (the shared expert's output) is needed");
  if (((uintptr_t)x | (uintptr_t)ws | (uintptr_t)L->pool) & 15) return fail(DSGX_EINVAL, "moe_decode: x, ws and pool must be 16-byte aligned");

  DecodeArgs a{};
  a.x = x, a.M = M, a.idx = idx, a.w = w, a.logits = c.logits, a.bias = c.bias, a.route_scale = c.route_scale, a.score_fn = c.score_fn;
  a.L = *L, a.h = static_cast<uint16_t*>(ws), a.yr = yr, a.ys = ys, a.ysum = c.ysum;
  a.shfmt = fp8sh ? DSGX_FMT_FP8_B128 : b16sh ? DSGX_FMT_BF16 : 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t f = L->fmt;
#define DSGX_GO(F, S) return launch_decode_m<F, S>(a, c.parts, st)
  if (f == DSGX_FMT_FP8_B128) {
    if (fp8sh) DSGX_GO(DSGX_FMT_FP8_B128, DSGX_FMT_FP8_B128);
    if (b16sh) return fail(DSGX_EUNSUPPORTED, "moe_decode: FP8 experts with a BF16 shared expert are not built");
    DSGX_GO(DSGX_FMT_FP8_B128, 0);
  }
  if (f == DSGX_FMT_INT4_G32) {
    if (fp8sh) return fail(DSGX_EUNSUPPORTED, "moe_decode: INT4 experts with an FP8 shared expert are not built");
    if (b16sh) DSGX_GO(DSGX_FMT_INT4_G32, DSGX_FMT_BF16);
    DSGX_GO(DSGX_FMT_INT4_G32, 0);
  }
  if (fp8sh || b16sh) return fail(DSGX_EUNSUPPORTED, "moe_decode: BF16 experts with a fused shared expert are not built");
  DSGX_GO(DSGX_FMT_BF16, 0);
#undef DSGX_GO
}

}  // extern "C"
