// The decode expert step for 1-8 rows: the gfx950 counterpart of the reference's gx::moe_decode
// (altar1-4xgx10-switchless/engine/experts/decode.cu; contract in engine/experts/experts.h:104-147).
//
// The arithmetic of the reference's two kernels:
//  up    every (slot, channel pair) of the union of the rows' picks (expert-id order; a fused shared expert first) is a
//        batch of four weight rows (gate c, gate c+1, up c, up c+1) owned by one wavefront, which streams them once,
//        K split over its 64 lanes, dequantises in registers, sums against the M activation rows staged in LDS, adds
//        the lanes' partials with cross-lane shuffles, and writes h = bf16(bf16(silu(bf16 g)) * bf16 u) (decode.cu:366-400).
//  down  a wavefront owns output rows and walks every slot in expert-id order: per lane acc = fma(s2 * w_row, partial,
//        acc), the routing weight 0 for rows that did not pick the expert, so a row's bits do not depend on the other
//        rows (decode.cu:526-566); the lanes are added once at the end. The fused shared expert's rows go to ys, and
//        with ysum yr += ys (decode.cu:569-581).
// Default: ONE persistent kernel runs both phases (k_decode): the grid is sized so that every workgroup is resident,
// each wavefront issues the first loads of its down rows, then the grid meets at a barrier in device memory (h is
// complete), then the down phase runs. This is what the reference gets from programmatic dependent launch
// (decode.cu:170-172, 448-452): the second phase's weights are already in flight while the first one drains. With
// DecodeCfg::logits the routing runs inside the kernel too (experts.h:123-127), so a layer is a single launch.
// The two phases are also built as two kernels (k_up, k_down) for the bench's `parts` switch.
// No atomics touch the results: they are deterministic and batch-invariant. The order of the f32 adds inside a dot
// product differs from the reference's (not part of its contract).
#pragma once
#include <algorithm>

#include "abi_internal.h"
#include "rowdot.cuh"

namespace dsgx {

// Diagnostic build only (-DDSGX_TRACE): thread 0 of every workgroup stamps the 100 MHz wall clock at phase marks.
#ifdef DSGX_TRACE
#define DSGX_MARK(k)                                                                        \
  do {                                                                                      \
    if (a.trace && threadIdx.x == 0) a.trace[blockIdx.x * 16 + (k)] = wall_clock64();       \
  } while (0)
#else
#define DSGX_MARK(k) do { } while (0)
#endif

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
  int* bar;     // the grid barrier's words in the workspace (grid_barrier)
#ifdef DSGX_TRACE
  unsigned long long* trace;
#endif
  int spin_limit;
};

int launch_decode_fp8(const DecodeArgs& a, int parts, bool shared, hipStream_t st);
int launch_decode_int4(const DecodeArgs& a, int parts, bool shared_bf16, hipStream_t st);
int launch_decode_bf16(const DecodeArgs& a, int parts, hipStream_t st);

// ---- what a workgroup knows about the step -------------------------------------------------------------------------
struct MatRef {
  const uint8_t* w;  // codes / weight_packed / bf16 rows
  const uint8_t* s;  // scales (FP8 f32, INT4 bf16); INT4's zero points follow at a fixed offset
  float s2;
  int pad;
};
struct Slot {
  MatRef g, u, d;
  int hslot, shared;
};
template <int M>
struct Step {
  int n;                               // distinct picked experts
  uint32_t mask[DSGX_MAX_EXPERTS / 32];
  int ri[M * DSGX_MAX_TOPK];
  float rw[M * DSGX_MAX_TOPK];
  int id[M * DSGX_MAX_TOPK];
  float wslot[M * DSGX_MAX_TOPK][M];   // per slot the rows' routing weights (0: the row did not pick it)
  Slot slots[M * DSGX_MAX_TOPK + 1];
  int gen;                             // the grid barrier's generation at kernel start
};

// The union of the rows' picks in expert-id order (build_union of the reference, decode.cu:57-106), by every
// workgroup for itself; with logits the rows are routed here first (a wavefront a row, route()'s code and bits).
template <int M>
__device__ void build_union(Step<M>& S, const DecodeArgs& a) {
  const int tid = threadIdx.x, E = a.L.E, topk = a.L.topk, ne = M * topk;
  if (tid < DSGX_MAX_EXPERTS / 32) S.mask[tid] = 0;
  for (int i = tid; i < M * DSGX_MAX_TOPK * M; i += blockDim.x) (&S.wslot[0][0])[i] = 0.f;
  if (a.logits) {
    for (int row = tid >> 6; row < M; row += blockDim.x >> 6) {
      int id;
      float w;
      route_row(a.logits + (size_t)row * E, a.bias, E, topk, a.route_scale, a.score_fn, tid & 63, id, w);
      if ((tid & 63) < topk) S.ri[row * topk + (tid & 63)] = id, S.rw[row * topk + (tid & 63)] = w;
    }
  } else {
    for (int i = tid; i < ne; i += blockDim.x) S.ri[i] = a.idx[i], S.rw[i] = a.w[i];
  }
  __syncthreads();
  for (int i = tid; i < ne; i += blockDim.x) atomicOr(&S.mask[S.ri[i] >> 5], 1u << (S.ri[i] & 31));
  __syncthreads();
  for (int i = tid; i < ne; i += blockDim.x) {
    const int e = S.ri[i];
    int r = __popc(S.mask[e >> 5] & ((1u << (e & 31)) - 1));
    for (int j = 0; j < (e >> 5); ++j) r += __popc(S.mask[j]);
    S.id[r] = e;
    S.wslot[r][i / topk] = S.rw[i];
  }
  if (tid == 0) {
    int n = 0;
    for (int j = 0; j < DSGX_MAX_EXPERTS / 32; ++j) n += __popc(S.mask[j]);
    S.n = n;
  }
  __syncthreads();
}

__device__ __forceinline__ size_t al256d(size_t b) { return (b + 255) / 256 * 256; }
template <int FMT>
__device__ __forceinline__ MatRef mat_ref(const uint8_t* base, int N, int K, float s2) {
  MatRef m;
  m.w = base, m.s = nullptr, m.s2 = s2, m.pad = 0;
  if (FMT == DSGX_FMT_FP8_B128) m.s = base + al256d((size_t)N * K);
  else if (FMT == DSGX_FMT_INT4_G32) m.s = base + al256d((size_t)N * K / 2);
  return m;
}
template <int FMT>
__device__ __forceinline__ MatDev mat_dev(const MatRef& r, int N, int K) {
  MatDev m;
  m.w = r.w, m.s = r.s, m.zp = nullptr, m.lrs = m.lks = 7, m.srow = K >> 7, m.s2 = r.s2;
  if (FMT == DSGX_FMT_INT4_G32) m.zp = r.s + al256d((size_t)N * (K / 32) * 2);
  return m;
}
// slots: a fused shared expert first (slot 0), then the union in expert-id order
template <int FMT, int SHFMT, int M>
__device__ void fill_slots(Step<M>& S, const DecodeArgs& a) {
  const int H = a.L.H, I = a.L.I, nsh = SHFMT != 0 ? 1 : 0;
  for (int s = threadIdx.x; s < nsh + S.n; s += blockDim.x) {
    Slot t;
    if (s < nsh) {
      if (SHFMT == DSGX_FMT_BF16) {
        t.g = MatRef{a.L.sh.bgu, nullptr, 1.f, 0};
        t.u = t.g;
        t.d = MatRef{a.L.sh.bd, nullptr, 1.f, 0};
      } else {
        t.g = MatRef{a.L.sh.g, reinterpret_cast<const uint8_t*>(a.L.sh.gs), 1.f, 0};
        t.u = MatRef{a.L.sh.u, reinterpret_cast<const uint8_t*>(a.L.sh.us), 1.f, 0};
        t.d = MatRef{a.L.sh.d, reinterpret_cast<const uint8_t*>(a.L.sh.ds), 1.f, 0};
      }
      t.hslot = DSGX_SH_SLOT, t.shared = 1;
    } else {
      const dsgx_mat_desc* d = a.L.desc + (size_t)S.id[s - nsh] * 3;
      t.g = mat_ref<FMT>(a.L.pool + d[0].off, I, H, d[0].s2);
      t.u = mat_ref<FMT>(a.L.pool + d[1].off, I, H, d[1].s2);
      t.d = mat_ref<FMT>(a.L.pool + d[2].off, H, I, d[2].s2);
      t.hslot = s - nsh, t.shared = 0;
    }
    S.slots[s] = t;
  }
  __syncthreads();
}

// ---- gate/up ------------------------------------------------------------------------------------------------------------
// Walks slots [s0, s0 + nsl) in format F. INTER: the slot's gate matrix is the BF16 shared expert's interleaved gate/up
// (rows 2c gate, 2c + 1 up). The wave is number gw of GW; batches go round-robin.
// CH channels a batch (RB = 2 CH weight rows a step): one channel at few activation rows, where an even split of the
// batches over the waves matters most (the benchmark's 9 slots x 2048 channels over 2048 waves: nine each).
template <int FMT, int M, bool INTER, int CH, int D>
__device__ __forceinline__ void up_body(const DecodeArgs& a, const uint4* xs, const Slot* slots, int nsl, int gw, int GW) {
  constexpr int RB = 2 * CH;
  const int lane = threadIdx.x & 63, H = a.L.H, I = a.L.I;
  const int nsegk = num_segs<FMT>(H), nq = nsegk * FmtT<FMT>::SEGK / 8;
  const int nb_e = I / CH, nbatch = nsl * nb_e;
  const int nmine = gw < nbatch ? (nbatch - gw + GW - 1) / GW : 0;
  const int nsteps = nmine * nsegk;
  // the batch cursors advance by GW batches: (slot, pair) += (GW / nb_e, GW % nb_e) with carry
  const int dsl = GW / nb_e, dp = GW % nb_e;
  int lsl = gw / nb_e, lp = gw % nb_e, lseg = 0;   // the load cursor
  int csl = lsl, cp = lp, cseg = 0;                 // the compute cursor
  Raw w[D][RB];
  float acc[RB][M];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[i][m] = 0.f;
  const uint8_t* dummy = reinterpret_cast<const uint8_t*>(a.x);  // where the loads past the last step go (cached)
  int lt = 0;
  auto load = [&](Raw (&r)[RB]) {
    const bool ok = lt < nsteps;
    ++lt;
    const Slot& S = slots[ok ? lsl : 0];
    const MatDev g = mat_dev<FMT>(S.g, INTER ? 2 * I : I, H), u = mat_dev<FMT>(S.u, I, H);
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      if (INTER) load_raw<FMT, false>(r[i], g, RB * lp + i, lseg, lane, H, acc[i][0], ok ? nullptr : dummy);
      else load_raw<FMT, false>(r[i], i < CH ? g : u, CH * lp + i % CH, lseg, lane, H, acc[i][0], ok ? nullptr : dummy);
    }
    if (ok && ++lseg == nsegk) {
      lseg = 0, lsl += dsl, lp += dp;
      if (lp >= nb_e) lp -= nb_e, ++lsl;
      if (lsl >= nsl) lsl = 0, lp = 0;  // past the wave's last batch: any valid place (these loads go to `dummy`)
    }
  };
  auto compute = [&](const Raw (&r)[RB]) {
    step_dot<FMT, M, RB>(r, xs, nq, cseg, lane, acc);
    if (++cseg < nsegk) return;
    cseg = 0;
    // lane m < M finishes the batch's channel(s) of activation row m and stores them as one 16- or 32-bit word. The
    // store is coherent at device scope (it bypasses the XCD-local L2): the down phase of the same kernel reads h on
    // other XCDs right after the grid barrier.
    float gv[CH], uv[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) gv[c] = uv[c] = 0.f;
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const float v = wave_sum(acc[i][m]);
        acc[i][m] = 0.f;
        const int ch = INTER ? i >> 1 : i % CH;
        const bool up = INTER ? (i & 1) : (i >= CH);
        if (lane == m) {
          if (up) uv[ch] = v;
          else gv[ch] = v;
        }
      }
    if (lane < M) {
      const Slot& S = slots[csl];
      const float sg = S.g.s2, su = S.u.s2;
      uint32_t hb = 0;
#pragma unroll
      for (int c = 0; c < CH; ++c) hb |= swiglu_bits(bf16_round(__fmul_rn(gv[c], sg)), bf16_round(__fmul_rn(uv[c], su))) << (16 * c);
      uint16_t* dst = a.h + ((size_t)S.hslot * M + lane) * I + CH * cp;
      if (CH == 1) __hip_atomic_store((DSGX_GLOBAL uint16_t*)(uintptr_t)dst, (uint16_t)hb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_store((DSGX_GLOBAL uint32_t*)(uintptr_t)dst, hb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    csl += dsl, cp += dp;
    if (cp >= nb_e) cp -= nb_e, ++csl;
  };
  // software pipeline: D steps in flight; every iteration computes a step (while there is one) and issues a load
  if (nsteps == 0) return;
#pragma unroll
  for (int d = 0; d < D; ++d) load(w[d]);
  for (int t = 0; t < nsteps; t += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (t + d < nsteps) compute(w[d]);
      load(w[d]);
    }
  }
}

// x staged for format F, then the up phase of this workgroup. With a shared expert of another format (INT4 experts,
// BF16 shared expert) the first `shared_wgs` workgroups do the shared expert's gate/up and the others the routed slots.
template <int FMT, int SHFMT, int M>
__device__ __forceinline__ void up_phase(const DecodeArgs& a, uint4* xs, Step<M>& S, int shared_wgs) {
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  constexpr int kUpCH = M <= 2 ? 1 : 2, kUpD = 8 / kUpCH;  // 16 KiB of weights in flight a wave either way
  const int H = a.L.H, wpb = blockDim.x >> 6, wave = threadIdx.x >> 6;
  const int nsh = SHFMT != 0 ? 1 : 0;
  if (kMixed) {
    if ((int)blockIdx.x < shared_wgs) {
      stage_x<FmtT<DSGX_FMT_BF16>::KL>(xs, a.x, H, M, H, num_segs<DSGX_FMT_BF16>(H) * 512);
      __syncthreads();
      up_body<kMixed ? DSGX_FMT_BF16 : FMT, M, kMixed, kUpCH, kUpD>(a, xs, S.slots, 1, blockIdx.x * wpb + wave, shared_wgs * wpb);
    } else {
      stage_x<FmtT<FMT>::KL>(xs, a.x, H, M, H, num_segs<FMT>(H) * FmtT<FMT>::SEGK);
      __syncthreads();
      up_body<FMT, M, false, kUpCH, kUpD>(a, xs, S.slots + nsh, S.n, ((int)blockIdx.x - shared_wgs) * wpb + wave, ((int)gridDim.x - shared_wgs) * wpb);
    }
  } else {
    stage_x<FmtT<FMT>::KL>(xs, a.x, H, M, H, num_segs<FMT>(H) * FmtT<FMT>::SEGK);
    __syncthreads();
    up_body<FMT, M, false, kUpCH, kUpD>(a, xs, S.slots, nsh + S.n, blockIdx.x * wpb + wave, gridDim.x * wpb);
  }
}

// ---- down ------------------------------------------------------------------------------------------------------------------
// The wave's rows [n_lo, n_hi) in sub-batches of RB; per sub-batch every slot in order. hs: LDS for `spc` slots' h.
// `between` runs after the first loads are issued and before any h is read (the fused kernel's grid barrier).
template <int FMT, int SHFMT, int M, int D, class Between>
__device__ __forceinline__ void down_phase(const DecodeArgs& a, uint4* hs, Step<M>& S, int spc, int n_lo, int n_hi, Between&& between) {
  constexpr int RB = 2;
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  constexpr int SF = SHFMT == 0 ? FMT : SHFMT;  // the shared slot's format
  const int H = a.L.H, I = a.L.I, lane = threadIdx.x & 63;
  const int nsh = SHFMT != 0 ? 1 : 0, nsl = nsh + S.n;
  const int nq = I / 8;
  const int segs_r = num_segs<FMT>(I), segs_s = nsh ? num_segs<SF>(I) : 0;
  const int nsub = n_hi > n_lo ? (n_hi - n_lo + RB - 1) / RB : 0;
  const int steps_sub = segs_s + S.n * segs_r;
  const int nsteps = nsub * steps_sub;  // this wave's steps with real loads
  // every wave of the workgroup walks the same number of steps (the barriers around the h chunks)
  __shared__ int s_maxsub;
  if (threadIdx.x == 0) s_maxsub = 0;
  __syncthreads();
  if (lane == 0) atomicMax(&s_maxsub, nsub);

  Raw w[D][RB];
  float yacc[RB][M], sacc[RB][M], acc[RB][M];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) yacc[r][m] = sacc[r][m] = acc[r][m] = 0.f;
  const uint8_t* dummy = reinterpret_cast<const uint8_t*>(a.x);
  int lt = 0, lsub = 0, ls = 0, lseg = 0;  // the load cursor
  auto load = [&](Raw (&r)[RB]) {
    const bool ok = lt < nsteps;
    ++lt;
    const Slot& T = S.slots[ok ? ls : 0];
    const bool sh = kMixed && ls < nsh;
    const int n0 = n_lo + lsub * RB;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      const int n = ok ? (n0 + i < n_hi ? n0 + i : n_hi - 1) : 0;  // a row past the end re-reads the last one (its result is dropped)
      if (sh) load_raw<SF, false>(r[i], mat_dev<SF>(T.d, H, I), n, lseg, lane, I, acc[i][0], ok ? nullptr : dummy);
      else load_raw<FMT, false>(r[i], mat_dev<FMT>(T.d, H, I), n, lseg, lane, I, acc[i][0], ok ? nullptr : dummy);
    }
    if (ok && ++lseg == (ls < nsh ? segs_s : segs_r)) {
      lseg = 0;
      if (++ls == nsl) ls = 0, ++lsub;
    }
  };
#pragma unroll
  for (int d = 0; d < D; ++d) load(w[d]);

  between();
  __syncthreads();
  const int maxsub = s_maxsub;
  const bool one_chunk = nsl <= spc;
  const int wg_steps = maxsub * steps_sub;

  int csub = 0, cs = 0, cseg = 0;  // the compute cursor
  auto compute = [&](const Raw (&r)[RB]) {
    const bool live = csub < nsub;
    const bool sh = cs < nsh;
    const int c0 = cs / spc * spc;
    if (cseg == 0 && cs == c0 && !(one_chunk && csub > 0)) {
      // entering a chunk of slots: stage their h rows, each slot in its format's lane order
      const int c1 = min(nsl, c0 + spc);
      __syncthreads();
      if (kMixed && c0 < nsh) {  // the shared slot (another format's lane order), then the routed ones
        stage_slots<FmtT<SF>::KL, false>(hs, 1, M, I, [&](int) { return a.h + (size_t)S.slots[0].hslot * M * I; });
        stage_slots<FmtT<FMT>::KL, false>(hs + (size_t)M * nq, c1 - c0 - 1, M, I,
                                         [&](int s) { return a.h + (size_t)S.slots[c0 + 1 + s].hslot * M * I; });
      } else {
        stage_slots<FmtT<FMT>::KL, false>(hs, c1 - c0, M, I, [&](int s) { return a.h + (size_t)S.slots[c0 + s].hslot * M * I; });
      }
      __syncthreads();
      DSGX_MARK(7);
    }
    const uint4* xs = hs + (size_t)(cs - c0) * M * nq;
    if (live) {
      if (kMixed && sh) step_dot<SF, M, RB>(r, xs, nq, cseg, lane, acc);
      else step_dot<FMT, M, RB>(r, xs, nq, cseg, lane, acc);
    }
    if (++cseg < (sh ? segs_s : segs_r)) return;
    cseg = 0;
    // the slot is complete: into the rows' running sums, in slot (= expert id) order
    const float s2 = S.slots[cs].d.s2;
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int m = 0; m < M; ++m) {
        if (sh) sacc[i][m] = acc[i][m];
        else yacc[i][m] = fmaf(__fmul_rn(s2, S.wslot[cs - nsh][m]), acc[i][m], yacc[i][m]);
        acc[i][m] = 0.f;
      }
    if (++cs < nsl) return;
    cs = 0;
    // the sub-batch is complete: add the lanes; lane i * M + m keeps output (row n0 + i, activation row m)
    const int n0 = n_lo + csub * RB;
    ++csub;
    float yv = 0.f, sv = 0.f;
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const float v = wave_sum(yacc[i][m]);
        if (lane == i * M + m) yv = v;
        if (SHFMT != 0) {
          const float s = wave_sum(sacc[i][m]);
          if (lane == i * M + m) sv = s;
        }
        yacc[i][m] = sacc[i][m] = 0.f;
      }
    if (live && lane < RB * M) {
      const int i = lane / M, m = lane % M;
      if (n0 + i < n_hi) {
        const size_t o = (size_t)m * H + n0 + i;
        if (SHFMT != 0) a.ys[o] = sv;
        else if (a.ysum) sv = a.ys[o];
        if (a.ysum) yv = __fadd_rn(yv, sv);
        a.yr[o] = yv;
      }
    }
  };
  for (int t = 0; t < wg_steps; t += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (t + d < wg_steps) compute(w[d]);
      load(w[d]);
    }
  }
}

// ---- the grid barrier ---------------------------------------------------------------------------------------------------------
// A two-level counting barrier in the workspace, every word on its own 128-byte line (kBarLine ints apart):
//   line g < kBarGroups        arrivals of group g (the workgroups with blockIdx % kBarGroups == g)
//   line kBarGroups            arrivals of the groups' last members
//   line kBarGroups + 1 + g    group g's release word: the generation, bumped by the very last arriver
//   line 2 kBarGroups + 1      error flag
// All zero before the first launch; arrivals are left at 0, the release words all equal. Counters on separate lines
// keep the 500-odd device-scope atomics from queueing on one address, and each waiter polls its own group's word.
// Every workgroup of the grid must be resident (the launch sizes the grid from the occupancy query). The wait is
// bounded: past spin_limit polls the workgroup raises the error flag and goes on (wrong results, never a hang).
constexpr int kBarGroups = 16, kBarLine = 32;
constexpr size_t kBarBytes = (size_t)(2 * kBarGroups + 2) * kBarLine * 4;
__device__ __forceinline__ int bar_load(int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int grid_barrier_gen(int* bar) { return bar_load(bar + (kBarGroups + 1 + blockIdx.x % kBarGroups) * kBarLine); }
__device__ __forceinline__ void grid_barrier(int* bar, int my_gen, int spin_limit) {
  // h was stored with device-scope coherent stores; __syncthreads() waits for every wave's stores to complete, so no
  // cache write-back or invalidate is needed around the counters (a device-scope fence would flush the whole L2 here)
  __syncthreads();
  if (threadIdx.x == 0) {
    const int g = blockIdx.x % kBarGroups;
    const int members = ((int)gridDim.x - g + kBarGroups - 1) / kBarGroups;
    const int groups = min((int)gridDim.x, kBarGroups);
    int* rel = bar + (kBarGroups + 1) * kBarLine;
    bool released = false;
    if (__hip_atomic_fetch_add(bar + g * kBarLine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == members - 1) {
      __hip_atomic_store(bar + g * kBarLine, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (__hip_atomic_fetch_add(bar + kBarGroups * kBarLine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == groups - 1) {
        __hip_atomic_store(bar + kBarGroups * kBarLine, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int i = 0; i < kBarGroups; ++i) __hip_atomic_store(rel + i * kBarLine, my_gen + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        released = true;
      }
    }
    if (!released) {
      int spins = 0;
      while (bar_load(rel + g * kBarLine) == my_gen) {
        __builtin_amdgcn_s_sleep(8);
        if (++spins > spin_limit) {
          __hip_atomic_store(bar + (2 * kBarGroups + 1) * kBarLine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
      }
    }
  }
  __syncthreads();
}

// ---- kernels ----------------------------------------------------------------------------------------------------------------
template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(256) k_decode(DecodeArgs a, int shared_wgs, int spc) {
  extern __shared__ uint4 lds[];
  __shared__ Step<M> S;
  DSGX_MARK(0);
  if (threadIdx.x == 0) S.gen = grid_barrier_gen(a.bar);
  build_union(S, a);
  DSGX_MARK(1);
  fill_slots<FMT, SHFMT, M>(S, a);
  DSGX_MARK(2);
  up_phase<FMT, SHFMT, M>(a, lds, S, shared_wgs);
  DSGX_MARK(4);
  const int H = a.L.H, GW = gridDim.x * (blockDim.x >> 6), gw = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int rpw = (H + GW - 1) / GW;
  const int n_lo = min(H, gw * rpw), n_hi = min(H, n_lo + rpw);
  down_phase<FMT, SHFMT, M, 4>(a, lds, S, spc, n_lo, n_hi, [&] { DSGX_MARK(5); grid_barrier(a.bar, S.gen, a.spin_limit); DSGX_MARK(6); });
  DSGX_MARK(8);
}
template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(256) k_up(DecodeArgs a, int shared_wgs) {
  extern __shared__ uint4 lds[];
  __shared__ Step<M> S;
  build_union(S, a);
  fill_slots<FMT, SHFMT, M>(S, a);
  up_phase<FMT, SHFMT, M>(a, lds, S, shared_wgs);
}
template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(256) k_down(DecodeArgs a, int spc) {
  extern __shared__ uint4 lds[];
  __shared__ Step<M> S;
  build_union(S, a);
  fill_slots<FMT, SHFMT, M>(S, a);
  const int H = a.L.H, gw = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int n_lo = min(H, gw * 2), n_hi = min(H, n_lo + 2);
  down_phase<FMT, SHFMT, M, 4>(a, lds, S, spc, n_lo, n_hi, [] {});
}

// ---- launches ---------------------------------------------------------------------------------------------------------------
template <int FMT, int SHFMT, int M>
int launch_decode(const DecodeArgs& a, int parts, hipStream_t st) {
  const int H = a.L.H, I = a.L.I, cus = num_cus_cached();
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  constexpr int SF = SHFMT == 0 ? FMT : SHFMT;
  const int nsl_max = std::min(a.M * a.L.topk, a.L.E) + (SHFMT != 0 ? 1 : 0);
  // x in LDS for the up phase
  const int segk = FmtT<FMT>::SEGK;
  size_t lds_up = (size_t)M * ((H + segk - 1) / segk * segk) * 2;
  if (kMixed) lds_up = std::max(lds_up, (size_t)M * ((H + 511) / 512 * 512) * 2);
  // h of a chunk of slots in LDS for the down phase: all of them when they fit in 64 KiB
  const size_t slot_bytes = (size_t)M * I * 2;
  int spc = std::max(1, (int)((64 * 1024) / slot_bytes));
  spc = std::min(spc, nsl_max);
  const size_t lds_down = (size_t)spc * slot_bytes;
  auto shared_split = [&](int grid) {
    if (!kMixed) return 0;
    // the workgroups split between the BF16 shared expert and the routed experts by their bytes
    const double bsh = 2.0 * I * H * 2, bro = (double)std::min(a.M * a.L.topk, a.L.E) * 2.0 * (double)dsgx_mat_bytes(FMT, I, H);
    return std::max(1, std::min(grid - 1, (int)(grid * bsh / (bsh + bro) + 0.5)));
  };
  (void)SF;
  if (parts == 3) {
    auto kern = k_decode<FMT, SHFMT, M>;
    const size_t lds = std::max(lds_up, lds_down);
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
    // every workgroup must be resident: the grid comes from the occupancy of this kernel with this much LDS
    int per_cu = 0;
    DSGX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, lds));
    if (per_cu >= 1) {
      per_cu = std::min(per_cu, 2);
      const int grid = cus * per_cu;
      hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, a, shared_split(grid), spc);
      DSGX_HIP(hipGetLastError());
      return DSGX_OK;
    }
    // (no resident grid possible: fall through to the two kernels)
  }
  if (parts & 1) {
    auto kern = k_up<FMT, SHFMT, M>;
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_up)) return rc;
    const int grid = cus * (lds_up <= 56 * 1024 ? 2 : 1);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_up, st, a, shared_split(grid));
    DSGX_HIP(hipGetLastError());
  }
  if (parts & 2) {
    auto kern = k_down<FMT, SHFMT, M>;
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_down)) return rc;
    const int waves = (H + 1) / 2, grid = (waves + 3) / 4;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_down, st, a, spc);
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

}  // namespace dsgx
