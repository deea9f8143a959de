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
#include <type_traits>

#include "abi_internal.h"
#include "rowdot.cuh"

#ifndef DSGX_UPD
#define DSGX_UPD 4
#endif
#ifndef DSGX_WGS
#define DSGX_WGS 1
#endif
// threads of a decode workgroup (one workgroup a CU)
#ifndef DSGX_DECODE_THREADS
#define DSGX_DECODE_THREADS 512
#endif
#ifndef DSGX_DOWND
#define DSGX_DOWND 4
#endif
namespace dsgx {

// Diagnostic build only (-DDSGX_TRACE): thread 0 of every workgroup stamps the 100 MHz wall clock at phase marks.
#ifdef DSGX_TRACE
#define DSGX_MARK(k)                                                                        \
  do {                                                                                      \
    if (a.trace && threadIdx.x == 0) a.trace[blockIdx.x * 16 + (k)] = wall_clock64();       \
  } while (0)
// (by lane 0 of whichever wave runs the code)
#define DSGX_MARKW(k)                                                                       \
  do {                                                                                      \
    if (a.trace && (threadIdx.x & 63) == 0) a.trace[blockIdx.x * 16 + (k)] = wall_clock64(); \
  } while (0)
#else
#define DSGX_MARK(k) do { } while (0)
#define DSGX_MARKW(k) do { } while (0)
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
  float* dpart; // the slot-partitioned down phase's results, f32 [slot][M][H] (k_down_part -> k_down_combine)
  float* fac;   // its slot table: fac[0] = slots (as int bits), fac[8 + slot * 8 + m] = s2_down * w of row m
#ifdef DSGX_TRACE
  unsigned long long* trace;
#endif
  int spin_limit;
  // DeepSeek's expert arithmetic (variant 1 only; moe_decode_mfma.cuh): gate and up clamped, the routing weight applied
  // before w2, h quantised per 32 on its way into the down phase, every expert's output rounded to bf16 before the fold
  int dsk;
  float dsk_limit;
  const uint8_t* dsk_xq;  // the rows as e4m3 codes [M][H] with ue8m0 scales [M][H / 32] (x is then not read)
  const uint8_t* dsk_xs;
  // Experts stacked by expert id in six tensors of their own (dsk::MoeWeights, ds41f-4xgx10-switchless/engine/kernels/
  // dsk.h:199-209) instead of a pool with descriptors: matrix j (gate, up, down) of expert e at stk_w[j] + e stk_wb[j], its
  // scales at stk_s[j] + e stk_sb[j]. stk_w[0] null: the layer's descriptors.
  const uint8_t* stk_w[3];
  const uint8_t* stk_s[3];
  size_t stk_wb[3], stk_sb[3];
  int* idx_out;     // fused routing: the selection is also written here (idx_out / wts_out of dsk::moe_routed, dsk.h:239-241)
  float* wts_out;
};

int launch_decode_mxfp4_mfma(const DecodeArgs& a, int parts, bool shared_fp8e, hipStream_t st);  // MXFP4 experts (+ FP8_B32E shared)
int launch_decode_fp8(const DecodeArgs& a, int parts, bool shared, hipStream_t st);
int launch_decode_fp8_mfma(const DecodeArgs& a, int parts, bool shared, hipStream_t st);  // variant 1 (moe_decode_mfma.cuh)
int launch_decode_int4(const DecodeArgs& a, int parts, bool shared_bf16, hipStream_t st);
int launch_decode_int4_mfma(const DecodeArgs& a, int parts, int shared_fmt, hipStream_t st);  // variant 1 (shared: 0, BF16 or FP8_B128)
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
  alignas(16) uint32_t mask[DSGX_MAX_EXPERTS / 32];  // the picked experts (read 16 bytes at a time)
  int n;                               // distinct picked experts
  int ri[M * DSGX_MAX_TOPK];
  float rw[M * DSGX_MAX_TOPK];
  float wslot[M * DSGX_MAX_TOPK][M];   // per slot the rows' routing weights (0: the row did not pick it)
  Slot slots[M * DSGX_MAX_TOPK + 1];
  int gen;                             // the grid barrier's generation at kernel start
  int next_up;                         // the gate/up phase's batch counter (up_body)
  int rdone, ready;                    // rows routed so far; the slots are complete (resolve)
  uint4 dtab[DSGX_MAX_EXPERTS * 3];    // the descriptors' first 16 bytes (off, s2, fmt), fetched before the routing is known
};

// The step's set-up comes in two parts, so that the weights that do not depend on the routing (the fused shared
// expert's, slot 0) stream while the routing's dependent memory round trips are under way:
//   prep()     by all threads: clears the tables, fills slot 0 and copies every expert's descriptor into LDS (a load
//              that depends on the routing would take a memory round trip under the weight streams' load: several
//              microseconds); a __syncthreads() follows it;
//   resolve()  by the workgroup's last few wavefronts only ("resolvers", resolver_waves()), without workgroup
//              barriers: with logits routes the rows (a wavefront a row at a time, route()'s code and bits), builds
//              the union of the rows' picks in expert-id order (build_union of the reference, decode.cu:57-106) and
//              the routed slots, then raises S.ready. The other wavefronts stream slot 0 meanwhile and look at
//              S.ready when they need a routed slot (wait_slots()).
// Every workgroup does both for itself.
template <int M> __device__ __forceinline__ constexpr int resolver_waves() { return M < 4 ? M : 4; }
template <int FMT, int SHFMT, int M>
__device__ __forceinline__ void prep(Step<M>& S, const DecodeArgs& a) {
  const int tid = threadIdx.x;
  // every expert's descriptors into S.dtab (their first 16 of 64 bytes), three loads in flight a thread
  // (loads past the end re-read the last descriptor: unconditional loads into named registers stay in flight together)
  const DSGX_GLOBAL u32x4_t* d = (const DSGX_GLOBAL u32x4_t*)(uintptr_t)a.L.desc;
  u32x4_t* tab = reinterpret_cast<u32x4_t*>(S.dtab);
  const int nd = a.stk_w[0] ? 0 : a.L.E * 3, bd = blockDim.x;  // (stacked experts are addressed by their id alone)
  for (int i0 = tid; i0 < nd; i0 += 3 * bd) {
    const int i1 = i0 + bd, i2 = i1 + bd;
    const u32x4_t v0 = d[(size_t)i0 * 4], v1 = d[(size_t)min(i1, nd - 1) * 4], v2 = d[(size_t)min(i2, nd - 1) * 4];
    tab[i0] = v0;
    if (i1 < nd) tab[i1] = v1;
    if (i2 < nd) tab[i2] = v2;
  }
  if (tid < DSGX_MAX_EXPERTS / 32) S.mask[tid] = 0;
  for (int i = tid; i < M * DSGX_MAX_TOPK * M; i += blockDim.x) (&S.wslot[0][0])[i] = 0.f;
  if (tid == 0) {
    S.next_up = 0, S.ready = 0, S.rdone = 0;
    if (SHFMT != 0) {
      Slot t;
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
      S.slots[0] = t;
    }
  }
}
__device__ __forceinline__ size_t al256d(size_t b) { return (b + 255) / 256 * 256; }
template <int FMT>
__device__ __forceinline__ MatRef mat_ref(const uint8_t* base, int N, int K, float s2) {
  MatRef m;
  m.w = base, m.s = nullptr, m.s2 = s2, m.pad = 0;
  if (FMT == DSGX_FMT_FP8_B128 || FMT == DSGX_FMT_FP8_B32E) m.s = base + al256d((size_t)N * K);
  else if (FMT == DSGX_FMT_INT4_G32 || FMT == DSGX_FMT_MXFP4_G32) m.s = base + al256d((size_t)N * K / 2);
  return m;
}
template <int FMT>
__device__ __forceinline__ MatDev mat_dev(const MatRef& r, int N, int K) {
  MatDev m;
  m.w = r.w, m.s = r.s, m.zp = nullptr, m.lrs = m.lks = 7, m.srow = K >> 7, m.s2 = r.s2;
  if (FMT == DSGX_FMT_INT4_G32) m.zp = r.s + al256d((size_t)N * (K / 32) * 2);
  return m;
}
// rw: this resolver's number, nr: how many there are. What a resolver can load before the routing is known it loads
// first, in resolve_fetch() at the start of the kernel (under the weight streams' load a dependent memory round trip
// takes several microseconds): its first row's logits and the bias.
// resolve() follows the workgroup's barrier after prep(). LDS operations of a wavefront complete in program order,
// and the release fences order them before the counter and the flag.
struct ResolveRegs {
  float lg[kRouteRJ], bs[kRouteRJ];
};
template <int M>
__device__ __forceinline__ void resolve_fetch(Step<M>& S, const DecodeArgs& a, int rw, int nr, ResolveRegs& R) {
  const int lane = threadIdx.x & 63, E = a.L.E;
  if (a.logits) {
    route_fetch(rw < M ? a.logits + (size_t)rw * E : nullptr, E, lane, R.lg);
    route_fetch(a.bias, E, lane, R.bs);
  }
}
template <int FMT, int SHFMT, int M>
__device__ __forceinline__ void resolve(Step<M>& S, const DecodeArgs& a, int rw, int nr, ResolveRegs& R) {
  const int lane = threadIdx.x & 63, E = a.L.E, topk = a.L.topk, ne = M * topk;
  const int H = a.L.H, I = a.L.I, nsh = SHFMT != 0 ? 1 : 0;
  __builtin_amdgcn_s_setprio(3);
  // the routed slot of expert e, its place r among the step's experts
  auto make_slot = [&](int e, int r) {
    Slot t;
    auto ref = [&](int which, int N, int K) {
      if (a.stk_w[0]) return MatRef{a.stk_w[which] + (size_t)e * a.stk_wb[which], a.stk_s[which] + (size_t)e * a.stk_sb[which], 1.f, 0};
      const uint4 d = S.dtab[e * 3 + which];
      return mat_ref<FMT>(a.L.pool + (((uint64_t)d.y << 32) | d.x), N, K, __uint_as_float(d.z));
    };
    t.g = ref(0, I, H), t.u = ref(1, I, H), t.d = ref(2, H, I);
    t.hslot = r, t.shared = 0;
    S.slots[nsh + r] = t;
  };
  if constexpr (M == 1) {
    // One row: its picks are the step's experts, and a pick's slot is the number of picks with a lower id - counted in
    // registers, without the tables' round trips through LDS. (Picks handed in by the caller that name an expert twice
    // take the general path below.)
    int id = 0;
    float w = 0.f;
    if (a.logits) route_row(R.lg, R.bs, E, topk, a.route_scale, a.score_fn, lane, id, w);
    else if (lane < topk) id = a.idx[lane], w = a.w[lane];
    int r = 0;
    bool twice = false;
#pragma unroll
    for (int j = 0; j < DSGX_MAX_TOPK; ++j) {
      const int ej = __builtin_amdgcn_readlane(id, j);
      if (j < topk) r += ej < id ? 1 : 0, twice |= ej == id && j != lane;
    }
    if (__ballot(twice && lane < topk) == 0) {
      DSGX_MARKW(9);
      if (lane < topk) {
        if (a.idx_out && blockIdx.x == 0) a.idx_out[lane] = id, a.wts_out[lane] = w;
        S.wslot[r][0] = w;
        make_slot(id, r);
      }
      if (lane == 0) S.n = topk;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      if (lane == 0) __hip_atomic_store(&S.ready, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __builtin_amdgcn_s_setprio(0);
      DSGX_MARKW(2);
      return;
    }
  }
  int mine = 0;
  for (int row = rw; row < M; row += nr, ++mine) {
    int id = 0;
    float w = 0.f;
    if (a.logits) {
      if (row != rw) route_fetch(a.logits + (size_t)row * E, E, lane, R.lg);
      route_row(R.lg, R.bs, E, topk, a.route_scale, a.score_fn, lane, id, w);
    } else if (lane < topk) {
      id = a.idx[row * topk + lane], w = a.w[row * topk + lane];
    }
    if (lane < topk) {
      S.ri[row * topk + lane] = id, S.rw[row * topk + lane] = w;
      atomicOr(&S.mask[id >> 5], 1u << (id & 31));
      if (a.idx_out && blockIdx.x == 0) a.idx_out[row * topk + lane] = id, a.wts_out[row * topk + lane] = w;
    }
  }
  DSGX_MARKW(9);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  int before = 0;
  if (lane == 0) before = __hip_atomic_fetch_add(&S.rdone, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  if (uni(before) + mine < M) {  // another resolver finishes later: it does the rest
    __builtin_amdgcn_s_setprio(0);
    return;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  // the mask in every lane's registers (four 16-byte reads in flight together, not a chain of dependent ones)
  constexpr int NW = DSGX_MAX_EXPERTS / 32;
  static_assert(NW % 4 == 0, "the mask is read 16 bytes at a time");
  uint32_t mk[NW];
#pragma unroll
  for (int j = 0; j < NW; j += 4) {
    const u32x4_t q = *reinterpret_cast<const u32x4_t*>(&S.mask[j]);
    mk[j] = q.x, mk[j + 1] = q.y, mk[j + 2] = q.z, mk[j + 3] = q.w;
  }
  for (int i = lane; i < ne; i += kWave) {
    const int e = S.ri[i];
    int r = 0;  // the picks below e: its slot
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      const uint32_t below = j < (e >> 5) ? 0xFFFFFFFFu : j == (e >> 5) ? (1u << (e & 31)) - 1 : 0u;
      r += __popc(mk[j] & below);
    }
    S.wslot[r][i / topk] = S.rw[i];
    make_slot(e, r);  // (rows that picked the same expert write the same values)
  }
  if (lane == 0) {
    int n = 0;
#pragma unroll
    for (int j = 0; j < NW; ++j) n += __popc(mk[j]);
    S.n = n;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  if (lane == 0) __hip_atomic_store(&S.ready, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  __builtin_amdgcn_s_setprio(0);
  DSGX_MARKW(2);
}
// The number of routed slots, once the resolvers have raised S.ready. No fence after the flag: a wavefront's LDS reads
// are served in order, the compiler barrier keeps them in program order, and a fence would also wait for every
// weight load the caller has in flight.
template <int M>
__device__ __forceinline__ int wait_slots(Step<M>& S) {
  while (__hip_atomic_load(&S.ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == 0) __builtin_amdgcn_s_sleep(2);
  asm volatile("" ::: "memory");
  return uni(*(volatile int*)&S.n);
}

// ---- gate/up ------------------------------------------------------------------------------------------------------------
// Walks slots [s0, s0 + nsl) in format F. INTER: the slot's gate matrix is the BF16 shared expert's interleaved gate/up
// (rows 2c gate, 2c + 1 up). A batch is CH channels of one slot (RB = 2 CH weight rows); batch b is (slot b / nb_e,
// channels CH (b % nb_e)...). Workgroup g of G owns the batches g, g + G, g + 2 G, ... (spread over the slots and the
// memory channels); its waves take them one at a time from a counter in LDS, so that a wave that is served faster
// by the memory system (on a busy CU the older waves are) simply takes more batches, and all waves finish together.
// The claim for the batch after the next is issued a batch ahead: its latency is never waited for.
// The routing is resolved late: the workgroup's batches of slot 0 (nsl0 = 1: a fused shared expert; 0: none) need no
// routing; a wave whose next batch lies beyond them calls wait_nsl(), which waits for the resolvers (wait_slots())
// and returns the number of slots. Every wave calls it before it leaves (its last claim lies beyond any count).
// ---- a sub-batch's dot products, reduced over the lanes ----------------------------------------------------------------
// The RB x M sums of a sub-batch (output q = i * M + m) in groups of up to 16 through fold_sum: own_var<NV>(g, lane) is
// the output of group g that `lane` keeps after reduce_own (-1: none), red[g] its sum.
template <int NV> struct Pow2Ceil { static constexpr int v = NV <= 1 ? 1 : NV <= 2 ? 2 : NV <= 4 ? 4 : NV <= 8 ? 8 : 16; };
template <int NV>
__device__ __forceinline__ int own_var(int g, uint32_t lane) {
  const int n = NV - 16 * g < 16 ? NV - 16 * g : 16;
  int q = -1;
  // (the group's size is a compile-time value in each branch)
  if (n <= 1) q = fold_owner<1>(lane) ? fold_var<1>(lane) : -1;
  else if (n <= 2) q = fold_owner<2>(lane) ? fold_var<2>(lane) : -1;
  else if (n <= 4) q = fold_owner<4>(lane) ? fold_var<4>(lane) : -1;
  else if (n <= 8) q = fold_owner<8>(lane) ? fold_var<8>(lane) : -1;
  else q = fold_owner<16>(lane) ? fold_var<16>(lane) : -1;
  return q >= 0 && q < n ? 16 * g + q : -1;
}
template <int RB, int M, int G>
__device__ __forceinline__ float reduce_group(float (&acc)[RB][M], uint32_t lane) {
  constexpr int NV = RB * M, n = NV - 16 * G < 16 ? NV - 16 * G : 16, NP = Pow2Ceil<n>::v;
  float t[NP];
#pragma unroll
  for (int q = 0; q < NP; ++q) {
    const int idx = 16 * G + q;
    t[q] = 0.f;
    if (idx < NV) t[q] = acc[idx / M][idx % M], acc[idx / M][idx % M] = 0.f;
  }
  return fold_sum<NP>(t, lane);
}
template <int RB, int M>
__device__ __forceinline__ void reduce_own(float (&acc)[RB][M], uint32_t lane, float (&red)[(RB * M + 15) / 16]) {
  red[0] = reduce_group<RB, M, 0>(acc, lane);
  if constexpr (RB * M > 16) red[1] = reduce_group<RB, M, 1>(acc, lane);
  static_assert(RB * M <= 32, "reduce_own: two groups at most");
}

template <int FMT, int M, bool INTER, int CH, int D, class WaitNsl>
__device__ __forceinline__ void up_body(const DecodeArgs& a, const uint4* xs, const Slot* slots, int nsl0, int* counter, int g, int G,
                                        WaitNsl&& wait_nsl) {
  // g, G are wave-uniform (uni()): the cursors below live on the scalar unit
  constexpr int RB = 2 * CH;
  const uint32_t lane = threadIdx.x & 63;
  const int H = a.L.H, I = a.L.I;
  const int nsegk = num_segs<FMT>(H), nq = nsegk * FmtT<FMT>::SEGK / 8;
  const int nb_e = I / CH;
  // (integer division runs on the vector unit: its results are declared uniform again)
  auto batches_of = [&](int nslots) { return uni(g < nslots * nb_e ? (nslots * nb_e - g + G - 1) / G : 0); };
  int nk = batches_of(nsl0);  // the workgroup's batches that can be opened: slot 0's until the routing is resolved
  bool resolved = false;
  Raw w[D][RB];
  int rsl[D], rp[D], rseg[D];  // what each ring entry holds: slot, pair, segment; rseg < 0: nothing
  float acc[RB][M];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[i][m] = 0.f;
  int pending = 0;  // lane 0: the claim in flight
  auto claim = [&]() {
    if (lane == 0) pending = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  RowSrc src[RB];
  int lsl = 0, lp = 0, lseg = 0;
  bool lvalid = true, opened = false;
  // (the INT4 stream waits for the vector unit, where the lane offset's select costs more than the tail's cache lines)
  constexpr bool kTailLine = FMT != DSGX_FMT_INT4_G32;
  auto open = [&]() {  // the next batch of this wave: the claim issued a batch ago; then claims the one after
    const int k = uni(pending);
    claim();
    if (k >= nk && !resolved) nk = batches_of(wait_nsl()), resolved = true;
    lvalid = k < nk;
    lseg = 0;
    // past the end the ring keeps loading: 16 bytes of the wave's last rows (cached, and other lines than the other waves')
    if (kTailLine && !lvalid && opened) return;  // (INT4: the first rows of the first slot, the same for all waves: L1 hits)
    opened = true;
    const int b = lvalid ? g + k * G : 0;
    lsl = uni(b / nb_e), lp = b - lsl * nb_e;
    const Slot& S = slots[lsl];
    MatRef gr{}, ur{};
    gr.w = uni(S.g.w), gr.s = uni(S.g.s), ur.w = uni(S.u.w), ur.s = uni(S.u.s);
    const MatDev gm = mat_dev<FMT>(gr, INTER ? 2 * I : I, H), um = mat_dev<FMT>(ur, I, H);
#pragma unroll
    for (int i = 0; i < RB; ++i) src[i] = INTER ? row_src<FMT>(gm, RB * lp + i, H) : row_src<FMT>(i < CH ? gm : um, CH * lp + i % CH, H);
  };
  claim();
  open();
  auto load = [&](Raw (&r)[RB], int& sl, int& p, int& seg) {
    if (lseg == nsegk) {  // the batch's loads are all issued: the next batch (opened only now, when it is needed)
      if (lvalid) open();
      else lseg = 0;
    }
#pragma unroll
    for (int i = 0; i < RB; ++i) load_row<FMT>(r[i], src[i], lvalid ? lseg : 0, kTailLine && !lvalid ? 0u : lane, 7, acc[i][0]);
    sl = lsl, p = lp, seg = lvalid ? lseg : -1;
    ++lseg;
  };
  auto compute = [&](const Raw (&r)[RB], int csl, int cp, int cseg) {
    step_dot<FMT, M, RB>(r, xs, nq, cseg, lane, acc);
    if (cseg + 1 < nsegk) return;
    // The batch's CH x M gate sums and up sums are reduced over the lanes by two fold_sums (the same tree whatever their
    // number), after which output q = c * M + m (channel c, activation row m) is owned by one lane, which finishes it and
    // stores its 16 bits. The store is coherent at device scope (it bypasses the XCD-local L2): the down phase of the
    // same kernel reads h on other XCDs right after the grid barrier.
    constexpr int NP = Pow2Ceil<CH * M>::v;
    float tg[NP], tu[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) tg[q] = tu[q] = 0.f;
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const int ch = INTER ? i >> 1 : i % CH;
        const bool up = INTER ? (i & 1) : (i >= CH);
        if (up) tu[ch * M + m] = acc[i][m];
        else tg[ch * M + m] = acc[i][m];
        acc[i][m] = 0.f;
      }
    const float gsum = fold_sum<NP>(tg, lane), usum = fold_sum<NP>(tu, lane);
    const int q = fold_var<NP>(lane);
    if (fold_owner<NP>(lane) && q < CH * M) {
      const Slot& S = slots[csl];
      const int c = q / M, m = q % M;
      const uint32_t hb = swiglu_bits(bf16_round(__fmul_rn(gsum, S.g.s2)), bf16_round(__fmul_rn(usum, S.u.s2)));
      uint16_t* dst = a.h + ((size_t)S.hslot * M + m) * I + CH * cp + c;
      __hip_atomic_store((DSGX_GLOBAL uint16_t*)(uintptr_t)dst, (uint16_t)hb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  // software pipeline: a ring of D steps in flight; every turn computes the oldest step and issues a load in its place
#pragma unroll
  for (int d = 0; d < D; ++d) load(w[d], rsl[d], rp[d], rseg[d]);
  for (;;) {
    bool any = lvalid;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (rseg[d] >= 0) compute(w[d], rsl[d], rp[d], rseg[d]), any = true;
      load(w[d], rsl[d], rp[d], rseg[d]);
    }
    if (!any) break;
  }
}

// x staged for format F, then the up phase of this workgroup. With a shared expert of another format (INT4 experts,
// BF16 shared expert) the first `shared_wgs` workgroups do the shared expert's gate/up and the others the routed slots.
// prep() has run; resolve() runs inside (up_body).
template <int FMT, int SHFMT, int M>
__device__ __forceinline__ void up_phase(const DecodeArgs& a, uint4* xs, Step<M>& S, int shared_wgs) {
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  constexpr int kUpCH = M <= 2 ? 1 : 2, kUpD = DSGX_UPD / kUpCH;
  constexpr int nsh = SHFMT != 0 ? 1 : 0, NR = resolver_waves<M>();
  const int H = a.L.H, wave = uni((int)(threadIdx.x >> 6)), nw = blockDim.x >> 6;
  const bool shared_wg = kMixed && (int)blockIdx.x < shared_wgs;
  const bool resolver = wave >= nw - NR;
  ResolveRegs rr;
  if (resolver) resolve_fetch(S, a, wave - (nw - NR), NR, rr);
  prep<FMT, SHFMT, M>(S, a);
  if (shared_wg) stage_x<FmtT<DSGX_FMT_BF16>::KL>(xs, a.x, H, M, H, num_segs<DSGX_FMT_BF16>(H) * 512);
  else stage_x<FmtT<FMT>::KL>(xs, a.x, H, M, H, num_segs<FMT>(H) * FmtT<FMT>::SEGK);
  __syncthreads();
  DSGX_MARK(1);
  if (resolver) resolve<FMT, SHFMT, M>(S, a, wave - (nw - NR), NR, rr);
  if (shared_wg) {
    up_body<kMixed ? DSGX_FMT_BF16 : FMT, M, kMixed, kUpCH, kUpD>(a, xs, S.slots, 1, &S.next_up, blockIdx.x, shared_wgs, [&] {
      wait_slots(S);
      return 1;
    });
  } else if (kMixed) {
    up_body<FMT, M, false, kUpCH, kUpD>(a, xs, S.slots + nsh, 0, &S.next_up, (int)blockIdx.x - shared_wgs, (int)gridDim.x - shared_wgs,
                                        [&] { return wait_slots(S); });
  } else {
    up_body<FMT, M, false, kUpCH, kUpD>(a, xs, S.slots, nsh, &S.next_up, blockIdx.x, gridDim.x, [&] { return nsh + wait_slots(S); });
  }
  // Every wave waits here for its own h stores to be acknowledged by the memory system (the stores are device-scope
  // write-through; the ring's trailing loads, which hit the cache, complete with them). The fused kernel's grid barrier
  // then needs only the workgroup barrier in front of its arrival: a workgroup-scope release alone does not wait for
  // the vector memory counter.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---- down ------------------------------------------------------------------------------------------------------------------
// The wave's rows [n_lo, n_hi) in sub-batches of RB (2, or 3 where the rows divide so: the launch picks); per sub-batch
// every slot in order. hs: LDS for `spc` slots' h.
// `between` runs after the first loads are issued and before any h is read (the fused kernel's grid barrier).
template <int FMT, int SHFMT, int M, int D, int RB, class Between>
__device__ __forceinline__ void down_phase(const DecodeArgs& a, uint4* hs, Step<M>& S, int spc, int n_lo, int n_hi, Between&& between) {
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  constexpr int SF = SHFMT == 0 ? FMT : SHFMT;  // the shared slot's format
  const int H = a.L.H, I = a.L.I;
  const uint32_t lane = threadIdx.x & 63;
  const int nsh = SHFMT != 0 ? 1 : 0, nrouted = uni(S.n), nsl = nsh + nrouted;
  const int nq = I / 8;
  const int segs_r = num_segs<FMT>(I), segs_s = nsh ? num_segs<SF>(I) : 0;
  const int nsub = uni(n_hi > n_lo ? (n_hi - n_lo + RB - 1) / RB : 0);
  const int steps_sub = segs_s + nrouted * segs_r;
  // every wave of the workgroup walks the same number of steps (the barriers around the h chunks)
  __shared__ int s_maxsub;
  if (threadIdx.x == 0) s_maxsub = 0;
  __syncthreads();
  if (lane == 0) atomicMax(&s_maxsub, nsub);

  Raw w[D][RB];
  float acc[RB][M];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
  // A slot's dot products are reduced over the lanes when the slot completes (reduce_own: lane l then holds the sum of
  // ITS output, number own_q of the sub-batch's RB x M), and the lane chains its output's slots in order:
  // y = fma(s2 w, dot, y) with complete dots, as the reference states it (decode.cu:526-566).
  constexpr int NG = (RB * M + 15) / 16;
  float yown[NG], sown[NG];
  int own_q[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) yown[g] = sown[g] = 0.f, own_q[g] = own_var<RB * M>(g, lane);
  int lsub = 0, ls = 0, lseg = 0;  // the load cursor (scalar): sub-batch, slot, segment
  bool lsh = kMixed && nsh > 0;    // the slot under the load cursor is the shared one in another format
  RowSrc src[RB];
  auto open = [&](int sub, int sl) {  // the RB rows of sub-batch `sub` in slot sl's down matrix
    const Slot& T = S.slots[sl];
    MatRef dr{};
    dr.w = uni(T.d.w), dr.s = uni(T.d.s);
    const int n0 = n_lo + sub * RB;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      // a row past the wave's end re-reads its last one (the result is dropped); sub < 0: the matrix's first rows
      const int n = sub < 0 ? min(i, H - 1) : n0 + i < n_hi ? n0 + i : n_hi - 1;
      if (kMixed && sl < nsh) src[i] = row_src<SF>(mat_dev<SF>(dr, H, I), n, I);
      else src[i] = row_src<FMT>(mat_dev<FMT>(dr, H, I), n, I);
    }
  };
  open(nsub > 0 ? 0 : -1, 0);
  auto load = [&](Raw (&r)[RB]) {
    // past the wave's last step the ring keeps loading: 16 bytes of its last rows (cached; other lines than other waves')
    const bool lv = lsub < nsub;
    const int sg = lv || FMT == DSGX_FMT_INT4_G32 ? lseg : 0;
    const uint32_t ll = lv || FMT == DSGX_FMT_INT4_G32 ? lane : 0u;  // (INT4: the select costs its stream more than it saves)
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      if (lsh) load_row<SF>(r[i], src[i], sg, ll, 7, acc[i][0]);
      else load_row<FMT>(r[i], src[i], sg, ll, 7, acc[i][0]);
    }
    if ((lv || FMT == DSGX_FMT_INT4_G32) && ++lseg == (ls < nsh ? segs_s : segs_r)) {
      lseg = 0;
      if (++ls == nsl) ls = 0, ++lsub;
      // (INT4, past the end: the first rows of every slot in turn, the same for all waves - L1 hits; its stream waits
      // for the vector unit, where a select a load costs more than those lines)
      if (lsub < nsub || FMT == DSGX_FMT_INT4_G32) {
        open(lsub < nsub ? lsub : -1, ls);
        lsh = kMixed && ls < nsh;
      }
    }
  };
#pragma unroll
  for (int d = 0; d < D; ++d) load(w[d]);

  between();
  __syncthreads();
  const int maxsub = uni(s_maxsub);
  const bool one_chunk = nsl <= spc;
  const int wg_steps = maxsub * steps_sub;

  int csub = 0, cs = 0, cseg = 0, c0 = 0;  // the compute cursor; c0: first slot of the chunk of h in LDS
  auto stage_chunk = [&]() {  // h of the slots [c0, c0 + spc) into LDS, each slot in its format's lane order
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
  };
  // restage: the step may enter a new chunk of slots (the variant without it is for h that fits LDS whole)
  auto compute = [&](const Raw (&r)[RB], auto restage) {
    const bool live = csub < nsub;
    const bool sh = cs < nsh;
    if constexpr (decltype(restage)::value) {
      if (cseg == 0 && cs == c0) stage_chunk();
    }
    const uint4* xs = hs + (size_t)(cs - c0) * M * nq;
    if (live) {
      if (kMixed && sh) step_dot<SF, M, RB>(r, xs, nq, cseg, lane, acc);
      else step_dot<FMT, M, RB>(r, xs, nq, cseg, lane, acc);
    }
    if (++cseg < (sh ? segs_s : segs_r)) return;
    cseg = 0;
    // the slot is complete: into the outputs' running sums, in slot (= expert id) order
    const float s2 = S.slots[cs].d.s2;
    float red[NG];
    reduce_own<RB, M>(acc, lane, red);
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      if (sh) sown[g] = red[g];
      else yown[g] = fmaf(__fmul_rn(s2, S.wslot[cs - nsh][own_q[g] >= 0 ? own_q[g] % M : 0]), red[g], yown[g]);
    }
    if (++cs < nsl) {
      if (cs == c0 + spc) c0 += spc;
      return;
    }
    cs = 0, c0 = 0;
    // the sub-batch is complete: the owning lanes store output (row n0 + q / M, activation row q % M)
    const int n0 = n_lo + csub * RB;
    ++csub;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      if (live && own_q[g] >= 0) {
        const int i = own_q[g] / M, m = own_q[g] % M;
        if (n0 + i < n_hi) {
          const size_t o = (size_t)m * H + n0 + i;
          float yv = yown[g], sv = sown[g];
          if (SHFMT != 0) a.ys[o] = sv;
          else if (a.ysum) sv = a.ys[o];
          if (a.ysum) yv = __fadd_rn(yv, sv);
          a.yr[o] = yv;
        }
      }
      yown[g] = sown[g] = 0.f;
    }
  };
  if (one_chunk) {
    if (wg_steps > 0) stage_chunk();
    for (int t = 0; t < wg_steps; t += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        if (t + d < wg_steps) compute(w[d], std::false_type{});
        load(w[d]);
      }
    }
  } else {
    for (int t = 0; t < wg_steps; t += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        if (t + d < wg_steps) compute(w[d], std::true_type{});
        load(w[d]);
      }
    }
  }
}

// ---- down, partitioned by slot ---------------------------------------------------------------------------------------------
// For steps whose h does not fit LDS (several rows with a large union): the rows-of-all-slots order above would bring
// every slot's h into every workgroup, as many bytes again as the weights. Here the (slot, row) pairs are cut into equal
// contiguous ranges, one a workgroup: a range spans two or three slots, whose h is staged once each; the complete dot
// products go to memory as f32 [slot][M][H] and k_down_combine chains them in slot order: the same sums, by the same
// tree and in the same order, as down_phase (a row's result is the same bits either way).
template <int F, int M, int D>
__device__ __forceinline__ void down_part_body(const DecodeArgs& a, uint4* hs, const Step<M>& S, int s0, int ns, int g, int G) {
  constexpr int RB = 2;
  const int H = a.L.H, I = a.L.I, nq = I / 8, segs = num_segs<F>(I);
  const uint32_t lane = threadIdx.x & 63;
  const int wave = uni((int)(threadIdx.x >> 6)), nw = blockDim.x >> 6;
  const int sps = (H + RB - 1) / RB;  // sub-batches a slot
  const long total = (long)ns * sps;
  const int t_lo = (int)(total * g / G), t_hi = (int)(total * (g + 1) / G);
  constexpr int NG = (RB * M + 15) / 16;
  int own_q[NG];
#pragma unroll
  for (int q = 0; q < NG; ++q) own_q[q] = own_var<RB * M>(q, lane);
  for (int sl = t_lo / sps; sl * sps < t_hi; ++sl) {  // (the same for every wave of the workgroup)
    const int ta = max(t_lo, sl * sps) - sl * sps, tb = min(t_hi, (sl + 1) * sps) - sl * sps;  // its sub-batches of this slot
    const Slot& T = S.slots[s0 + sl];
    __syncthreads();
    stage_slots<FmtT<F>::KL, false>(hs, 1, M, I, [&](int) { return a.h + (size_t)T.hslot * M * I; });
    __syncthreads();
    MatRef dr{};
    dr.w = uni(T.d.w), dr.s = uni(T.d.s);
    const MatDev dm = mat_dev<F>(dr, H, I);
    float* out = a.dpart + (size_t)(s0 + sl) * M * H;
    const int nsub = uni(tb - ta > wave ? (tb - ta - wave + nw - 1) / nw : 0);  // the wave's: ta + wave, + nw, ...
    if (nsub == 0) continue;
    const int steps = nsub * segs;
    Raw w[D][RB];
    float acc[RB][M];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
    int lsub = 0, lseg = 0, csub = 0, cseg = 0;
    RowSrc src[RB];
    auto open = [&](int sub) {
      const int n0 = (ta + wave + sub * nw) * RB;
#pragma unroll
      for (int i = 0; i < RB; ++i) src[i] = row_src<F>(dm, min(n0 + i, H - 1), I);
    };
    open(0);
    auto load = [&](Raw (&r)[RB]) {
      // past the end the ring keeps loading (unused): 16 bytes of the wave's last rows, one cache line a load
      const bool lv = lsub < nsub;
#pragma unroll
      for (int i = 0; i < RB; ++i) load_row<F>(r[i], src[i], lv ? lseg : 0, lv ? lane : 0u, 7, acc[i][0]);
      if (lv && ++lseg == segs) {
        lseg = 0;
        if (++lsub < nsub) open(lsub);
      }
    };
    auto compute = [&](const Raw (&r)[RB]) {
      step_dot<F, M, RB>(r, hs, nq, cseg, lane, acc);
      if (++cseg < segs) return;
      cseg = 0;
      float red[NG];
      reduce_own<RB, M>(acc, lane, red);
      const int n0 = (ta + wave + csub * nw) * RB;
      ++csub;
#pragma unroll
      for (int q = 0; q < NG; ++q)
        if (own_q[q] >= 0) {
          const int i = own_q[q] / M, m = own_q[q] % M;
          if (n0 + i < H) out[(size_t)m * H + n0 + i] = red[q];
        }
    };
#pragma unroll
    for (int d = 0; d < D; ++d) load(w[d]);
    for (int t = 0; t < steps; t += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        if (t + d < steps) compute(w[d]);
        load(w[d]);
      }
    }
  }
}

template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(DSGX_DECODE_THREADS) k_down_part(DecodeArgs a, int shared_wgs) {
  extern __shared__ uint4 lds[];
  __shared__ Step<M> S;
  constexpr bool kMixed = SHFMT != 0 && SHFMT != FMT;
  constexpr int nsh = SHFMT != 0 ? 1 : 0;
  {
    constexpr int NR = resolver_waves<M>();
    const int wave = uni((int)(threadIdx.x >> 6)), nw = blockDim.x >> 6;
    ResolveRegs rr;
    if (wave >= nw - NR) resolve_fetch(S, a, wave - (nw - NR), NR, rr);
    prep<FMT, SHFMT, M>(S, a);
    __syncthreads();
    if (wave >= nw - NR) resolve<FMT, SHFMT, M>(S, a, wave - (nw - NR), NR, rr);
    __syncthreads();
  }
  const int nrouted = uni(S.n);
  if (blockIdx.x == 0) {  // the slot table for k_down_combine
    if (threadIdx.x == 0) reinterpret_cast<int*>(a.fac)[0] = nrouted;
    for (int i = threadIdx.x; i < nrouted * M; i += blockDim.x)
      a.fac[8 + (i / M) * 8 + i % M] = __fmul_rn(S.slots[nsh + i / M].d.s2, S.wslot[i / M][i % M]);
  }
  if (kMixed) {
    if ((int)blockIdx.x < shared_wgs) down_part_body<SHFMT == 0 ? FMT : SHFMT, M, 4>(a, lds, S, 0, 1, blockIdx.x, shared_wgs);
    else down_part_body<FMT, M, 4>(a, lds, S, 1, nrouted, (int)blockIdx.x - shared_wgs, (int)gridDim.x - shared_wgs);
  } else {
    down_part_body<FMT, M, 4>(a, lds, S, 0, nsh + nrouted, blockIdx.x, gridDim.x);
  }
}

// yr[m][n] = the slots' dots chained in slot (expert id) order, acc = fma(s2 w, dot, acc); ys = the shared slot's dot
template <int M, bool SH>
__global__ void __launch_bounds__(256) k_down_combine(DecodeArgs a) {
  const int H = a.L.H;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= M * H) return;
  const int m = i / H;
  const float* d = a.dpart + (size_t)(SH ? 1 : 0) * M * H + i;
  float acc = 0.f;
  // sixteen slots' loads in flight together (past the end: the last slot again, unused), then their adds in slot order. The
  // first sixteen are loaded before the slot count is known (the buffers hold that many slots whatever the step: stale
  // values past the count are not used), so that a step with up to sixteen slots takes one memory round trip, not two.
  constexpr int B = 16;
  static_assert(B <= DSGX_MAX_UNION, "the first batch lies within the buffers");
  float v[B], f[B];
#pragma unroll
  for (int j = 0; j < B; ++j) v[j] = d[(size_t)j * M * H], f[j] = a.fac[8 + j * 8 + m];
  const int nrouted = reinterpret_cast<const int*>(a.fac)[0];
  for (int s0 = 0; s0 < nrouted; s0 += B) {
    if (s0 > 0) {
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const int s = min(s0 + j, nrouted - 1);
        v[j] = d[(size_t)s * M * H], f[j] = a.fac[8 + s * 8 + m];
      }
    }
#pragma unroll
    for (int j = 0; j < B; ++j)
      if (s0 + j < nrouted) {
        // DeepSeek's fold: the outputs of the experts the row picked (their routing weight, never zero, went in before
        // w2), each rounded to bf16, added in expert-id order (ds41f engine/kernels/moe.cu:974-981)
        if (a.dsk) acc = f[j] != 0.f ? __fadd_rn(acc, bf16_round(v[j])) : acc;
        else acc = fmaf(f[j], v[j], acc);
      }
  }
  float sv = 0.f;
  if (SH) a.ys[i] = sv = a.dsk ? bf16_round(a.dpart[i]) : a.dpart[i];
  else if (a.ysum) sv = a.ys[i];
  if (a.ysum || (a.dsk && SH)) acc = __fadd_rn(acc, sv);  // (DeepSeek: the shared expert last, always)
  a.yr[i] = acc;
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
// The two halves, both for one thread of the workgroup, after a workgroup barrier that follows every wave's wait for its own
// h stores. arrive counts the workgroup in (and, as the very last, releases everyone: it then returns true); wait polls the
// group's release word. Work placed between the two (the down phase's first loads) overlaps the counters' round trips.
// (Measured alternatives, all slower: one counter that every waiter polls - the polls delay the arrivals' adds by
// microseconds; no counter at all, every workgroup polling h itself at the memory side - 256 readers of the same few KiB
// queue on its memory channels; an extra wave a workgroup that stages h in the background - its loads wait behind the
// streaming waves' and it saw the first slot whole only when its workgroup's stream had ended.)
__device__ __forceinline__ bool grid_barrier_arrive(int* bar, int my_gen) {
  const int g = blockIdx.x % kBarGroups;
  const int members = ((int)gridDim.x - g + kBarGroups - 1) / kBarGroups;
  const int groups = min((int)gridDim.x, kBarGroups);
  int* rel = bar + (kBarGroups + 1) * kBarLine;
  if (__hip_atomic_fetch_add(bar + g * kBarLine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == members - 1) {
    __hip_atomic_store(bar + g * kBarLine, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (__hip_atomic_fetch_add(bar + kBarGroups * kBarLine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == groups - 1) {
      __hip_atomic_store(bar + kBarGroups * kBarLine, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      for (int i = 0; i < kBarGroups; ++i) __hip_atomic_store(rel + i * kBarLine, my_gen + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return true;
    }
  }
  return false;
}
__device__ __forceinline__ void grid_barrier_wait(int* bar, int my_gen, int spin_limit) {
  const int g = blockIdx.x % kBarGroups;
  int* rel = bar + (kBarGroups + 1) * kBarLine;
  int spins = 0;
  while (bar_load(rel + g * kBarLine) == my_gen) {
    __builtin_amdgcn_s_sleep(8);
    if (++spins > spin_limit) {
      __hip_atomic_store(bar + (2 * kBarGroups + 1) * kBarLine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
  }
}
__device__ __forceinline__ void grid_barrier(int* bar, int my_gen, int spin_limit) {
  // h was stored with device-scope write-through stores and every wave has waited for its own to complete (the
  // s_waitcnt vmcnt(0) that ends the gate/up phase), so after the workgroup barrier all of this workgroup's h is in
  // memory and no cache write-back or invalidate is needed around the counters (a device-scope fence would flush the
  // whole L2 here)
  __syncthreads();
  if (threadIdx.x == 0 && !grid_barrier_arrive(bar, my_gen)) grid_barrier_wait(bar, my_gen, spin_limit);
  __syncthreads();
}

// ---- kernels ----------------------------------------------------------------------------------------------------------------
template <int FMT, int SHFMT, int M, int RBD>
__global__ void __launch_bounds__(DSGX_DECODE_THREADS) k_decode(DecodeArgs a, int shared_wgs, int spc) {
  extern __shared__ uint4 lds[];
  __shared__ Step<M> S;
  DSGX_MARK(0);
  if (threadIdx.x == 0) S.gen = grid_barrier_gen(a.bar);
  up_phase<FMT, SHFMT, M>(a, lds, S, shared_wgs);
  DSGX_MARK(4);
  const int H = a.L.H, GW = gridDim.x * (blockDim.x >> 6), gw = uni((int)(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)));
  const int rpw = uni((H + GW - 1) / GW);
  const int n_lo = min(H, gw * rpw), n_hi = min(H, n_lo + rpw);
  // the workgroup is counted in before the down phase issues its first loads; it waits for the release after them
  __shared__ int s_released;
  __syncthreads();
  if (threadIdx.x == 0) s_released = grid_barrier_arrive(a.bar, S.gen) ? 1 : 0;
  down_phase<FMT, SHFMT, M, DSGX_DOWND, RBD>(a, lds, S, spc, n_lo, n_hi, [&] {
    DSGX_MARK(5);
    if (threadIdx.x == 0 && !s_released) grid_barrier_wait(a.bar, S.gen, a.spin_limit);
    __syncthreads();
    DSGX_MARK(6);
  });
  DSGX_MARK(8);
}
template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(DSGX_DECODE_THREADS) k_up(DecodeArgs a, int shared_wgs) {
  extern __shared__ uint4 lds[];
  __shared__ Step<M> S;
  up_phase<FMT, SHFMT, M>(a, lds, S, shared_wgs);
}
template <int FMT, int SHFMT, int M>
__global__ void __launch_bounds__(256) k_down(DecodeArgs a, int spc) {
  extern __shared__ uint4 lds[];
  __shared__ Step<M> S;
  {
    constexpr int NR = resolver_waves<M>();
    const int wave = uni((int)(threadIdx.x >> 6)), nw = blockDim.x >> 6;
    ResolveRegs rr;
    if (wave >= nw - NR) resolve_fetch(S, a, wave - (nw - NR), NR, rr);
    prep<FMT, SHFMT, M>(S, a);
    __syncthreads();
    if (wave >= nw - NR) resolve<FMT, SHFMT, M>(S, a, wave - (nw - NR), NR, rr);
    __syncthreads();
  }
  const int H = a.L.H, gw = uni((int)(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)));
  const int n_lo = min(H, gw * 2), n_hi = min(H, n_lo + 2);
  down_phase<FMT, SHFMT, M, 4, 2>(a, lds, S, spc, n_lo, n_hi, [] {});
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
  // h of a chunk of slots in LDS for the down phase: all of them when they fit (96 KiB with one workgroup a CU, 40 with two; the kernels' own tables take up to 36 KiB)
  const size_t slot_bytes = (size_t)M * I * 2;
  auto slots_per_chunk = [&](size_t lds_bytes) { return std::min(std::max(1, (int)(lds_bytes / slot_bytes)), nsl_max); };
  auto shared_split = [&](int grid) {
    if (!kMixed) return 0;
    // the workgroups split between the BF16 shared expert and the routed experts by their bytes, an INT4 byte counted
    // as 2.45 BF16 bytes (it holds four times the values, and the gate/up phase is bound by their decoding)
    const double bsh = 2.0 * I * H * 2, bro = 2.45 * (double)std::min(a.M * a.L.topk, a.L.E) * 2.0 * (double)dsgx_mat_bytes(FMT, I, H);
    return std::max(1, std::min(grid - 1, (int)(grid * bsh / (bsh + bro) + 0.5)));
  };
  (void)SF;
  // h of all the slots does not fit a workgroup's LDS: gate/up as its own launch, then the down phase partitioned by
  // slot and its combine (three launches; every row's bits are those of the other paths)
  const bool part_ok = slot_bytes <= 64 * 1024;
  if ((parts & 2) && part_ok && nsl_max > slots_per_chunk(parts == 3 && DSGX_WGS == 1 ? 96 * 1024 : 40 * 1024)) {
    if (parts & 1) {
      auto kern = k_up<FMT, SHFMT, M>;
      if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_up)) return rc;
      const int grid = cus * DSGX_WGS;
      hipLaunchKernelGGL(kern, dim3(grid), dim3(DSGX_DECODE_THREADS), lds_up, st, a, shared_split(grid));
      DSGX_HIP(hipGetLastError());
    }
    auto kern = k_down_part<FMT, SHFMT, M>;
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), slot_bytes)) return rc;
    const int grid = cus * DSGX_WGS;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(DSGX_DECODE_THREADS), slot_bytes, st, a, shared_split(grid));
    DSGX_HIP(hipGetLastError());
    if (SHFMT != 0) hipLaunchKernelGGL((k_down_combine<M, true>), dim3((M * H + 255) / 256), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((k_down_combine<M, false>), dim3((M * H + 255) / 256), dim3(256), 0, st, a);
    DSGX_HIP(hipGetLastError());
    return DSGX_OK;
  }
  if (parts == 3) {
    // rows a wave in the down phase: sub-batches of three where that divides them evenly (built for the INT4 layers,
    // whose hidden size 6144 gives three rows a wave on 256 CUs), else of two
    const int rpw = (H + cus * (DSGX_DECODE_THREADS / 64) - 1) / (cus * (DSGX_DECODE_THREADS / 64));
#ifdef DSGX_NO_RB3
    const bool rb3 = false;
#else
    const bool rb3 = FMT == DSGX_FMT_INT4_G32 && rpw % 3 == 0;
#endif
    auto kern = rb3 ? k_decode<FMT, SHFMT, M, (FMT == DSGX_FMT_INT4_G32 ? 3 : 2)> : k_decode<FMT, SHFMT, M, 2>;
    const int spc = slots_per_chunk(DSGX_WGS == 1 ? 96 * 1024 : 40 * 1024);
    const size_t lds = std::max(lds_up, (size_t)spc * slot_bytes);
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
    // every workgroup must be resident: the grid comes from the occupancy of this kernel with this much LDS
    int per_cu = 0;
    DSGX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, DSGX_DECODE_THREADS, lds));
    if (per_cu >= 1) {
      per_cu = std::min(per_cu, DSGX_WGS);
      const int grid = cus * per_cu;
      hipLaunchKernelGGL(kern, dim3(grid), dim3(DSGX_DECODE_THREADS), lds, st, a, shared_split(grid), spc);
      DSGX_HIP(hipGetLastError());
      return DSGX_OK;
    }
    // (no resident grid possible: fall through to the two kernels)
  }
  if (parts & 1) {
    auto kern = k_up<FMT, SHFMT, M>;
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_up)) return rc;
    const int grid = cus * DSGX_WGS;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(DSGX_DECODE_THREADS), lds_up, st, a, shared_split(grid));
    DSGX_HIP(hipGetLastError());
  }
  if (parts & 2) {
    auto kern = k_down<FMT, SHFMT, M>;
    const int spc = slots_per_chunk(40 * 1024);
    const size_t lds_down = (size_t)spc * slot_bytes;
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
