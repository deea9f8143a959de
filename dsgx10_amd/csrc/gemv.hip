// Dense GEMV for 1-16 activation rows over FP8-128x128, INT4-g32 and BF16 weights: the gfx950 counterpart of the
// reference's glm::gemv (altar1-4xgx10-switchless/engine/attn/gemv.cu:173-333, attn.h:59-123).
//
//   y[r][n] = sum_k x[r][k] W[n][k], f32 accumulation, outputs bf16 / f32 / SwiGLU (gemv.cu:138-170).
//   FP8: per 128-k block the unscaled f32 sum, then acc = fma(S, sum, acc) (gemv.cu:230-244, micro/gemv.cu:512);
//   INT4: W = bf16_rne((u - u_z) s) per element in registers (attn_common.cuh:65-76), then as BF16.
//
// One wavefront owns RB rows of W and the whole of K (rowdot.cuh); the grid is sized to the chip and walks the row
// batches round-robin. The order of the adds inside a dot product is not the reference's (not part of its contract).
#include "abi_internal.h"
#include "addnorm.cuh"
#include "rowdot.cuh"

namespace dsgx {
namespace {

constexpr int kMaxSegs = 4;  // attn.h:94
struct GemvSegDev {
  MatDev m;
  void* y;
  int n, ldy, row0;
};
struct GemvArgs {
  const uint16_t* x;
  int ldx, K, nq, nsegk, nsegs, total_rows, out, splitk;
  GemvSegDev sg[kMaxSegs];
  NormIn norm;  // norm.part set: the rows are not read from x but made here, xn = RMSNorm(bf16(res + part)) (dsgx_add_norm_gemv)
};

// The activation rows into LDS: from x, or (fused add + norm) computed by this workgroup from the partial sums and the
// residual - every workgroup makes all M rows for itself (M H values: a few KB from L2), workgroup 0 also writes the new
// residual and the normed rows to memory for the kernels that follow.
template <int KL, int M>
__device__ __forceinline__ void stage_rows(uint4* xs, const GemvArgs& a, float* red) {
  if (!a.norm.part) {
    stage_x<KL>(xs, a.x, a.ldx, M, a.K, a.nq * 8);
    return;
  }
  const bool writer = blockIdx.x == 0;
  const int H = a.K;
#pragma unroll 1
  for (int m = 0; m < M; ++m)
    add_norm_row(a.norm, m, H, red, true,
                 [&](int q, u32x4_t v) { if (writer && a.norm.res_out) *reinterpret_cast<u32x4_t*>(a.norm.res_out + (size_t)m * H + 8 * q) = v; },
                 [&](int q, u32x4_t v) {
                   xs[(size_t)m * a.nq + xchunk_index<KL>(q)] = make_uint4(v.x, v.y, v.z, v.w);
                   if (writer && a.norm.xn) *reinterpret_cast<u32x4_t*>(a.norm.xn + (size_t)m * H + 8 * q) = v;
                 });
}

template <int FMT, int M, int RB, int D>
__global__ void __launch_bounds__(256) k_gemv(GemvArgs a) {
  extern __shared__ uint4 xs[];
  __shared__ float red[4];
  const int lane = threadIdx.x & 63;
  // (the wave's number is the same in every lane: said so, which keeps the row cursors and the segment's descriptor on the
  // scalar unit - read from a vector register they came through vector loads of the kernel's arguments, which a wave's
  // weight loads then queued behind, one ring entry after the other)
  const int gw = uni(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)), GW = gridDim.x * (blockDim.x >> 6);
  const int nbatch = a.total_rows / RB;
  const int nmine = gw < nbatch ? (nbatch - gw + GW - 1) / GW : 0;
  const int nsteps = nmine * a.nsegk;

  auto locate = [&](int row, int& si) {
    si = 0;
#pragma unroll
    for (int i = 1; i < kMaxSegs; ++i)
      if (i < a.nsegs && row >= a.sg[i].row0) si = i;
  };
  Raw w[D][RB];
  float acc[RB][M];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
  // where the loads past the last step go: the first 16 bytes of this wave's first row (cached; a line of its own, not one
  // that every wave of the launch reads)
  const uint8_t* dummy;
  {
    const int row = min(gw * RB, a.total_rows - 1);
    int si = 0;
    if (a.nsegs > 1) locate(row, si);
    dummy = a.sg[si].m.w + (size_t)(row - a.sg[si].row0) * FmtT<FMT>::row_bytes(a.K);
  }
  int lt = 0, lj = 0, lseg = 0;  // the load cursor: step, batch number of this wave, segment
  // the matrix of the batch under the load cursor and the batch's first row in it: fetched from the kernel's arguments when
  // the cursor enters a batch, not at every step (scalar loads, but each is a wait in front of the step's weight loads)
  // (a call with one segment, the common one, fetches once: every later fetch would be two dependent scalar round trips)
  MatDev lm = a.sg[0].m;
  int lrow = 0;
  auto enter = [&]() {
    const int row = lt < nsteps ? (gw + lj * GW) * RB : 0;
    int row0 = 0;
    if (a.nsegs > 1) {
      int si;
      locate(row, si);
      lm = a.sg[si].m, row0 = a.sg[si].row0;
    }
    lrow = row - row0;
  };
  enter();
  auto load = [&](Raw (&r)[RB]) {
    const bool ok = lt < nsteps;
    ++lt;
#pragma unroll
    for (int i = 0; i < RB; ++i) load_raw<FMT, true>(r[i], lm, lrow + i, lseg, lane, a.K, acc[i][0], ok ? nullptr : dummy);
    if (ok && ++lseg == a.nsegk) {
      lseg = 0, ++lj;
      enter();
    }
  };
  int cj = 0, cseg = 0;
  auto compute = [&](const Raw (&raw)[RB]) {
    step_dot<FMT, M, RB, true>(raw, xs, a.nq, cseg, lane, acc, a.K);
    if (++cseg < a.nsegk) return;
    cseg = 0;
    // the batch is complete: add the lanes' partials, lane r * M + m keeps output (row r, activation row m)
    const int row = (gw + cj * GW) * RB;
    ++cj;
    float mine = 0.f, mine2 = 0.f;
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const float v = wave_sum(acc[i][m]);
        acc[i][m] = 0.f;
        if (lane == i * M + m) mine = v;
        if (lane == (i ^ 1) * M + m) mine2 = v;  // the pair's other row (SwiGLU)
      }
    if (lane >= RB * M) return;
    int si = 0;
    if (a.nsegs > 1) locate(row, si);
    const GemvSegDev& sg = a.sg[si];
    const int r = lane / M, m = lane % M, n = row - sg.row0 + r;
    if (a.out == DSGX_OUT_BF16) {
      static_cast<uint16_t*>(sg.y)[(size_t)m * sg.ldy + n] = (uint16_t)f32_to_bf16_bits(mine);
    } else if (a.out == DSGX_OUT_F32) {
      static_cast<float*>(sg.y)[(size_t)m * sg.ldy + n] = mine;
    } else if ((r & 1) == 0) {  // SwiGLU: row 2i gate, 2i + 1 up -> column i (gemv.cu:164-168)
      static_cast<uint16_t*>(sg.y)[(size_t)m * sg.ldy + n / 2] = (uint16_t)swiglu_bits(bf16_round(mine), bf16_round(mine2));
    }
  };
  // the first weight loads are issued before the activations are staged: one memory round trip, not two, before the
  // first product (these calls are a few microseconds long: latency is most of them)
#pragma unroll
  for (int d = 0; d < D; ++d) load(w[d]);
  stage_rows<FmtT<FMT>::KL, M>(xs, a, red);
  __syncthreads();
  for (int t = 0; t < nsteps; t += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (t + d < nsteps) compute(w[d]);
      load(w[d]);
    }
  }
}

// Split-K (engine/attn/attn.h:119 of the reference: warps of a CTA share a tile's k range, for small N): a workgroup of
// four waves holds 4 / SK row batches, the SK waves of a batch take the K segments slice, slice + SK, ... of its rows;
// the waves' sums meet in LDS and the batch's first wave adds them in slice order (a fixed order, as the reference's
// finish(), gemv.cu:138-151), then the epilogue of k_gemv. One batch a group and launch: this form is for matrices of
// few rows, where whole-K waves would leave most of the chip idle and walk K in several dependent round trips.
template <int FMT, int M, int RB, int SK>
__global__ void __launch_bounds__(256) k_gemv_sk(GemvArgs a) {
  extern __shared__ uint4 xs[];
  __shared__ float part[4][RB * M];
  __shared__ float red[4];
  const int lane = threadIdx.x & 63, wave = uni(threadIdx.x >> 6);  // (uniform: the segment's descriptor stays on the scalar unit)
  constexpr int GPW = 4 / SK;  // batches a workgroup
  const int grp = wave / SK, slice = wave % SK;
  const int nbatch = a.total_rows / RB;
  const int batch = blockIdx.x * GPW + grp;
  const bool live = batch < nbatch;
  const int row = live ? batch * RB : 0;
  int si = 0;
#pragma unroll
  for (int i = 1; i < kMaxSegs; ++i)
    if (i < a.nsegs && row >= a.sg[i].row0) si = i;
  const GemvSegDev& sg = a.sg[si];
  const int nmine = live && slice < a.nsegk ? (a.nsegk - slice + SK - 1) / SK : 0;  // this wave's segments
  constexpr int D = 4;
  Raw w[D][RB];
  float acc[RB][M];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
  // (loads past the last step: the first 16 bytes of this wave's row)
  const uint8_t* dummy = reinterpret_cast<const uint8_t*>(sg.m.w) + (size_t)(row - sg.row0) * FmtT<FMT>::row_bytes(a.K);
  int lt = 0;
  auto load = [&](Raw (&r)[RB]) {
    const bool ok = lt < nmine;
    const int seg = slice + (ok ? lt : 0) * SK;
    ++lt;
#pragma unroll
    for (int i = 0; i < RB; ++i) load_raw<FMT, true>(r[i], sg.m, row - sg.row0 + i, seg, lane, a.K, acc[i][0], ok ? nullptr : dummy);
  };
#pragma unroll
  for (int d = 0; d < D; ++d) load(w[d]);
  stage_rows<FmtT<FMT>::KL, M>(xs, a, red);
  __syncthreads();
  for (int t = 0; t < nmine; t += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (t + d < nmine) step_dot<FMT, M, RB, true>(w[d], xs, a.nq, slice + (t + d) * SK, lane, acc, a.K);
      load(w[d]);
    }
  }
  // the wave's sums over its lanes, value (i, m) kept by lane i * M + m
  float mine = 0.f;
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float v = wave_sum(acc[i][m]);
      if (lane == i * M + m) mine = v;
    }
  if (lane < RB * M) part[wave][lane] = mine;
  __syncthreads();
  if (!live || slice != 0 || lane >= RB * M) return;
  float sum = part[grp * SK][lane];
#pragma unroll
  for (int k = 1; k < SK; ++k) sum = __fadd_rn(sum, part[grp * SK + k][lane]);
  const int r = lane / M, m = lane % M, n = row - sg.row0 + r;
  if (a.out == DSGX_OUT_BF16) {
    static_cast<uint16_t*>(sg.y)[(size_t)m * sg.ldy + n] = (uint16_t)f32_to_bf16_bits(sum);
  } else if (a.out == DSGX_OUT_F32) {
    static_cast<float*>(sg.y)[(size_t)m * sg.ldy + n] = sum;
  } else if ((r & 1) == 0) {  // SwiGLU: row 2i gate, 2i + 1 up -> column i; the up row's sum sits M lanes further
    float up = part[grp * SK][lane + M];
#pragma unroll
    for (int k = 1; k < SK; ++k) up = __fadd_rn(up, part[grp * SK + k][lane + M]);
    static_cast<uint16_t*>(sg.y)[(size_t)m * sg.ldy + n / 2] = (uint16_t)swiglu_bits(bf16_round(sum), bf16_round(up));
  }
}

template <int FMT, int M, int SK>
int launch_gemv_sk(const GemvArgs& a, hipStream_t st) {
  constexpr int RB = 2;
  const size_t lds = (size_t)M * a.nq * 16;
  const int nbatch = a.total_rows / RB, gpw = 4 / SK;
  auto kern = k_gemv_sk<FMT, M, RB, SK>;
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
  hipLaunchKernelGGL(kern, dim3((nbatch + gpw - 1) / gpw), dim3(256), lds, st, a);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}

template <int FMT, int M, int RB>
int launch_gemv(const GemvArgs& a, hipStream_t st) {
  constexpr int D = 4;
  const size_t lds = (size_t)M * a.nq * 16;
  const int nbatch = a.total_rows / RB;
  // two workgroups of four wavefronts a CU when the activations leave room in LDS, never more workgroups than batches
  const int per_cu = lds <= 64 * 1024 ? 2 : 1;
  int grid = num_cus_cached() * per_cu;
  if (grid > (nbatch + 3) / 4) grid = (nbatch + 3) / 4;
  if (grid < 1) grid = 1;
  auto kern = k_gemv<FMT, M, RB, D>;
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, a);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}
template <int FMT, int M>
int launch_gemv_rb(const GemvArgs& a, hipStream_t st) {
  // split-K as asked for, where the rows are few enough for one batch a wave group and launch
  if (a.splitk > 1 && a.total_rows / 2 <= 16 * num_cus_cached()) {
    if (a.splitk == 2) return launch_gemv_sk<FMT, M, 2>(a, st);
    return launch_gemv_sk<FMT, M, 4>(a, st);
  }
  // few rows: two rows a wavefront so that every wavefront of the launch (two workgroups of four a CU) has rows to stream
  if (a.total_rows / 4 < 2 * 8 * num_cus_cached()) return launch_gemv<FMT, M, 2>(a, st);
  return launch_gemv<FMT, M, 4>(a, st);
}
template <int FMT>
int launch_gemv_m(int M, const GemvArgs& a, hipStream_t st) {
  switch (M) {
    case 1: return launch_gemv_rb<FMT, 1>(a, st);
    case 2: return launch_gemv_rb<FMT, 2>(a, st);
    case 3: return launch_gemv_rb<FMT, 3>(a, st);
    case 4: return launch_gemv_rb<FMT, 4>(a, st);
    case 5: return launch_gemv_rb<FMT, 5>(a, st);
    case 6: return launch_gemv_rb<FMT, 6>(a, st);
    case 7: return launch_gemv_rb<FMT, 7>(a, st);
    case 8: return launch_gemv_rb<FMT, 8>(a, st);
  }
  return fail(DSGX_EINVAL, "gemv: %d rows a launch", M);
}

int ilog2_exact(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return (1 << l) == v ? l : -1;
}

// one launch: the segments of one format (gemv_one of the reference, gemv.cu:459-516)
int gemv_one(int fmt, const uint16_t* x, int ldx, int rows, int K, const dsgx_gemv_seg* segs, int nseg, int out, int splitk, hipStream_t st,
             const NormIn* norm = nullptr) {
  GemvArgs a{};
  a.x = x, a.ldx = ldx, a.K = K, a.out = out, a.nsegs = nseg, a.splitk = splitk;
  if (norm) a.norm = *norm;
  const int segk = fmt == DSGX_FMT_FP8_B128 ? 1024 : fmt == DSGX_FMT_INT4_G32 ? 2048 : 512;
  a.nsegk = (K + segk - 1) / segk;
  a.nq = a.nsegk * segk / 8;
  int row0 = 0;
  for (int i = 0; i < nseg; ++i) {
    const dsgx_gemv_seg& g = segs[i];
    GemvSegDev& d = a.sg[i];
    d.m.w = static_cast<const uint8_t*>(g.w);
    d.m.s = static_cast<const uint8_t*>(g.s);
    d.m.zp = static_cast<const uint8_t*>(g.zp);
    d.m.s2 = 1.f;
    if (!g.w || !g.y) return fail(DSGX_EINVAL, "gemv: segment %d has a null weight or output", i);
    if (fmt == DSGX_FMT_FP8_B128) {
      d.m.lrs = ilog2_exact(g.rs), d.m.lks = ilog2_exact(g.ks);
      if (!g.s || d.m.lrs < 0 || d.m.lks < 4 || K % g.ks) return fail(DSGX_EINVAL, "gemv: FP8 segment %d scale block %dx%d (powers of two, k >= 16)", i, g.rs, g.ks);
      if (out == DSGX_OUT_SWIGLU) return fail(DSGX_EUNSUPPORTED, "gemv: SwiGLU output over FP8 weights is not built");
      d.m.srow = K >> d.m.lks;
    } else if (fmt == DSGX_FMT_INT4_G32) {
      if (!g.s || !g.zp) return fail(DSGX_EINVAL, "gemv: INT4 segment %d needs scales and zero points", i);
    }
    d.y = g.y, d.n = g.n, d.ldy = g.ldy, d.row0 = row0;
    row0 += g.n;
  }
  a.total_rows = row0;
  if (rows > 8) return fail(DSGX_EINVAL, "gemv_one: %d rows", rows);
  switch (fmt) {
    case DSGX_FMT_FP8_B128: return launch_gemv_m<DSGX_FMT_FP8_B128>(rows, a, st);
    case DSGX_FMT_INT4_G32: return launch_gemv_m<DSGX_FMT_INT4_G32>(rows, a, st);
    case DSGX_FMT_BF16: return launch_gemv_m<DSGX_FMT_BF16>(rows, a, st);
  }
  return fail(DSGX_EFORMAT, "gemv: format %d", fmt);
}

}  // namespace
}  // namespace dsgx

using namespace dsgx;

extern "C" int dsgx_gemv(const uint16_t* x, int ldx, int rows, int K, const dsgx_gemv_seg* segs, int nseg, int out, int splitk,
                         void* stream) {
  // argument checks of the reference (gemv.cu:524-543): it dies, this returns an error
  if (rows < 1 || rows > DSGX_MAX_ROWS) return fail(DSGX_EINVAL, "gemv: %d rows", rows);
  if (!x || !segs || nseg < 1 || nseg > kMaxSegs) return fail(DSGX_EINVAL, "gemv: K %d, %d segments", K, nseg);
  if (K < 32 || K % 32 || ldx < K || ldx % 8) return fail(DSGX_EINVAL, "gemv: K %d (a multiple of 32), ldx %d (>= K, a multiple of 8)", K, ldx);
  if (splitk != 1 && splitk != 2 && splitk != 4) return fail(DSGX_EINVAL, "gemv: splitk %d", splitk);
  if (out != DSGX_OUT_BF16 && out != DSGX_OUT_F32 && out != DSGX_OUT_SWIGLU) return fail(DSGX_EINVAL, "gemv: output kind %d", out);
  for (int i = 0; i < nseg; ++i) {
    const int f = segs[i].fmt;
    if (f != DSGX_FMT_BF16 && f != DSGX_FMT_INT4_G32 && f != DSGX_FMT_FP8_B128)
      return fail(DSGX_EFORMAT, "gemv: segment %d has no supported weight format (%d)", i, f);
    if (segs[i].n < 8 || segs[i].n % 8) return fail(DSGX_EINVAL, "gemv: segment %d has %d rows", i, segs[i].n);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  // one launch a format, in the order BF16, INT4, FP8 (outputs do not depend on it); more than 8 activation rows run
  // as two passes over the weights
  for (int fmt : {DSGX_FMT_BF16, DSGX_FMT_INT4_G32, DSGX_FMT_FP8_B128}) {
    dsgx_gemv_seg g[kMaxSegs];
    int n = 0;
    for (int i = 0; i < nseg; ++i)
      if (segs[i].fmt == fmt) g[n++] = segs[i];
    if (!n) continue;
    for (int r0 = 0; r0 < rows; r0 += 8) {
      const int nr = rows - r0 < 8 ? rows - r0 : 8;
      dsgx_gemv_seg gg[kMaxSegs];
      for (int i = 0; i < n; ++i) {
        gg[i] = g[i];
        const size_t esz = out == DSGX_OUT_F32 ? 4 : 2;
        gg[i].y = static_cast<uint8_t*>(g[i].y) + (size_t)r0 * g[i].ldy * esz;
      }
      const int rc = gemv_one(fmt, x + (size_t)r0 * ldx, ldx, nr, K, gg, n, out, splitk, st);
      if (rc) return rc;
    }
  }
  return DSGX_OK;
}

// The residual add + RMSNorm of dsgx_add_norm as the GEMV's prologue: x = the normed rows, made inside the GEMV kernel.
extern "C" int dsgx_add_norm_gemv(const dsgx_norm_in* n, int rows, int K, const dsgx_gemv_seg* segs, int nseg, int out, int splitk, void* stream) {
  if (!n || !n->part || !n->res || !n->w) return fail(DSGX_EINVAL, "add_norm_gemv: the partial sums, the residual and the norm's weight are needed");
  if (rows < 1 || rows > 8) return fail(DSGX_EUNSUPPORTED, "add_norm_gemv: %d rows (1..8; more: dsgx_add_norm, then dsgx_gemv)", rows);
  if (K < 2048 || K % 2048 || K > 16384) return fail(DSGX_EINVAL, "add_norm_gemv: hidden %d (a multiple of 2048 up to 16384)", K);
  if (n->res_out == n->res) return fail(DSGX_EINVAL, "add_norm_gemv: res_out must not be res (every workgroup reads the residual while one writes the new one)");
  if (!segs || nseg < 1 || nseg > kMaxSegs) return fail(DSGX_EINVAL, "add_norm_gemv: %d segments", nseg);
  if (splitk != 1 && splitk != 2 && splitk != 4) return fail(DSGX_EINVAL, "add_norm_gemv: splitk %d", splitk);
  if (out != DSGX_OUT_BF16 && out != DSGX_OUT_F32 && out != DSGX_OUT_SWIGLU) return fail(DSGX_EINVAL, "add_norm_gemv: output kind %d", out);
  const int f = segs[0].fmt;
  if (f != DSGX_FMT_BF16 && f != DSGX_FMT_INT4_G32 && f != DSGX_FMT_FP8_B128) return fail(DSGX_EFORMAT, "add_norm_gemv: no supported weight format (%d)", f);
  for (int i = 0; i < nseg; ++i) {
    if (segs[i].fmt != f) return fail(DSGX_EUNSUPPORTED, "add_norm_gemv: the segments of one call share a format (one launch)");
    if (segs[i].n < 8 || segs[i].n % 8) return fail(DSGX_EINVAL, "add_norm_gemv: segment %d has %d rows", i, segs[i].n);
  }
  const NormIn ni{n->part, n->part2, n->res, n->res_out, n->w, n->xn, n->eps, n->round2};
  return gemv_one(f, nullptr, K, rows, K, segs, nseg, out, splitk, static_cast<hipStream_t>(stream), &ni);
}
