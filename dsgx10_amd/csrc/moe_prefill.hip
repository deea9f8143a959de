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
// The GEMMs run on v_mfma_f32_32x32x64_f8f6f4: weights are the A operand (rows n), activations the B operand, so a
// lane's 16 accumulators of a 32 x 32 tile belong to ONE token row and the block's combined scale is one value a lane.
#include "abi_internal.h"
#include "common.cuh"

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
constexpr int kTile = 128;  // rows of a tile (token positions) and weight rows a workgroup
struct PfLayout {
  size_t cnt, off, ntiles, tile_e, tile_m0, perm, pickpos, rpos, re, rk, xq, xs, h, hq, hs, hsh, hshq, hshs, d, total;
  int P, max_tiles;
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
  o.perm = take(P * 4), o.pickpos = take(P * 4), o.rpos = take(P * 4), o.re = take(P * 4), o.rk = take(P * 4);
  o.xq = take((size_t)T * H), o.xs = take((size_t)T * (H / 128) * 4);
  o.h = take(P * I * 2), o.hq = take(P * I), o.hs = take(P * (I / 128) * 4);
  o.hsh = take((size_t)T * I * 2), o.hshq = take((size_t)T * I), o.hshs = take((size_t)T * (I / 128) * 4);
  o.d = take(P * H * 4);
  o.total = at;
  return o;
}

// ---- bucketing -----------------------------------------------------------------------------------------------------------
// picks of expert e (one workgroup an expert)
__global__ void __launch_bounds__(256) k_pf_count(const int* __restrict__ idx, int P, int* __restrict__ cnt) {
  const int e = blockIdx.x;
  int c = 0;
  for (int p = threadIdx.x; p < P; p += blockDim.x) c += idx[p] == e;
  __shared__ int part[4];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) cnt[e] = part[0] + part[1] + part[2] + part[3];
}
// bucket offsets and the list of 128-row tiles in expert order (one thread: E <= 512)
__global__ void k_pf_scan(const int* __restrict__ cnt, int E, int* __restrict__ off, int* __restrict__ ntiles, int* __restrict__ tile_e,
                          int* __restrict__ tile_m0) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int at = 0, nt = 0;
  for (int e = 0; e < E; ++e) {
    off[e] = at;
    for (int m0 = 0; m0 < cnt[e]; m0 += kTile) tile_e[nt] = e, tile_m0[nt] = m0, ++nt;
    at += cnt[e];
  }
  off[E] = at;
  *ntiles = nt;
}
// the picks of expert e in pick order (row-major over [T][topk]) to positions off[e] ...: perm[position] = row,
// pickpos[pick] = position
__global__ void __launch_bounds__(256) k_pf_scatter(const int* __restrict__ idx, int P, int topk, const int* __restrict__ off,
                                                    int* __restrict__ perm, int* __restrict__ pickpos) {
  const int e = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __shared__ int wcnt[4];
  int base = off[e];
  for (int p0 = 0; p0 < P; p0 += 256) {
    const int p = p0 + threadIdx.x;
    const bool hit = p < P && idx[p] == e;
    const uint64_t m = __ballot(hit);
    if (lane == 0) wcnt[wave] = __popcll(m);
    __syncthreads();
    int before = __popcll(m & ((1ull << lane) - 1));
    for (int w = 0; w < wave; ++w) before += wcnt[w];
    if (hit) perm[base + before] = p / topk, pickpos[p] = base + before;
    base += wcnt[0] + wcnt[1] + wcnt[2] + wcnt[3];
    __syncthreads();
  }
}
// per row: its picks in expert-id order (ids are distinct in a row): expert, bucket position, combine factor s2 * w
__global__ void __launch_bounds__(256) k_pf_rowsort(const int* __restrict__ idx, const float* __restrict__ w, const int* __restrict__ pickpos,
                                                    const dsgx_mat_desc* __restrict__ desc, int T, int topk, int* __restrict__ rpos,
                                                    int* __restrict__ re, float* __restrict__ rk) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  for (int k = 0; k < topk; ++k) {
    const int e = idx[t * topk + k];
    int r = 0;
    for (int j = 0; j < topk; ++j) r += idx[t * topk + j] < e;
    re[t * topk + r] = e;
    rpos[t * topk + r] = pickpos[t * topk + k];
    rk[t * topk + r] = __fmul_rn(desc[(size_t)e * 3 + 2].s2, w[t * topk + k]);
  }
}

// ---- the grouped GEMM ---------------------------------------------------------------------------------------------------
// A workgroup (4 waves, 2 x 2) computes 128 weight rows x 128 positions of one tile; UP: the weight rows are 64 gate and
// 64 up channels (a wave: 32 + 32 of the same channels, so g and u of a channel meet in one lane). K in blocks of 128:
// the block's A and B panels go through LDS (rows padded to 144 bytes: the 32-byte fragment reads of 32 consecutive
// rows then fall on distinct banks), double buffered, the next block's global loads in flight during the MFMAs.
constexpr int kLdsRow = 144;
constexpr int kPanel = kTile * kLdsRow;  // bytes of one 128-row panel

struct GemmArgs {
  const uint8_t* aq;   // activations, e4m3 [rows][K]
  const float* as;     // their scales [rows][K / 128]
  const int* gather;   // position -> activation row (null: the position itself)
  const int* tile_e;   // (null: one pseudo-expert -1 holding rows [0, nrows): the shared expert)
  const int* tile_m0;
  const int* ntiles;
  const int* off;
  int nrows;           // shared expert: T
  dsgx_layer_w L;
  uint16_t* h;         // UP: h bf16 [position][I]
  float* d;            // DOWN: f32 [position][H]
};

template <bool UP>
__global__ void __launch_bounds__(256, 2) k_pf_gemm(GemmArgs g) {
  extern __shared__ uint8_t smem[];
  const int K = UP ? g.L.H : g.L.I, KB = K / 128;
  const int NS = UP ? g.L.I / 64 : g.L.H / kTile;  // workgroups along the weight rows
  const int tile = blockIdx.x / NS, ns = blockIdx.x % NS;
  int e = -1, m0 = tile * kTile, mend = g.nrows;
  if (g.tile_e) {
    if (tile >= *g.ntiles) return;
    e = g.tile_e[tile];
    const int o = g.off[e];
    m0 = o + g.tile_m0[tile], mend = g.off[e + 1];
  } else if (m0 >= mend) {
    return;
  }
  // the tile's matrices
  const uint8_t *wa, *wb;   // UP: gate, up; DOWN: down (wb unused)
  const float *sa, *sb;
  float s2a = 1.f, s2b = 1.f;
  const size_t NK = (size_t)g.L.H * g.L.I;
  if (e < 0) {
    if (UP) wa = g.L.sh.g, sa = g.L.sh.gs, wb = g.L.sh.u, sb = g.L.sh.us;
    else wa = wb = g.L.sh.d, sa = sb = g.L.sh.ds;
  } else {
    const dsgx_mat_desc* d = g.L.desc + (size_t)e * 3;
    if (UP) {
      wa = g.L.pool + d[0].off, wb = g.L.pool + d[1].off, s2a = d[0].s2, s2b = d[1].s2;
    } else {
      wa = wb = g.L.pool + d[2].off;
    }
    sa = reinterpret_cast<const float*>(wa + (NK + 255) / 256 * 256);
    sb = reinterpret_cast<const float*>(wb + (NK + 255) / 256 * 256);
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wn = wave >> 1, wm = wave & 1;
  const int n0 = UP ? ns * 64 : ns * kTile;  // first channel (UP) / first weight row (DOWN) of the workgroup

  // staging: thread t brings chunk t % 8 (16 bytes) of panel rows t / 8 + 32 i, i < 4, of A and of B
  const int chunk = tid & 7, srow = tid >> 3;
  const uint8_t* pa[4];
  const uint8_t* pb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int a = srow + 32 * i;  // panel row of A: wave-major (wn', nt, row)
    if (UP) {
      const int c = n0 + 32 * (a >> 6) + (a & 31);
      pa[i] = ((a >> 5) & 1 ? wb : wa) + (size_t)c * K + chunk * 16;
    } else {
      pa[i] = wa + (size_t)(n0 + a) * K + chunk * 16;
    }
    int pos = m0 + srow + 32 * i;
    if (pos >= mend) pos = mend - 1;  // a ragged tile re-reads its last row (never stored)
    const int row = g.gather ? g.gather[pos] : pos;
    pb[i] = g.aq + (size_t)row * K + chunk * 16;
  }
  // the lane's two token columns (one a 32-column tile) and their activation rows, for the block scales
  int mpos[2];
  const float* xs[2];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
    int pos = m0 + 64 * wm + 32 * mt + (lane & 31);
    mpos[mt] = pos;
    if (pos >= mend) pos = mend - 1;
    xs[mt] = g.as + (size_t)(g.gather ? g.gather[pos] : pos) * KB;
  }
  // the wave's weight scale rows (its 64 weight rows lie in one 128-row scale block)
  const float* swa = sa + (size_t)((UP ? n0 + 32 * wn : n0 + 64 * wn) / 128) * KB;
  const float* swb = UP ? sb + (size_t)((n0 + 32 * wn) / 128) * KB : swa;

  v16f_t acc[2][2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) acc[nt][mt] = v16f_t{};

  uint4 ra[4], rb[4];
  auto fetch = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 4; ++i) ra[i] = *reinterpret_cast<const uint4*>(pa[i] + (size_t)kb * 128);
#pragma unroll
    for (int i = 0; i < 4; ++i) rb[i] = *reinterpret_cast<const uint4*>(pb[i] + (size_t)kb * 128);
  };
  auto stash = [&](int buf) {
    uint8_t* A = smem + (size_t)buf * 2 * kPanel;
    uint8_t* B = A + kPanel;
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(A + (srow + 32 * i) * kLdsRow + chunk * 16) = ra[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(B + (srow + 32 * i) * kLdsRow + chunk * 16) = rb[i];
  };
  fetch(0);
  stash(0);
  __syncthreads();
  for (int kb = 0; kb < KB; ++kb) {
    if (kb + 1 < KB) fetch(kb + 1);
    const float x0 = xs[0][kb], x1 = xs[1][kb], wsa = swa[kb], wsb = swb[kb];
    const uint8_t* A = smem + (size_t)(kb & 1) * 2 * kPanel + (size_t)(wn * 64 + (lane & 31)) * kLdsRow + (lane >> 5) * 32;
    const uint8_t* B = smem + (size_t)(kb & 1) * 2 * kPanel + kPanel + (size_t)(wm * 64 + (lane & 31)) * kLdsRow + (lane >> 5) * 32;
    v16f_t p[2][2];
#pragma unroll
    for (int kc = 0; kc < 2; ++kc) {
      v8i_t fa[2], fb[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        fa[t] = *reinterpret_cast<const v8i_t*>(A + t * 32 * kLdsRow + kc * 64);
        fb[t] = *reinterpret_cast<const v8i_t*>(B + t * 32 * kLdsRow + kc * 64);
      }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) p[nt][mt] = mfma_fp8(fa[nt], fb[mt], kc == 0 ? v16f_t{} : p[nt][mt]);
    }
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const float sc = __fmul_rn(mt ? x1 : x0, nt ? wsb : wsa);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[nt][mt][r] = fmaf(sc, p[nt][mt][r], acc[nt][mt][r]);
      }
    if (kb + 1 < KB) stash((kb + 1) & 1);
    __syncthreads();
  }

  // epilogue: register r of lane l is weight row 8 (r / 4) + 4 (l / 32) + r % 4 of the 32-row tile, column l % 32
  if (UP) {
    const int I = g.L.I;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      if (mpos[mt] >= mend) continue;
      uint16_t* hr = g.h + (size_t)mpos[mt] * I + n0 + 32 * wn + 4 * (lane >> 5);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint32_t hb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
          hb[j] = swiglu_bits(bf16_round(__fmul_rn(acc[0][mt][4 * q + j], s2a)), bf16_round(__fmul_rn(acc[1][mt][4 * q + j], s2b)));
        *reinterpret_cast<uint2*>(hr + 8 * q) = make_uint2(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16));
      }
    }
  } else {
    const int H = g.L.H;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      if (mpos[mt] >= mend) continue;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        float* dr = g.d + (size_t)mpos[mt] * H + n0 + 64 * wn + 32 * nt + 4 * (lane >> 5);
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<float4*>(dr + 8 * q) =
              make_float4(acc[nt][mt][4 * q], acc[nt][mt][4 * q + 1], acc[nt][mt][4 * q + 2], acc[nt][mt][4 * q + 3]);
      }
    }
  }
}

// yr[t][n] over the row's picks in expert-id order: acc = fma(s2 * w, d, acc); four columns a thread
__global__ void __launch_bounds__(256) k_pf_combine(const float* __restrict__ d, const int* __restrict__ rpos, const float* __restrict__ rk,
                                                    int T, int H, int topk, float* __restrict__ yr) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per = H / 4;
  if (i >= (size_t)T * per) return;
  const int t = (int)(i / per), n = (int)(i % per) * 4;
  float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int r = 0; r < topk; ++r) {
    const float k = rk[t * topk + r];
    const float4 v = *reinterpret_cast<const float4*>(d + (size_t)rpos[t * topk + r] * H + n);
    a.x = fmaf(k, v.x, a.x), a.y = fmaf(k, v.y, a.y), a.z = fmaf(k, v.z, a.z), a.w = fmaf(k, v.w, a.w);
  }
  *reinterpret_cast<float4*>(yr + (size_t)t * H + n) = a;
}

bool layer_has_fp8_shared(const dsgx_layer_w* L) { return L->sh.g && L->sh.u && L->sh.d && L->sh.gs && L->sh.us && L->sh.ds; }

}  // namespace
}  // namespace dsgx

using namespace dsgx;

extern "C" {

// raw[lane][r]: the accumulator registers of one v_mfma_f32_32x32x64_f8f6f4 of A [32][64] and B [32][64] (e4m3 codes,
// k contiguous), so that a test can pin the operand and result layouts the prefill kernels assume.
int dsgx_probe_mfma_fp8(const void* A, const void* B, float* raw, void* stream) {
  if (!A || !B || !raw) return fail(DSGX_EINVAL, "probe_mfma_fp8: null argument");
  hipLaunchKernelGGL(k_probe_mfma_fp8, dim3(1), dim3(64), 0, (hipStream_t)stream, (const uint8_t*)A, (const uint8_t*)B, raw);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}

void dsgx_prefill_cfg_default(dsgx_prefill_cfg* c) {
  if (!c) return;
  c->shared = 1;
  c->phases = 31;
  c->act_fp8 = 1;
}

static int prefill_check(const dsgx_layer_w* L, int T, const char* who) {
  if (!L) return fail(DSGX_EINVAL, "%s: null layer", who);
  if (L->fmt != DSGX_FMT_FP8_B128) return fail(DSGX_EUNSUPPORTED, "%s: only FP8_B128 layers are built (format %u)", who, L->fmt);
  if (T < 1 || T > DSGX_MAX_CHUNK) return fail(DSGX_EINVAL, "%s: T %d (1..%d)", who, T, DSGX_MAX_CHUNK);
  if (L->H < 128 || L->H % 128 || L->I < 128 || L->I % 128) return fail(DSGX_EINVAL, "%s: H %d, I %d (multiples of 128)", who, L->H, L->I);
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
  if (!cfg.act_fp8) return fail(DSGX_EUNSUPPORTED, "moe_prefill: bf16 activations (act_fp8 = 0) are not built yet");
  const bool shared = cfg.shared && layer_has_fp8_shared(L);
  if (cfg.shared && L->sh.bgu) return fail(DSGX_EUNSUPPORTED, "moe_prefill: BF16 shared expert is not built yet");
  if (shared && !ys) return fail(DSGX_EINVAL, "moe_prefill: the layer has a fused shared expert and ys is null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const PfLayout o = pf_layout(L, T);
  uint8_t* W = static_cast<uint8_t*>(ws);
  auto I32 = [&](size_t off) { return reinterpret_cast<int*>(W + off); };
  auto F32 = [&](size_t off) { return reinterpret_cast<float*>(W + off); };
  const int H = L->H, I = L->I, E = L->E, topk = L->topk, P = o.P;
  const size_t lds = 2 * 2 * (size_t)kPanel;
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(k_pf_gemm<true>), lds)) return rc;
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(k_pf_gemm<false>), lds)) return rc;

  if (cfg.phases & 1) {
    hipLaunchKernelGGL(k_pf_count, dim3(E), dim3(256), 0, st, idx, P, I32(o.cnt));
    hipLaunchKernelGGL(k_pf_scan, dim3(1), dim3(64), 0, st, I32(o.cnt), E, I32(o.off), I32(o.ntiles), I32(o.tile_e), I32(o.tile_m0));
    hipLaunchKernelGGL(k_pf_scatter, dim3(E), dim3(256), 0, st, idx, P, topk, I32(o.off), I32(o.perm), I32(o.pickpos));
    hipLaunchKernelGGL(k_pf_rowsort, dim3((T + 255) / 256), dim3(256), 0, st, idx, w, I32(o.pickpos), L->desc, T, topk, I32(o.rpos),
                       I32(o.re), F32(o.rk));
    DSGX_HIP(hipGetLastError());
  }
  GemmArgs g{};
  g.L = *L;
  if (cfg.phases & (2 | 16)) {
    if (int rc = dsgx_act_quant(x, T, H, W + o.xq, F32(o.xs), stream)) return rc;
  }
  if (cfg.phases & 2) {
    g.aq = W + o.xq, g.as = F32(o.xs), g.gather = I32(o.perm);
    g.tile_e = I32(o.tile_e), g.tile_m0 = I32(o.tile_m0), g.ntiles = I32(o.ntiles), g.off = I32(o.off), g.nrows = P;
    g.h = reinterpret_cast<uint16_t*>(W + o.h), g.d = nullptr;
    hipLaunchKernelGGL(k_pf_gemm<true>, dim3((unsigned)o.max_tiles * (I / 64)), dim3(256), lds, st, g);
    DSGX_HIP(hipGetLastError());
  }
  if (cfg.phases & 4) {
    if (int rc = dsgx_act_quant(reinterpret_cast<const uint16_t*>(W + o.h), P, I, W + o.hq, F32(o.hs), stream)) return rc;
    g.aq = W + o.hq, g.as = F32(o.hs), g.gather = nullptr;
    g.tile_e = I32(o.tile_e), g.tile_m0 = I32(o.tile_m0), g.ntiles = I32(o.ntiles), g.off = I32(o.off), g.nrows = P;
    g.h = nullptr, g.d = F32(o.d);
    hipLaunchKernelGGL(k_pf_gemm<false>, dim3((unsigned)o.max_tiles * (H / kTile)), dim3(256), lds, st, g);
    DSGX_HIP(hipGetLastError());
  }
  if (cfg.phases & 8) {
    const size_t n = (size_t)T * (H / 4);
    hipLaunchKernelGGL(k_pf_combine, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, F32(o.d), I32(o.rpos), F32(o.rk), T, H, topk, yr);
    DSGX_HIP(hipGetLastError());
  }
  if ((cfg.phases & 16) && shared) {
    const int tiles = (T + kTile - 1) / kTile;
    g.aq = W + o.xq, g.as = F32(o.xs), g.gather = nullptr;
    g.tile_e = g.tile_m0 = g.ntiles = g.off = nullptr, g.nrows = T;
    g.h = reinterpret_cast<uint16_t*>(W + o.hsh), g.d = nullptr;
    hipLaunchKernelGGL(k_pf_gemm<true>, dim3((unsigned)tiles * (I / 64)), dim3(256), lds, st, g);
    if (int rc = dsgx_act_quant(reinterpret_cast<const uint16_t*>(W + o.hsh), T, I, W + o.hshq, F32(o.hshs), stream)) return rc;
    g.aq = W + o.hshq, g.as = F32(o.hshs), g.h = nullptr, g.d = ys;
    hipLaunchKernelGGL(k_pf_gemm<false>, dim3((unsigned)tiles * (H / kTile)), dim3(256), lds, st, g);
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

}  // extern "C"
