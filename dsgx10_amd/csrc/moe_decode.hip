// The C ABI of the decode expert step (dsgx_moe_decode = gx::moe_decode of the reference,
// altar1-4xgx10-switchless/engine/experts/decode.cu:708-730): argument checks and the dispatch on the layer's format.
// The kernels are in moe_decode_impl.cuh, instantiated per format in moe_decode_{fp8,int4,bf16}.hip.
#include <mutex>

#include "moe_decode_impl.cuh"

using namespace dsgx;

#ifdef DSGX_TRACE
static unsigned long long* g_trace_buf = nullptr;  // device memory, [workgroups][16]
extern "C" __attribute__((visibility("default"))) void dsgx_trace_set(void* dev) { g_trace_buf = static_cast<unsigned long long*>(dev); }
extern "C" unsigned long long* dsgx_trace_buf() { return g_trace_buf; }
#endif

// The workspace of dsgx_moe_decode_noalloc: a device array of the library itself, sized for the largest layer that entry
// point takes (h of 129 slots x 16 rows x DSGX_NOALLOC_MAX_I, the barrier's words, the slot-partitioned down phase's
// table and its f32 [129][8][DSGX_NOALLOC_MAX_H] results: 34.0 MB on every GPU the library runs on, zero when the
// module loads, which is the barrier's initial state). In host code the array's name is not a device address: the
// address is asked for once a device (static_ws) and only that pointer is used.
static constexpr size_t kStaticWsBytes = (size_t)(DSGX_MAX_UNION + 1) * DSGX_MAX_ROWS * DSGX_NOALLOC_MAX_I * 2 + dsgx::kBarBytes +
                                         (size_t)(8 + (DSGX_MAX_UNION + 1) * 8) * 4 + 192 +
                                         (size_t)(DSGX_MAX_UNION + 1) * 8 * DSGX_NOALLOC_MAX_H * 4 + (size_t)DSGX_MAX_ROWS * DSGX_NOALLOC_MAX_H * 2;
static __device__ __align__(256) uint8_t scratch[kStaticWsBytes];
// (never launched: keeps the array referenced from device code of this file)
__global__ void k_scratch_probe(uint8_t* out) {
  if (out) *out = scratch[0];
}
static int static_ws(void** out) {
  constexpr int kMaxDev = 64;
  static void* ptr[kMaxDev] = {};
  static std::mutex mu;
  int dev = 0;
  DSGX_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDev) return fail(DSGX_EINVAL, "moe_decode_noalloc: device %d", dev);
  std::lock_guard<std::mutex> lk(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    DSGX_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));  // (the current device's copy of the array)
    if (!p) return fail(DSGX_EHIP, "moe_decode_noalloc: no address for the built-in workspace");
    ptr[dev] = p;
  }
  *out = ptr[dev];
  return DSGX_OK;
}

extern "C" {

void dsgx_decode_cfg_default(dsgx_decode_cfg* c) {
  if (!c) return;
  c->up = -1;  // the faster variant for the layer's format and the row count (decode_variant)
  c->down = 0;
  c->parts = 3;
  c->ysum = 0;
  c->logits = c->bias = nullptr;
  c->route_scale = 1.f;
  c->score_fn = 0;
  c->post = nullptr;
}

// dsgx_decode_cfg::up = -1: INT4 layers run on the MFMA kernels at every row count; FP8 layers on the vector-unit
// kernels at one row (the stream is then bound by memory alone) and on the MFMA kernels from two rows on; BF16 layers
// have the vector-unit kernels only.
static int decode_variant(uint32_t fmt, int M, int H, int I) {
  if (fmt == DSGX_FMT_INT4_G32) return 1;
  if (fmt == DSGX_FMT_FP8_B128) return M >= 2 || H % 1024 || I % 1024 ? 1 : 0;  // (shapes only the MFMA kernels' steps divide)
  return 0;
}

}  // extern "C"

// The workspace: h [DSGX_MAX_UNION + 1 slots][DSGX_MAX_ROWS][I] | the barrier's words (kBarBytes) | the slot-partitioned down
// phase's slot table (kFacBytes) and its f32 results [slot][8 rows][H] | a reserved row buffer [16][H] bf16. I and H here are the LAYOUT's: the layer's own for a
// caller's workspace; the built-in workspace is laid out for its largest shapes whatever the layer, so that every layer run
// on it finds the barrier's words in one place (at an offset that moved with the layer, one layer's h or partial sums would
// lie where another's counters are expected to be zero).
struct WsLayout {
  int I, H;
  static constexpr size_t kFacBytes = (size_t)(8 + (DSGX_MAX_UNION + 1) * 8) * 4 + 192;  // (a multiple of 256)
  constexpr size_t h_bytes() const { return (size_t)(DSGX_MAX_UNION + 1) * DSGX_MAX_ROWS * I * 2; }
  constexpr size_t bar_off() const { return h_bytes(); }
  constexpr size_t fac_off() const { return bar_off() + kBarBytes; }
  constexpr size_t dpart_off() const { return fac_off() + kFacBytes; }
  constexpr size_t xdeq_off() const { return dpart_off() + (size_t)(DSGX_MAX_UNION + 1) * 8 * H * 4; }  // (reserved)
  constexpr size_t bytes() const { return xdeq_off() + (size_t)DSGX_MAX_ROWS * H * 2; }
  // dsgx_dsk_moe_stacked's workspace: the same, then the shared expert's output rows f32 [DSGX_MAX_ROWS][H]
  constexpr size_t dsk_ys_off() const { return (bytes() + 255) / 256 * 256; }
  constexpr size_t dsk_bytes() const { return dsk_ys_off() + (size_t)DSGX_MAX_ROWS * H * 4; }
};
static constexpr WsLayout kStaticLayout{DSGX_NOALLOC_MAX_I, DSGX_NOALLOC_MAX_H};
static_assert(kStaticLayout.bytes() == kStaticWsBytes, "the built-in workspace's size");
// DeepSeek's entry point: the rows as e4m3 codes with a ue8m0 scale per 32 values (x then only names the workspace's row buffer)
struct DskIn {
  int on = 0;
  float limit = 0.f;
  const uint8_t* xq = nullptr;
  const uint8_t* xs = nullptr;
  const dsgx_dsk_weights* stacked = nullptr;  // experts stacked by id in their own tensors (no pool, no descriptors)
  int* idx_out = nullptr;                     // fused routing: the selection, for the caller
  float* wts_out = nullptr;
};
static int moe_decode_at(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, void* ws, const WsLayout& lay,
                         float* yr, float* ys, void* stream, const dsgx_decode_cfg* cfg, DskIn dsk = DskIn{});

extern "C" {
size_t dsgx_decode_ws_bytes(const dsgx_layer_w* L) {
  if (!L || L->I <= 0 || L->H <= 0) return 0;
  return WsLayout{L->I, L->H}.bytes();
}
size_t dsgx_decode_ws_flag_offset(const dsgx_layer_w* L) {
  if (!L || L->I <= 0) return 0;
  return WsLayout{L->I, L->H}.bar_off() + (size_t)(2 * kBarGroups + 1) * kBarLine * 4;
}

int dsgx_moe_decode(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, void* ws, float* yr, float* ys,
                    void* stream, const dsgx_decode_cfg* cfg) {
  if (!L) return fail(DSGX_EINVAL, "moe_decode: null layer, x or workspace");
  return moe_decode_at(L, x, idx, w, M, ws, WsLayout{L->I, L->H}, yr, ys, stream, cfg);
}
}  // extern "C"

// up = DSGX_UP_PREFILL_ORDER (the reference's kUpPrefillOrder, experts.h:111-113, 138): the rows go through the prefill
// kernels as a chunk of M rows (bf16 activations), so yr and ys are moe_prefill's bit for bit - for callers that verify
// drafted tokens against a prefill of the same rows. The chunk's intermediates take the h part of the workspace (in
// dsgx_prefill_view's layout, not the decode step's slots); the barrier's words behind it are left alone.
namespace {
__global__ void __launch_bounds__(256) k_ysum(float* __restrict__ yr, const float* __restrict__ ys, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) yr[i] = __fadd_rn(yr[i], ys[i]);
}
}  // namespace
static int decode_by_prefill(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, void* ws, const WsLayout& lay,
                             float* yr, float* ys, void* stream, const dsgx_decode_cfg& c, bool dsk) {
  if (dsk) return fail(DSGX_EUNSUPPORTED, "dsk_moe: no prefill-order variant");
  if (c.parts != 3) return fail(DSGX_EUNSUPPORTED, "moe_decode: the prefill-order variant runs both phases (parts 3), not %d", c.parts);
  if (!yr) return fail(DSGX_EINVAL, "moe_decode: null yr");
  if (L->E < 1 || L->E > DSGX_MAX_EXPERTS || L->topk < 1 || L->topk > DSGX_MAX_TOPK || L->topk > L->E)
    return fail(DSGX_EINVAL, "moe_decode: E %d, top-k %d", L->E, L->topk);
  const size_t pick_bytes = (size_t)DSGX_MAX_ROWS * DSGX_MAX_TOPK * 4, need = dsgx_prefill_ws_bytes(L, M);
  if (need == 0) return DSGX_EINVAL;  // (dsgx_prefill_ws_bytes has said why)
  const size_t tail = (need + 255) / 256 * 256;
  if (tail + 2 * pick_bytes > lay.bar_off())
    return fail(DSGX_EUNSUPPORTED, "moe_decode: the prefill-order variant needs %zu bytes of the workspace's %zu in front of the barrier's words", tail + 2 * pick_bytes,
                lay.bar_off());
  uint8_t* W = static_cast<uint8_t*>(ws);
  if (c.logits) {  // the routing's picks behind the chunk's intermediates
    int* ri = reinterpret_cast<int*>(W + tail);
    float* rw = reinterpret_cast<float*>(W + tail + pick_bytes);
    if (int rc = dsgx_route(c.logits, c.bias, M, L->E, L->topk, c.route_scale, c.score_fn, ri, rw, stream)) return rc;
    idx = ri, w = rw;
  }
  dsgx_prefill_cfg p;
  dsgx_prefill_cfg_default(&p);
  p.act_fp8 = c.up == DSGX_UP_PREFILL_ORDER_ACT_FP8 ? 1 : 0;
  if (p.act_fp8 && L->fmt != DSGX_FMT_FP8_B128)
    return fail(DSGX_EUNSUPPORTED, "moe_decode: up = %d pairs with a prefill on FP8 activations, which FP8_B128 layers have (format %u)", c.up, L->fmt);
  if (int rc = dsgx_moe_prefill(L, x, idx, w, M, ws, yr, ys, stream, &p)) return rc;
  if (c.ysum) {
    if (!ys) return fail(DSGX_EINVAL, "moe_decode: ysum without ys");
    const int n = M * L->H;
    hipLaunchKernelGGL(k_ysum, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), yr, ys, n);
    DSGX_HIP(hipGetLastError());
  }
  return DSGX_OK;
}

static int moe_decode_at(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, void* ws, const WsLayout& lay,
                         float* yr, float* ys, void* stream, const dsgx_decode_cfg* cfg, DskIn dsk) {
  dsgx_decode_cfg c;
  if (cfg) c = *cfg;
  else dsgx_decode_cfg_default(&c);
  // the reference's checks (decode.cu:710-729): it dies, this returns an error
  if (!L || !x || !ws) return fail(DSGX_EINVAL, "moe_decode: null layer, x or workspace");
  if (M < 1 || M > DSGX_MAX_ROWS) return fail(DSGX_EINVAL, "moe_decode: M=%d", M);
  if (!c.logits && (!idx || !w)) return fail(DSGX_EINVAL, "moe_decode: idx and w, or logits");
  if (c.post) return fail(DSGX_EUNSUPPORTED, "moe_decode: posted outputs need the reference's ring; one GPU has none");
  if (c.parts < 1 || c.parts > 3) return fail(DSGX_EINVAL, "moe_decode: parts %d", c.parts);
  if (c.up == DSGX_UP_PREFILL_ORDER || c.up == DSGX_UP_PREFILL_ORDER_ACT_FP8) return decode_by_prefill(L, x, idx, w, M, ws, lay, yr, ys, stream, c, dsk.on != 0);
  if (c.up < -1 || c.up > 1 || c.down < 0 || c.down > 1) return fail(DSGX_EINVAL, "moe_decode: up variant %d / down variant %d", c.up, c.down);
  if (c.up == -1) c.up = c.down == 1 ? 0 : decode_variant(L->fmt, M, L->H, L->I);  // (the two-launch form is the vector-unit kernels')
  if (c.up == 1 && L->fmt != DSGX_FMT_FP8_B128 && L->fmt != DSGX_FMT_INT4_G32 && L->fmt != DSGX_FMT_MXFP4_G32)
    return fail(DSGX_EUNSUPPORTED, "moe_decode: variant 1 (MFMA) is built for FP8_B128 and INT4_G32 layers");
  if (c.down == 1 && c.parts == 3) c.parts = 3 | 4;  // variant 1: the two phases as two launches
  if (L->fmt == DSGX_FMT_REF_NVFP4 || L->fmt == DSGX_FMT_REF_INT4 || L->fmt == DSGX_FMT_REF_BF16)
    return fail(DSGX_EFORMAT, "moe_decode: layer expert format %u names a GB10 block tiling; repack to FP8_B128 (16), INT4_G32 (18) or BF16 (19)", L->fmt);
  if (L->fmt == DSGX_FMT_MXFP4_G32 && !dsk.on)
    return fail(DSGX_EFORMAT, "moe_decode: MXFP4 experts follow DeepSeek's expert arithmetic: dsgx_dsk_moe");
  if (dsk.on && L->fmt != DSGX_FMT_MXFP4_G32) return fail(DSGX_EFORMAT, "dsk_moe: layer expert format %u is not MXFP4_G32 (20)", L->fmt);
  if (dsk.on) c.up = 1;  // (the MFMA kernels are the ones built for it)
  if (L->fmt != DSGX_FMT_FP8_B128 && L->fmt != DSGX_FMT_INT4_G32 && L->fmt != DSGX_FMT_BF16 && L->fmt != DSGX_FMT_MXFP4_G32)
    return fail(DSGX_EFORMAT, "moe_decode: layer expert format %u is not FP8_B128 (16), INT4_G32 (18) or BF16 (19)", L->fmt);
  if (!dsk.stacked && (!L->pool || !L->desc)) return fail(DSGX_EINVAL, "moe_decode: null pool or descriptors");
  const int H = L->H, I = L->I;
  if (L->E < 1 || L->E > DSGX_MAX_EXPERTS || L->topk < 1 || L->topk > DSGX_MAX_TOPK || L->topk > L->E)
    return fail(DSGX_EINVAL, "moe_decode: E %d, top-k %d", L->E, L->topk);
  // the vector-unit kernels walk whole 1 KiB segments of a row (2048 INT4, 1024 FP8, 512 BF16 values); the MFMA kernels
  // steps of 256 k, so they also take the narrow per-rank shapes (the reference's intermediate 512, experts.h:18-22)
  const int kmul = c.up == 1 ? 256 : L->fmt == DSGX_FMT_INT4_G32 ? 2048 : L->fmt == DSGX_FMT_FP8_B128 ? 1024 : 512;
  if (H < kmul || H % kmul || I < kmul || I % kmul || I % 128 || H % 128)
    return fail(DSGX_EINVAL, "moe_decode: hidden %d, intermediate %d (multiples of %d for this format and variant)", H, I, kmul);
  const bool fp8sh = L->sh.g != nullptr, b16sh = L->sh.bgu != nullptr;
  if (fp8sh && b16sh) return fail(DSGX_EINVAL, "moe_decode: an FP8 and a BF16 shared expert");
  if (fp8sh && (!L->sh.u || !L->sh.d || !L->sh.gs || !L->sh.us || !L->sh.ds)) return fail(DSGX_EINVAL, "moe_decode: the FP8 shared expert needs g, u, d and their scales");
  if (fp8sh && c.up != 1 && (H % 1024 || I % 1024)) return fail(DSGX_EINVAL, "moe_decode: the FP8 shared expert needs hidden and intermediate multiples of 1024");
  if (b16sh && !L->sh.bd) return fail(DSGX_EINVAL, "moe_decode: the BF16 shared expert needs its down");
  if ((c.parts & 2) && !yr) return fail(DSGX_EINVAL, "moe_decode: null yr");
  if ((fp8sh || b16sh || c.ysum) && (c.parts & 2) && !ys) return fail(DSGX_EINVAL, "moe_decode: ys (the shared expert's output) is needed");
  if (((uintptr_t)x | (uintptr_t)ws | (uintptr_t)L->pool) & 15) return fail(DSGX_EINVAL, "moe_decode: x, ws and pool must be 16-byte aligned");

  if (M > 8) {
    // 9-16 rows (the reference's limit, experts.h:104): two passes of the kernels built for up to eight rows, rows 0-7
    // then the rest; every row's result is what it is alone or in any batch, so the split is invisible in the output.
    // The second pass reads the weights of its experts again; the workspace is reused in stream order.
    const int M1 = 8, topk = L->topk, E = L->E;
    dsgx_decode_cfg c1 = c, c2 = c;
    c1.parts = c2.parts = c.parts & 3;
    if (c.logits) c2.logits = c.logits + (size_t)M1 * E;
    if (int rc = moe_decode_at(L, x, idx, w, M1, ws, lay, yr, ys, stream, &c1, dsk)) return rc;
    DskIn dsk2 = dsk;
    if (dsk.xq) dsk2.xq = dsk.xq + (size_t)M1 * H, dsk2.xs = dsk.xs + (size_t)M1 * (H / 32);
    if (dsk.idx_out) dsk2.idx_out = dsk.idx_out + (size_t)M1 * topk, dsk2.wts_out = dsk.wts_out + (size_t)M1 * topk;
    return moe_decode_at(L, x + (size_t)M1 * H, idx ? idx + (size_t)M1 * topk : nullptr, w ? w + (size_t)M1 * topk : nullptr, M - M1, ws, lay,
                         yr ? yr + (size_t)M1 * H : nullptr, ys ? ys + (size_t)M1 * H : nullptr, stream, &c2, dsk2);
  }
  DecodeArgs a{};
  a.x = x, a.M = M, a.idx = idx, a.w = w, a.logits = c.logits, a.bias = c.bias, a.route_scale = c.route_scale, a.score_fn = c.score_fn;
  a.L = *L, a.h = static_cast<uint16_t*>(ws), a.yr = yr, a.ys = ys, a.ysum = c.ysum;
  uint8_t* wsb = static_cast<uint8_t*>(ws);
  a.bar = reinterpret_cast<int*>(wsb + lay.bar_off());
  a.fac = reinterpret_cast<float*>(wsb + lay.fac_off());
  a.dpart = reinterpret_cast<float*>(wsb + lay.dpart_off());
  a.dsk = dsk.on, a.dsk_limit = dsk.limit, a.dsk_xq = dsk.xq, a.dsk_xs = dsk.xs;
  a.idx_out = c.logits ? dsk.idx_out : nullptr, a.wts_out = c.logits ? dsk.wts_out : nullptr;
  if (const dsgx_dsk_weights* W = dsk.stacked) {
    const size_t gu = (size_t)I * H, dn = (size_t)H * I;
    a.stk_w[0] = W->w1, a.stk_w[1] = W->w3, a.stk_w[2] = W->w2;
    a.stk_s[0] = W->s1, a.stk_s[1] = W->s3, a.stk_s[2] = W->s2;
    a.stk_wb[0] = a.stk_wb[1] = gu / 2, a.stk_wb[2] = dn / 2;
    a.stk_sb[0] = a.stk_sb[1] = gu / 32, a.stk_sb[2] = dn / 32;
  }
  a.spin_limit = 1 << 22;
#ifdef DSGX_TRACE
  a.trace = g_trace_buf;
#endif
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t f = L->fmt;
  if (f == DSGX_FMT_FP8_B128) {
    if (b16sh) return fail(DSGX_EUNSUPPORTED, "moe_decode: FP8 experts with a BF16 shared expert are not built");
    if (c.up == 1) return launch_decode_fp8_mfma(a, c.parts & 3, fp8sh, st);
    return launch_decode_fp8(a, c.parts, fp8sh, st);
  }
  if (f == DSGX_FMT_INT4_G32) {
    if (c.up == 1) return launch_decode_int4_mfma(a, c.parts & 3, b16sh ? DSGX_FMT_BF16 : fp8sh ? DSGX_FMT_FP8_B128 : 0, st);
    if (fp8sh) return fail(DSGX_EUNSUPPORTED, "moe_decode: INT4 experts with an FP8 shared expert run on variant 1 only (dsgx_decode_cfg::up = 1 or -1)");
    return launch_decode_int4(a, c.parts, b16sh, st);
  }
  if (f == DSGX_FMT_MXFP4_G32) {
    if (b16sh) return fail(DSGX_EUNSUPPORTED, "dsk_moe: MXFP4 experts take an FP8 shared expert (ue8m0 scales per 32 x 32)");
    return launch_decode_mxfp4_mfma(a, c.parts & 3, fp8sh, st);
  }
  if (fp8sh || b16sh) return fail(DSGX_EUNSUPPORTED, "moe_decode: BF16 experts with a fused shared expert are not built");
  return launch_decode_bf16(a, c.parts, st);
}

// ---- DeepSeek's decode MoE: dsk::moe / dsk::moe_routed (ds41f-4xgx10-switchless/engine/kernels/dsk.h:199-241) -----------------
extern "C" {
void dsgx_dsk_cfg_default(dsgx_dsk_cfg* c) {
  if (!c) return;
  c->swiglu_limit = 10.f;
  c->logits = c->bias = nullptr;
  c->route_scale = 1.f;
  c->parts = 3;
}
int dsgx_dsk_moe(const dsgx_layer_w* L, const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* w, void* ws, float* y,
                 float* ys, void* stream, const dsgx_dsk_cfg* cfg) {
  dsgx_dsk_cfg c;
  if (cfg) c = *cfg;
  else dsgx_dsk_cfg_default(&c);
  if (!L || !xq || !xs || !ws || !y || !ys) return fail(DSGX_EINVAL, "dsk_moe: null layer, rows, workspace or output");
  if (M < 1 || M > DSGX_MAX_ROWS) return fail(DSGX_EINVAL, "dsk_moe: M=%d", M);
  if (L->H <= 0 || L->H % 256 || L->I <= 0 || L->I % 256) return fail(DSGX_EINVAL, "dsk_moe: hidden %d, intermediate %d (multiples of 256)", L->H, L->I);
  if (!(c.swiglu_limit > 0.f)) return fail(DSGX_EINVAL, "dsk_moe: swiglu_limit %g", (double)c.swiglu_limit);
  if ((uintptr_t)xq & 7) return fail(DSGX_EINVAL, "dsk_moe: the rows' codes must be 8-byte aligned");
  const WsLayout lay{L->I, L->H};
  uint16_t* xd = reinterpret_cast<uint16_t*>(static_cast<uint8_t*>(ws) + lay.xdeq_off());
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.up = 1, d.parts = c.parts, d.logits = c.logits, d.bias = c.bias, d.route_scale = c.route_scale, d.score_fn = 1;
  return moe_decode_at(L, xd, idx, w, M, ws, lay, y, ys, stream, &d, DskIn{1, c.swiglu_limit, xq, xs});
}
size_t dsgx_dsk_ws_bytes(int H, int I) {
  if (H <= 0 || I <= 0) return 0;
  return WsLayout{I, H}.dsk_bytes();
}
int dsgx_dsk_moe_stacked(const dsgx_dsk_weights* W, const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* w, void* ws,
                         float* y, void* stream, const dsgx_dsk_cfg* cfg, int* idx_out, float* wts_out) {
  dsgx_dsk_cfg c;
  if (cfg) c = *cfg;
  else dsgx_dsk_cfg_default(&c);
  if (!W || !xq || !xs || !ws || !y) return fail(DSGX_EINVAL, "dsk_moe_stacked: null weights, rows, workspace or output");
  if (!W->w1 || !W->s1 || !W->w3 || !W->s3 || !W->w2 || !W->s2) return fail(DSGX_EINVAL, "dsk_moe_stacked: the routed experts need w1, s1, w3, s3, w2, s2");
  const bool sh = W->sh_w1 != nullptr;
  if (sh && (!W->sh_s1 || !W->sh_w3 || !W->sh_s3 || !W->sh_w2 || !W->sh_s2)) return fail(DSGX_EINVAL, "dsk_moe_stacked: the shared expert needs all of sh_w1 ... sh_s2");
  if (M < 1 || M > DSGX_MAX_ROWS) return fail(DSGX_EINVAL, "dsk_moe_stacked: M=%d", M);
  if (W->H <= 0 || W->H % 256 || W->I <= 0 || W->I % 256) return fail(DSGX_EINVAL, "dsk_moe_stacked: hidden %d, intermediate %d (multiples of 256)", W->H, W->I);
  if (!(c.swiglu_limit > 0.f)) return fail(DSGX_EINVAL, "dsk_moe_stacked: swiglu_limit %g", (double)c.swiglu_limit);
  if (((uintptr_t)xq & 7) || (((uintptr_t)W->w1 | (uintptr_t)W->w3 | (uintptr_t)W->w2) & 15))
    return fail(DSGX_EINVAL, "dsk_moe_stacked: the rows' codes must be 8-byte aligned, the weight tensors 16-byte aligned");
  if ((idx_out == nullptr) != (wts_out == nullptr)) return fail(DSGX_EINVAL, "dsk_moe_stacked: idx_out and wts_out go together");
  dsgx_layer_w L{};
  L.pool = W->w1, L.desc = nullptr, L.fmt = DSGX_FMT_MXFP4_G32, L.H = W->H, L.I = W->I, L.E = W->E, L.topk = W->topk;
  if (sh) {
    L.sh.g = W->sh_w1, L.sh.u = W->sh_w3, L.sh.d = W->sh_w2;
    L.sh.gs = reinterpret_cast<const float*>(W->sh_s1), L.sh.us = reinterpret_cast<const float*>(W->sh_s3), L.sh.ds = reinterpret_cast<const float*>(W->sh_s2);
  }
  const WsLayout lay{L.I, L.H};
  uint8_t* wsb = static_cast<uint8_t*>(ws);
  uint16_t* xd = reinterpret_cast<uint16_t*>(wsb + lay.xdeq_off());
  float* ys = reinterpret_cast<float*>(wsb + lay.dsk_ys_off());
  dsgx_decode_cfg d;
  dsgx_decode_cfg_default(&d);
  d.up = 1, d.parts = c.parts, d.logits = c.logits, d.bias = c.bias, d.route_scale = c.route_scale, d.score_fn = 1;
  DskIn in{1, c.swiglu_limit, xq, xs};
  in.stacked = W, in.idx_out = idx_out, in.wts_out = wts_out;
  return moe_decode_at(&L, xd, idx, w, M, ws, lay, y, ys, stream, &d, in);
}
}  // extern "C"

// ---- the barrier's error flag ------------------------------------------------------------------------------------------
extern "C" {
int dsgx_decode_status(const dsgx_layer_w* L, void* ws, void* stream) {
  if (!L || L->I <= 0 || L->H <= 0) return fail(DSGX_EINVAL, "decode_status: null or empty layer");
  WsLayout lay{L->I, L->H};
  if (!ws) {
    void* p = nullptr;
    if (int rc = static_ws(&p)) return rc;
    ws = p, lay = kStaticLayout;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* bar = static_cast<uint8_t*>(ws) + lay.bar_off();
  int flag = 0;
  DSGX_HIP(hipMemcpyAsync(&flag, bar + (size_t)(2 * kBarGroups + 1) * kBarLine * 4, 4, hipMemcpyDeviceToHost, st));
  DSGX_HIP(hipStreamSynchronize(st));
  if (!flag) return DSGX_OK;
  // the barrier's counters may be anywhere after a wait that gave up: all of its words back to zero
  DSGX_HIP(hipMemsetAsync(bar, 0, kBarBytes, st));
  DSGX_HIP(hipStreamSynchronize(st));
  return fail(DSGX_ETIMEOUT, "moe_decode: a workgroup gave up waiting at the fused kernel's grid barrier (the grid was not resident: "
                             "another kernel or process held part of the GPU); the outputs of the steps since the last check are invalid. "
                             "The workspace is usable again; dsgx_decode_cfg::down = 1 runs the step without a grid barrier");
}

// ---- the decode step on the library's own workspace ----------------------------------------------------------------------
int dsgx_moe_decode_noalloc(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, float* yr, float* ys,
                            void* stream, const dsgx_decode_cfg* cfg) {
  if (!L) return fail(DSGX_EINVAL, "moe_decode_noalloc: null layer");
  if (L->I < 1 || L->I > DSGX_NOALLOC_MAX_I || L->H < 1 || L->H > DSGX_NOALLOC_MAX_H)
    return fail(DSGX_EINVAL, "moe_decode_noalloc: hidden %d, intermediate %d exceed the built-in workspace (hidden <= %d, intermediate <= %d); "
                             "use dsgx_moe_decode with a workspace of dsgx_decode_ws_bytes()", L->H, L->I, DSGX_NOALLOC_MAX_H, DSGX_NOALLOC_MAX_I);
  void* ws = nullptr;
  if (int rc = static_ws(&ws)) return rc;
  return moe_decode_at(L, x, idx, w, M, ws, kStaticLayout, yr, ys, stream, cfg);
}

}  // extern "C"
