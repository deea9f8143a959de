/* dsgx.h - the C ABI of the MI355X (gfx950) build of dsgx10's quantised-MoE hot path.
 *
 * Every entry point is what the reference engine's own C++ operator for this path would bind through an FFI:
 * plain pointers and sizes, no C++ types, no HIP types (a stream is passed as void*, it is a hipStream_t).
 * bf16 values are uint16_t bit patterns. All device pointers are caller-owned; every call is asynchronous on
 * the given stream and allocates nothing.
 *
 * Error convention: every function that can fail returns 0 on success and a non-zero dsgx_status otherwise and
 * leaves a message in a thread-local buffer (dsgx_last_error()). The reference dies (prints and aborts:
 * altar1-4xgx10-switchless/engine/common/check.h:8-21); the C++ mirror headers under include/gx, include/glm and
 * include/dsk turn a non-zero status into the same die().
 *
 * Weight formats. The reference's formats tags 0 (NVFP4), 2 (INT4) and 3 (BF16) name GB10 lane-map block tilings
 * (altar1-4xgx10-switchless/engine/experts/experts.h:29-46). Those tilings are not used here: on gfx950 a 64-lane
 * wavefront reading 16 bytes a lane covers 1 KiB of a K-contiguous row, so the checkpoint's own row-major tensors are
 * already the coalesced streaming layout. The tags below name them; the reference's tags are refused.
 */
#ifndef DSGX_H_
#define DSGX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DSGX_API __attribute__((visibility("default")))

typedef enum dsgx_status {
  DSGX_OK = 0,
  DSGX_EINVAL = 1,      /* an argument the reference would die() on */
  DSGX_EFORMAT = 2,     /* unknown / unsupported weight format tag (never guessed) */
  DSGX_EUNSUPPORTED = 3,/* a reference feature that has no meaning on one GPU (ring posting) or is not built */
  DSGX_EHIP = 4,        /* a HIP runtime error (message has hipGetErrorString) */
  DSGX_ETIMEOUT = 5     /* dsgx_decode_status: a fused decode step gave up at its grid barrier; its outputs are invalid */
} dsgx_status;

/* Weight format tags (dsgx_mat_desc::fmt, dsgx_layer_w::fmt, dsgx_gemv_seg::fmt). */
enum {
  DSGX_FMT_REF_NVFP4 = 0, /* reference tilings: refused */
  DSGX_FMT_REF_INT4 = 2,
  DSGX_FMT_REF_BF16 = 3,
  /* FP8 e4m3fn codes u8 [N][K] row-major, then (256-byte aligned) f32 scales [ceil(N/128)][K/128]:
     W(n,k) = e4m3(code) * S[n/128][k/128]   (engine/experts/tests/testdata.h:120-125, attn/tools/pack.py:216-241) */
  DSGX_FMT_FP8_B128 = 16,
  /* compressed-tensors pack-quantized INT4, group 32 along K, asymmetric, the checkpoint's three tensors back to
     back, each 256-byte aligned: weight_packed u32 [N][K/8] (value k at bits 4(k%8) of word k/8), weight_scale
     bf16 [N][K/32], weight_zero_point u32 [N/8][K/32] (row n at bits 4(n%8)):
     W(n,k) = bf16_rne((u - u_z) * s)       (engine/experts/layout.h:24-42, docs/model.md:111-195) */
  DSGX_FMT_INT4_G32 = 18,
  /* bf16 bits [N][K] row-major */
  DSGX_FMT_BF16 = 19,
  /* OCP MXFP4, the routed experts of DeepSeek's layers: e2m1 pairs u8 [N][K/2] row-major (the low nibble the even k),
     then (256-byte aligned) ue8m0 scales u8 [N][K/32]: W(n,k) = e2m1(nibble) * 2^(S[n][k/32] - 127)
     (ds41f-4xgx10-switchless/engine/kernels/README.md, L3's source form; ref/torchref/kernel.py:111-117). K a multiple of 256. */
  DSGX_FMT_MXFP4_G32 = 20,
  /* FP8 e4m3fn codes u8 [N][K] row-major, then (256-byte aligned) ue8m0 scales u8 [N/32][K/32], one a 32 x 32 block
     (the same layers' shared expert: README.md L1's source form; kernel.py:105-108 with block 32) */
  DSGX_FMT_FP8_B32E = 21
};

/* Bytes of one [N][K] matrix in a format, parts laid as above (0 for an unknown tag or a bad shape).
   Mirrors gx::mat_bytes (engine/experts/experts.h:47-50). */
DSGX_API size_t dsgx_mat_bytes(uint32_t fmt, int N, int K);
/* Byte offsets, from the matrix's start, of its second and third part (scales; zero points). */
DSGX_API size_t dsgx_mat_scale_off(uint32_t fmt, int N, int K);
DSGX_API size_t dsgx_mat_zp_off(uint32_t fmt, int N, int K);

/* One routed matrix of one expert. Mirrors gx::MatDesc, 64 bytes (engine/experts/experts.h:58-64). */
typedef struct dsgx_mat_desc {
  uint64_t off;     /* byte offset of the matrix in the pool, a multiple of 256 */
  float s2;         /* per-tensor f32 factor applied in the epilogue; exactly 1 for INT4, BF16 and FP8_B128 */
  uint32_t fmt;
  uint32_t rsv[12]; /* zero */
} dsgx_mat_desc;

/* A shared expert fused into the routed kernels. Mirrors gx::SharedW (engine/experts/experts.h:66-87).
   FP8: g, u [I][H] and d [H][I] e4m3 row-major with f32 scales gs, us [I/128][H/128], ds [H/128][I/128].
   BF16: bgu [2I][H] bf16 row-major with rows 2i = gate i, 2i+1 = up i (the reference's interleave), bd [H][I]. */
typedef struct dsgx_shared_w {
  const uint8_t *g, *u, *d;
  const float *gs, *us, *ds;
  const uint8_t *bgu, *bd;
} dsgx_shared_w;

/* One MoE layer's weights. Mirrors gx::LayerW (engine/experts/experts.h:91-97); the reference's compile-time shapes
   (experts.h:18-26) are runtime fields here. desc is a DEVICE array [E][3]: gate [I][H], up [I][H], down [H][I]. */
typedef struct dsgx_layer_w {
  const uint8_t* pool;
  const dsgx_mat_desc* desc;
  dsgx_shared_w sh;
  uint32_t fmt;
  int32_t H, I, E, topk;
} dsgx_layer_w;

#define DSGX_MAX_ROWS 16   /* decode rows a step (engine/experts/experts.h:24) */
#define DSGX_MAX_TOPK 8
#define DSGX_MAX_UNION (DSGX_MAX_ROWS * DSGX_MAX_TOPK) /* 128 (engine/experts/experts.h:25) */
#define DSGX_SH_SLOT DSGX_MAX_UNION /* the shared expert's slot in the decode h workspace (experts.h:26) */
#define DSGX_MAX_EXPERTS 512
#define DSGX_MAX_CHUNK 8192 /* prefill rows a chunk (engine/experts/experts.h:155) */

/* ---- routing: gx::route (engine/experts/experts.h:99-102, route.cu:11-33) --------------------------------------
   logits f32 [M][E], bias f32 [E] (selection only; may be null = 0) -> idx i32 [M][topk] (descending key, ties to the
   lower id), w f32 [M][topk] = s / (sum + 1e-20) * route_scale, s = sigmoid(logit). topk <= 8, E <= 512.
   score_fn 0: sigmoid (GLM / DeepSeek-V3); 1: sqrt(softplus) (ds41f-4xgx10-switchless/engine/kernels/common.cuh:261-315). */
DSGX_API int dsgx_route(const float* logits, const float* bias, int M, int E, int topk, float route_scale, int score_fn,
                        int* idx, float* w, void* stream);

/* ---- decode: gx::moe_decode (engine/experts/experts.h:104-147, decode.cu:708-730) ------------------------------- */
#define DSGX_UP_PREFILL_ORDER 6 /* gx::kUpPrefillOrder (engine/experts/experts.h:138) */
#define DSGX_UP_PREFILL_ORDER_ACT_FP8 7 /* the same against a prefill on FP8 activations (dsgx_prefill_cfg::act_fp8 = 1, its default) */
typedef struct dsgx_decode_cfg {
  int32_t up, down;        /* kernel variants (the reference's DecodeCfg::up / down choose among its launch shapes too).
                              up -1 (the default): the faster of the two below for the layer's format and row count
                              (INT4_G32: 1; FP8_B128: 0 at one row, 1 from two rows on; BF16: 0). up 0: dot products on the
                              vector unit; up 1: on the bf16 MFMA (FP8_B128 and INT4_G32 layers, 1-16 rows). A row's bits are
                              the same in any batch within a variant; the two variants differ in the order of the f32 adds
                              inside a dot product, so a caller that needs a row's bits not to depend on the row count
                              names the variant. up DSGX_UP_PREFILL_ORDER (6, the reference's kUpPrefillOrder): the rows go
                              through the prefill kernels with bf16 activations and yr, ys are bit for bit those of
                              dsgx_moe_prefill with act_fp8 = 0 on the same rows; up DSGX_UP_PREFILL_ORDER_ACT_FP8 (7; FP8_B128
                              layers): with FP8 activations, the bits of dsgx_moe_prefill's DEFAULT configuration (act_fp8 = 1) - a
                              caller that verifies drafted tokens against a prefill names the one its prefill uses. Both: parts 3
                              only; the workspace then holds the chunk's intermediates (dsgx_prefill_view's layout) instead of the
                              step's h slots. down (with up 0) 0: both phases in one persistent
                              kernel; 1: two launches */
  int32_t parts;           /* 1 up only, 2 down only, 3 both (bench) */
  int32_t ysum;            /* 1: yr += ys in f32 after the routed experts (experts.h:132-136) */
  const float* logits;     /* fused routing (experts.h:123-127): with logits (+ optional bias) idx, w are not read */
  const float* bias;
  float route_scale;       /* used by fused routing */
  int32_t score_fn;
  const void* post;        /* the reference's ring channel (experts.h:128-131): must be null on one GPU */
} dsgx_decode_cfg;
DSGX_API void dsgx_decode_cfg_default(dsgx_decode_cfg* cfg);
/* Workspace bytes of a decode step (gx::decode_ws_bytes; engine/experts/decode.cu:33-35): h bf16
   [DSGX_MAX_UNION + 1 slots][DSGX_MAX_ROWS][I] plus the grid barrier's counters (a few KiB). Zero it once before the first call. */
DSGX_API size_t dsgx_decode_ws_bytes(const dsgx_layer_w* L);
/* Byte offset in ws of a 32-bit error flag. The default decode step is one persistent kernel whose workgroups meet at a
   barrier in device memory between the two phases; the wait is bounded, and a workgroup that gives up (it can only
   happen when the grid is not resident, e.g. the GPU is shared with another process) sets this flag to 1 and the step's
   outputs are invalid. No counterpart in the reference (its two kernels are ordered by the stream). */
DSGX_API size_t dsgx_decode_ws_flag_offset(const dsgx_layer_w* L);
/* Reads that flag: waits for `stream`, returns DSGX_OK when no step since the last check gave up at the barrier, else
   DSGX_ETIMEOUT after putting the barrier's words back to their initial state (the workspace is usable again; the outputs
   of the steps since the last check are invalid). ws null: the workspace of dsgx_moe_decode_noalloc. Synchronous, so not for
   use under stream capture: call it where the host waits for results anyway. No counterpart in the reference (its two
   kernels are ordered by the stream and cannot time out); the C++ mirrors expose it as gx::decode_check(). */
DSGX_API int dsgx_decode_status(const dsgx_layer_w* L, void* ws, void* stream);
/* x bf16 [M][H]; idx, w from dsgx_route; yr, ys f32 [M][H]. ys is written when the layer has a fused shared expert,
   otherwise it is an input (only read with ysum). h of the step stays in ws: slot s (the s-th picked expert in
   expert-id order) at ((s * M + m) * I + c), the shared expert's at slot DSGX_SH_SLOT. */
DSGX_API int dsgx_moe_decode(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, void* ws,
                             float* yr, float* ys, void* stream, const dsgx_decode_cfg* cfg);
/* dsgx_moe_decode on a workspace inside the library, for callers that cannot allocate device memory (code under HIP graph
   capture, serving loops and harnesses that forbid hipMalloc): no workspace argument, no allocation of any kind. It has
   no counterpart in the reference, whose moe_decode always takes the caller's workspace. The workspace is one array of
   34.0 MB on every GPU the library runs on, held until the process ends; it fits layers with hidden <= DSGX_NOALLOC_MAX_H
   and intermediate <= DSGX_NOALLOC_MAX_I (larger ones: DSGX_EINVAL). All calls on a GPU share it: calls that overlap on
   one GPU (two streams) race; stream-ordered calls are fine (h and the barrier's words are rewritten by every step).
   Same arguments, bits and errors as dsgx_moe_decode otherwise. */
#define DSGX_NOALLOC_MAX_H 6144
#define DSGX_NOALLOC_MAX_I 2048
DSGX_API int dsgx_moe_decode_noalloc(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int M, float* yr,
                                     float* ys, void* stream, const dsgx_decode_cfg* cfg);
/* out = bf16(bf16(R) + bf16(S)): gx::finalize (engine/experts/experts.h:146-147, decode.cu:591-598) */
DSGX_API int dsgx_finalize(const float* R, const float* S, int n, uint16_t* out, void* stream);

/* ---- DeepSeek's decode MoE: dsk::moe / dsk::moe_routed (ds41f-4xgx10-switchless/engine/kernels/dsk.h:199-241) ------------
   L: MXFP4_G32 experts (pool + descriptors as for the other formats; desc.s2 = 1) and, optionally, the FP8 shared expert
   in L->sh.g / u / d (e4m3 [I][H], [I][H], [H][I]) with its ue8m0 scales per 32 x 32 block in L->sh.gs / us / ds (the three
   pointers then address BYTES [N/32][K/32], not floats). xq, xs = act_quant(x): e4m3 [M][H] and ue8m0 [M][H/32]. idx, w
   [M][topk] from the router, or cfg->logits (+ bias): the sqrt-softplus router runs inside the kernel.
   Arithmetic (engine/kernels/moe.cu:519-534, 974-981; ref/inference/model.py:841-851): per expert gate, up = bf16(f32 sums of
   the block-scaled products), up clamped to +-limit and gate from above, h = bf16(w_row * (silu(gate) * up)) (no weight for
   the shared expert), h quantised like x, the expert's w2 output rounded to bf16; y = the f32 sum of the picked experts'
   outputs in expert-id order, then the shared expert's. y f32 [M][H] the sum, ys f32 [M][H] the shared expert's bf16
   output alone. ws: dsgx_decode_ws_bytes(L), zeroed once. M <= 16 (9-16: two passes). */
typedef struct dsgx_dsk_cfg {
  float swiglu_limit;   /* 10 */
  const float* logits;  /* fused routing (moe_routed): f32 [M][E]; idx, w are then not read */
  const float* bias;
  float route_scale;
  int32_t parts;        /* 1 gate/up only, 2 down only, 3 both (bench) */
} dsgx_dsk_cfg;
DSGX_API void dsgx_dsk_cfg_default(dsgx_dsk_cfg* cfg);
DSGX_API int dsgx_dsk_moe(const dsgx_layer_w* L, const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* w, void* ws,
                          float* y, float* ys, void* stream, const dsgx_dsk_cfg* cfg);
/* The same layer as the reference hands it over: dsk::MoeWeights (engine/kernels/dsk.h:199-209), the routed experts stacked
   by expert id in six tensors (expert e at e times the per-expert size) and the FP8 shared expert in six more, all in the
   row-major forms of DSGX_FMT_MXFP4_G32 / DSGX_FMT_FP8_B32E (not the reference's GB10 lane tilings):
     w1, w3 e2m1 pairs [E][I][H/2]; s1, s3 ue8m0 [E][I][H/32]; w2 [E][H][I/2]; s2 [E][H][I/32];
     sh_w1, sh_w3 e4m3 [I][H]; sh_s1, sh_s3 ue8m0 [I/32][H/32]; sh_w2 [H][I]; sh_s2 [H/32][I/32] (sh_w1 null: no shared expert).
   dsgx_dsk_moe_stacked is dsk::moe (idx, w given) and dsk::moe_routed (cfg->logits given; idx_out / wts_out [M][topk],
   optional, then receive the router's selection, dsk.h:234-241): y f32 [M][H] as dsgx_dsk_moe's. The shared expert's rows
   stay inside the workspace (the reference keeps them in shared memory): ws of dsgx_dsk_ws_bytes(H, I), zeroed once. */
typedef struct dsgx_dsk_weights {
  const uint8_t *w1, *s1, *w3, *s3, *w2, *s2;
  const uint8_t *sh_w1, *sh_s1, *sh_w3, *sh_s3, *sh_w2, *sh_s2;
  int32_t H, I, E, topk;
} dsgx_dsk_weights;
DSGX_API size_t dsgx_dsk_ws_bytes(int H, int I);
DSGX_API int dsgx_dsk_moe_stacked(const dsgx_dsk_weights* W, const uint8_t* xq, const uint8_t* xs, int M, const int* idx, const float* w,
                                  void* ws, float* y, void* stream, const dsgx_dsk_cfg* cfg, int* idx_out, float* wts_out);

/* DeepSeek's prefill MoE: dsk::moe_prefill (ds41f-4xgx10-switchless/engine/kernels/dsk.h:268-295, prefill.cu:1605-1675) for a
   chunk of T rows given as act_quant(x) (xq e4m3 [T][H], xs ue8m0 [T][H/32]) with the router's idx, w [T][topk]: picks
   bucketed by expert, grouped GEMMs on v_mfma_scale_f32_16x16x128_f8f6f4 (e2m1 / e4m3 weights, e4m3 rows and both ue8m0
   scale tensors go to the instruction as stored), dsgx_dsk_moe's arithmetic per expert (clamped SwiGLU times the routing
   weight, h quantised per 32, each pick's output rounded to bf16), then per row the f32 sum in expert-id order, the shared
   expert last: y f32 [T][H]. The sums inside a dot product are the matrix unit's (block-scaled, 128 k an instruction),
   not the decode kernels' bf16-MFMA sums: a row's y agrees with dsgx_dsk_moe_stacked's to the tolerance both are tested
   at, not bit for bit. phases as dsk::MoePCfg: 1 bucketing, 2 shared expert, 4 routed gate/up, 8 routed down, 16 combine.
   ws: dsgx_dsk_prefill_ws_bytes(...) bytes, no initialisation needed. H a multiple of 256, I of 128, T <= DSGX_MAX_CHUNK. */
typedef struct dsgx_dsk_prefill_cfg {
  float swiglu_limit;  /* 10 */
  int32_t phases;      /* 31 */
} dsgx_dsk_prefill_cfg;
DSGX_API void dsgx_dsk_prefill_cfg_default(dsgx_dsk_prefill_cfg* cfg);
DSGX_API size_t dsgx_dsk_prefill_ws_bytes(int H, int I, int E, int topk, int T);
DSGX_API int dsgx_dsk_moe_prefill(const dsgx_dsk_weights* W, const uint8_t* xq, const uint8_t* xs, int T, const int* idx, const float* w,
                                  void* ws, float* y, void* stream, const dsgx_dsk_prefill_cfg* cfg);
/* The workspace's intermediates after a call: device pointers into ws (bucket positions as dsgx_prefill_view). h: bf16
   [position][I] before its quantisation, hq / hs: as the down GEMM reads it (e4m3, ue8m0 [position][I/32]); d: each pick's
   output bf16 [position][H]; hsh / dsh: the shared expert's h [T][I] and output [T][H]. */
typedef struct dsgx_dsk_prefill_view {
  const int *rpos, *re, *off, *perm;
  const uint16_t *h, *hsh, *d, *dsh;
  const uint8_t *hq, *hs;
} dsgx_dsk_prefill_view;
DSGX_API int dsgx_dsk_prefill_view_get(const dsgx_dsk_weights* W, void* ws, int T, dsgx_dsk_prefill_view* out);

/* The residual add after the expert step and the next layer's RMSNorm, the local half of the reference's
   comm::glm::allreduce_add_norm / allreduce2_add_norm (engine/comm/glmcoll.h:34-62; the norm: engine/attn/prep.cu:12-66),
   M rows of H (a multiple of 2048, up to 16384):
     sum = part, or with part2 bf16(bf16(part) + bf16(part2)) (the old combine of yr and ys)
     h   = bf16(f32(res) + sum), the contract's single rounding (ref/glmref.py:269-276 add_residual); round2: the sum is
           rounded to bf16 first (the engine's order before its decision 8)
     xn  = bf16(w * bf16(h * rstd)), rstd = 1 / sqrt(mean(h^2) + eps), statistics in f32
   res_out (may be res itself) receives h, xn the normed row for the next layer; either may be null. */
DSGX_API int dsgx_add_norm(const float* part, const float* part2, int M, int H, const uint16_t* res, uint16_t* res_out,
                           const uint16_t* w, float eps, uint16_t* xn, int round2, void* stream);

/* ---- prefill: gx::moe_prefill (engine/experts/experts.h:149-193, prefill.cu:1056-1116) --------------------------- */
typedef struct dsgx_prefill_cfg {
  int32_t shared;   /* run the fused shared expert (if the layer has one) */
  int32_t phases;   /* gx::PrefillPhase bits: 1 bucket, 2 up, 4 down, 8 combine, 16 shared; 31 all */
  int32_t act_fp8;  /* FP8 layers: 1 = quantise activations per row and 128 k to e4m3 and run the fp8 MFMA
                       (ds41f-4xgx10-switchless/ref/torchref/kernel.py:56-77, ref/inference/kernel.py:207-274);
                       0 = bf16 activations, weights widened to bf16 (the altar-1 contract) */
  int32_t fast_act; /* FP8 activations only. 0 (the default): SwiGLU with expf() and the IEEE division, as the decode kernels
                       and the reference compute it (engine/experts/decode.cu:110-113); 1: the hardware's exponential and
                       reciprocal (each within 1 ulp; h then differs from the exact form's in about one value in 10^4, by one
                       bf16 step), for callers that trade that for the epilogue's time */
  int32_t tile_order; /* FP8 activations only: the order in which the grouped GEMMs walk the tiles (the reference's
                       prefill_tuning tord, ds41f-4xgx10-switchless/engine/kernels/dsk.h:252, prefill.cu:658-668). 0: by
                       expert id, an expert's tiles next to each other; 1: the experts by falling count, their
                       256-position tiles and the remainders merged evenly (tiles bound by the matrix unit beside tiles
                       bound by the weight stream); 2: every 256-position tile first, then the remainders by falling
                       size; -1 (the default): the library's choice (0: on MI355X 1 and 2 measured no faster). The
                       results do not depend on it; a call that runs later phases alone names the same order as the
                       call that ran the bucketing (any order finds a valid list). */
} dsgx_prefill_cfg;
DSGX_API void dsgx_prefill_cfg_default(dsgx_prefill_cfg* cfg);
DSGX_API size_t dsgx_prefill_ws_bytes(const dsgx_layer_w* L, int T);
DSGX_API int dsgx_moe_prefill(const dsgx_layer_w* L, const uint16_t* x, const int* idx, const float* w, int T, void* ws,
                              float* yr, float* ys, void* stream, const dsgx_prefill_cfg* cfg);
/* The workspace's intermediates after a call (gx::prefill_view, experts.h:184-190): device pointers into ws. */
typedef struct dsgx_prefill_view {
  const int *rpos, *re;      /* [T][topk]: per row its picks in expert-id order: bucket position, expert */
  const uint16_t *h, *hsh;   /* h bf16 [position][I]; shared expert's h [T][I] */
  const int *off;            /* [E+1] bucket offsets */
  const int *perm;           /* [T*topk] bucket position -> row */
} dsgx_prefill_view;
DSGX_API int dsgx_prefill_view_get(const dsgx_layer_w* L, void* ws, int T, dsgx_prefill_view* out);

/* ---- dense GEMV: glm::gemv (engine/attn/attn.h:59-123, gemv.cu:522-543) ------------------------------------------ */
enum { DSGX_OUT_BF16 = 0, DSGX_OUT_F32 = 1, DSGX_OUT_SWIGLU = 2 };
typedef struct dsgx_gemv_seg {
  int32_t fmt;        /* DSGX_FMT_BF16, DSGX_FMT_INT4_G32, DSGX_FMT_FP8_B128 */
  const void* w;      /* the matrix in its format; INT4: weight_packed */
  const void* s;      /* FP8: f32 scales [ceil(N/rs)][K/ks]; INT4: bf16 scales [N][K/32] */
  const void* zp;     /* INT4: weight_zero_point u32 [N/8][K/32] */
  int32_t n;          /* rows of W (outputs), a multiple of 8 */
  int32_t rs, ks;     /* FP8 scale block (rows, k): 128, 128 */
  void* y;
  int32_t ldy;        /* y's row stride in elements */
} dsgx_gemv_seg;
/* y[r][n] = sum_k x[r][k] W[n][k]; x bf16 [rows][ldx], rows 1..16, K a multiple of 128 (INT4: of 256).
   out: DSGX_OUT_*; SwiGLU: rows interleaved gate/up in pairs. splitk 1, 2 or 4 (engine/attn/attn.h:119): with 2 or 4 the
   waves of a workgroup share a row pair's K range and their sums are added in a fixed order (for matrices of few rows,
   e.g. the router's; ignored above 32 rows a CU, where whole-K waves already fill the chip). A given splitk always gives
   the same bits; different values add in different orders. */
DSGX_API int dsgx_gemv(const uint16_t* x, int ldx, int rows, int K, const dsgx_gemv_seg* segs, int nseg, int out,
                       int splitk, void* stream);
/* dsgx_add_norm fused into the GEMV that reads its output: y = W xn with xn made inside the GEMV kernel (every workgroup
   computes the M normed rows for itself from part, res and w - a few KB out of L2 - and workgroup 0 writes res_out and xn for
   the kernels that follow). One launch where the reference's step has two (allreduce_add_norm, then the router's or the next
   projection's gemv: engine/model/model.cu:309-352): same bits as dsgx_add_norm followed by dsgx_gemv. rows 1..8, K = the
   hidden size (a multiple of 2048), the segments of one format; res_out must not alias res. */
typedef struct dsgx_norm_in {
  const float* part;
  const float* part2;      /* may be null */
  const uint16_t* res;
  uint16_t* res_out;       /* may be null */
  const uint16_t* w;
  float eps;
  uint16_t* xn;            /* may be null */
  int32_t round2;
} dsgx_norm_in;
DSGX_API int dsgx_add_norm_gemv(const dsgx_norm_in* n, int rows, int K, const dsgx_gemv_seg* segs, int nseg, int out, int splitk,
                                void* stream);

/* glm::dequant_int4 (engine/attn/attn.h:154-158): the contract's bf16 weight [N][ld] from the canonical tensors */
DSGX_API int dsgx_dequant_int4(const void* packed, const void* scale, const void* zp, int N, int K, uint16_t* out,
                               size_t ld, void* stream);
/* The same through the streaming kernels' own in-register decode: the probe that pins the hot loops' INT4 arithmetic to
   the contract bit for bit, as the reference's k_deq does (engine/experts/tests/test_experts.cu:217-235). Bit-exact for
   positive scales below 2^124 (the checkpoint's are 2^-15 .. 2^-4; a negative scale, which the format forbids, gives
   +0 instead of -0 where u = u_z); dsgx_dequant_int4 is exact for every finite scale. */
DSGX_API int dsgx_probe_dequant_int4(const void* packed, const void* scale, const void* zp, int N, int K, uint16_t* out,
                                     size_t ld, void* stream);
/* FP8 codes -> bf16 bits of the exact e4m3 values [N][ld] (the widening the GEMV and MoE kernels use;
   engine/experts/formats.cuh:121-128, tests/test_experts.cu:124-134) */
DSGX_API int dsgx_widen_fp8(const void* codes, int N, int K, uint16_t* out, size_t ld, void* stream);
/* act_quant(x, 128): x bf16 [T][K] -> e4m3 codes [T][K], f32 scales [T][K/128]
   (ds41f-4xgx10-switchless/ref/torchref/kernel.py:56-77) */
DSGX_API int dsgx_act_quant(const uint16_t* x, int T, int K, uint8_t* q, float* s, void* stream);

/* Probe: raw[lane][16], the accumulator registers of one e4m3 MFMA with operands loaded the way the prefill kernels
   load them (pins the layouts in a test). form 0: v_mfma_f32_32x32x64_f8f6f4 over A [32][64], B [32][64];
   form 1: v_mfma_f32_16x16x128_f8f6f4 over A [16][128], B [16][128] (four registers a lane). */
DSGX_API int dsgx_probe_mfma_fp8(const void* A, const void* B, float* raw, int form, void* stream);
/* Probe: one v_mfma_scale_f32_16x16x128_f8f6f4. A [16][128 k]: e2m1 pairs (a_fp4 = 1: 64 bytes a row, the low nibble the even
   k) or e4m3 codes; B [16][128] e4m3; SA, SB [16][4]: the ue8m0 byte of each row's four groups of 32 k. out f32 [16][16]:
   out[i][j] = C[i][j] (null: 0) + sum over k of A[i][k] 2^(SA[i][k/32] - 127) B[j][k] 2^(SB[j][k/32] - 127), as the matrix unit
   adds it. */
DSGX_API int dsgx_probe_mfma_scaled(const void* A, const void* SA, const void* B, const void* SB, int a_fp4, const float* C, float* out,
                                    void* stream);
/* Probe: one v_mfma_f32_16x16x32_bf16 (the decode kernels' variant 1 and the bf16-activation prefill GEMMs): A, B bf16 bits
   [16][32], C f32 [16][16] or null; out[i][j] = C[i][j] + sum over k of A[i][k] B[j][k] as the matrix unit adds it. */
DSGX_API int dsgx_probe_mfma_bf16(const void* A, const void* B, const float* C, float* out, void* stream);
/* Probe: n times v_dot2_f32_bf16, the multiply-add of the vector-unit kernels (decode variant 0, the dense GEMV): a, b packed
   bf16 pairs [n] (the low half first), c f32 [n]; out[i] = c[i] + a[i].lo b[i].lo + a[i].hi b[i].hi as the instruction adds it. */
DSGX_API int dsgx_probe_dot2_bf16(const void* a, const void* b, const float* c, float* out, int n, void* stream);

/* ---- misc ---------------------------------------------------------------------------------------------------- */
DSGX_API const char* dsgx_last_error(void);
DSGX_API const char* dsgx_version(void);
/* A plain streaming-read kernel over n bytes (the bandwidth baseline the bench prints beside the kernels,
   as engine/experts/tests/bench_experts.cu:102-130 does); sink: 4 bytes of device memory. */
DSGX_API int dsgx_stream_read(const void* p, size_t n, void* sink, void* stream);
/* The same with the launch shape given: workgroups (of 256 threads) a CU and 16-byte loads in flight a lane (2, 4, 8, 16). */
DSGX_API int dsgx_stream_read_cfg(const void* p, size_t n, void* sink, int wgs_per_cu, int unroll, void* stream);
/* Seeded N(0, sigma) values, the generator the tests' oracle uses (splitmix64 of the reference, engine/experts/formats.cuh:
   131-136, keyed by (seed, tensor id, index) -> Box-Muller in f64): value i of tensor `tid` under `seed`. out: n values as
   f32 (bf16 = 0) or bf16 bits (bf16 = 1). For benchmark inputs made on the GPU. */
DSGX_API int dsgx_fill_normal(uint64_t seed, uint64_t tid, size_t n, double sigma, void* out, int bf16, void* stream);
/* What a launch costs with nothing in it, for the latency-bound calls' floor: kind 0 an empty kernel of one wavefront;
   kind 1 one wavefront doing two dependent 16-byte loads from p (at least 64 KiB; the second address comes out of the
   first's data) and one store to sink - the dependency chain of the smallest GEMV (activations, then weights, then y). */
DSGX_API int dsgx_launch_floor(int kind, const void* p, void* sink, void* stream);
/* A plain copy kernel (the reference for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE counters). */
DSGX_API int dsgx_stream_copy(const void* src, void* dst, size_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DSGX_H_ */
