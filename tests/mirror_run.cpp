// Test program: drives the C++ mirror headers (include/gx/experts.h, include/glm/attn.h) on the GPU the way the
// reference's runner calls its operators (altar1-4xgx10-switchless/engine/model/model.cu:309-343): route -> moe_decode
// (routing apart, then fused) -> finalize, one dense GEMV with K split four ways, and the residual add + RMSNorm. Inputs are raw files written by
// tests/test_gpu_mirror.py into a directory; outputs go back as raw files, and the test compares them bit for bit with
// what the same calls give through the ctypes binding of the C ABI.
//   mirror_run <dir> <fmt> <H> <I> <E> <topk> <M> <route scale> <up variant>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "glm/attn.h"
#include "glm/coll.h"
#include "gx/experts.h"

#define HIPOK(x)                                                          \
  do {                                                                    \
    hipError_t e_ = (x);                                                  \
    if (e_ != hipSuccess) die("%s: %s", #x, hipGetErrorString(e_));       \
  } while (0)

static std::vector<char> slurp(const std::string& p, bool optional = false) {
  std::vector<char> b;
  FILE* f = std::fopen(p.c_str(), "rb");
  if (!f) {
    if (optional) return b;
    die("cannot read %s", p.c_str());
  }
  std::fseek(f, 0, SEEK_END);
  b.resize((size_t)std::ftell(f));
  std::fseek(f, 0, SEEK_SET);
  if (!b.empty() && std::fread(b.data(), 1, b.size(), f) != b.size()) die("short read of %s", p.c_str());
  std::fclose(f);
  return b;
}
static void* upload(const std::vector<char>& b) {
  if (b.empty()) return nullptr;
  void* d = nullptr;
  HIPOK(hipMalloc(&d, b.size()));
  HIPOK(hipMemcpy(d, b.data(), b.size(), hipMemcpyHostToDevice));
  return d;
}
static void* dalloc(size_t n, int fill) {
  void* d = nullptr;
  HIPOK(hipMalloc(&d, n));
  HIPOK(hipMemset(d, fill, n));
  return d;
}
static void dump(const std::string& p, const void* d, size_t n) {
  std::vector<char> b(n);
  HIPOK(hipMemcpy(b.data(), d, n, hipMemcpyDeviceToHost));
  FILE* f = std::fopen(p.c_str(), "wb");
  if (!f || std::fwrite(b.data(), 1, n, f) != n) die("cannot write %s", p.c_str());
  std::fclose(f);
}

int main(int argc, char** argv) {
  if (argc != 10) die("usage: mirror_run dir fmt H I E topk M scale up");
  const std::string dir = std::string(argv[1]) + "/";
  const uint32_t fmt = (uint32_t)std::atoi(argv[2]);
  const int H = std::atoi(argv[3]), I = std::atoi(argv[4]), E = std::atoi(argv[5]), topk = std::atoi(argv[6]), M = std::atoi(argv[7]);
  const float scale = (float)std::atof(argv[8]);
  const int up = std::atoi(argv[9]);
  hipStream_t st;
  HIPOK(hipStreamCreate(&st));

  gx::LayerW L;
  L.fmt = fmt, L.H = H, L.I = I, L.E = E, L.topk = topk;
  L.pool = static_cast<const uint8_t*>(upload(slurp(dir + "pool.bin")));
  L.desc = static_cast<const gx::MatDesc*>(upload(slurp(dir + "desc.bin")));
  L.sh.g = static_cast<const uint8_t*>(upload(slurp(dir + "sh_g.bin", true)));
  L.sh.u = static_cast<const uint8_t*>(upload(slurp(dir + "sh_u.bin", true)));
  L.sh.d = static_cast<const uint8_t*>(upload(slurp(dir + "sh_d.bin", true)));
  L.sh.gs = static_cast<const float*>(upload(slurp(dir + "sh_gs.bin", true)));
  L.sh.us = static_cast<const float*>(upload(slurp(dir + "sh_us.bin", true)));
  L.sh.ds = static_cast<const float*>(upload(slurp(dir + "sh_ds.bin", true)));
  L.sh.bgu = static_cast<const uint8_t*>(upload(slurp(dir + "sh_bgu.bin", true)));
  L.sh.bd = static_cast<const uint8_t*>(upload(slurp(dir + "sh_bd.bin", true)));
  const uint16_t* x = static_cast<const uint16_t*>(upload(slurp(dir + "x.bin")));
  const float* logits = static_cast<const float*>(upload(slurp(dir + "logits.bin")));
  const float* bias = static_cast<const float*>(upload(slurp(dir + "bias.bin")));
  const float* resid = static_cast<const float*>(upload(slurp(dir + "resid.bin")));

  const size_t wsb = gx::decode_ws_bytes(L);
  void* ws = dalloc(wsb, 0);
  int* idx = static_cast<int*>(dalloc((size_t)M * topk * 4, 0xFF));
  float* w = static_cast<float*>(dalloc((size_t)M * topk * 4, 0xFF));
  float* yr = static_cast<float*>(dalloc((size_t)M * H * 4, 0xFF));
  float* ys = static_cast<float*>(dalloc((size_t)M * H * 4, 0xFF));
  float* yr2 = static_cast<float*>(dalloc((size_t)M * H * 4, 0xFF));
  float* ys2 = static_cast<float*>(dalloc((size_t)M * H * 4, 0xFF));
  uint16_t* out = static_cast<uint16_t*>(dalloc((size_t)M * H * 2, 0xFF));

  // the runner's sequence with the routing as its own launch ...
  gx::route(logits, bias, M, idx, w, st, true, E, topk, scale);
  gx::DecodeCfg dc;
  dc.up = up;
  gx::moe_decode(L, x, idx, w, M, ws, yr, ys, st, dc);
  gx::finalize(L, resid, yr, M, out, st);
  // ... and with the routing fused into the expert kernel and yr += ys
  gx::DecodeCfg df;
  df.up = up, df.logits = logits, df.bias = bias, df.route_scale = scale, df.ysum = true;
  gx::moe_decode(L, x, nullptr, nullptr, M, ws, yr2, ys2, st, df);
  gx::decode_check(L, ws, st);

  // one dense GEMV through glm::gemv: the shared expert's gate matrix (FP8 layers) or its interleaved gate/up (BF16)
  float* gv = nullptr;
  int gn = 0;
  if (L.sh.g || L.sh.bgu) {
    glm::GemvSeg seg;
    gn = L.sh.g ? I : 2 * I;
    gv = static_cast<float*>(dalloc((size_t)M * gn * 4, 0xFF));
    seg.fmt = L.sh.g ? glm::WFmt::kFP8 : glm::WFmt::kBF16;
    seg.w = L.sh.g ? static_cast<const void*>(L.sh.g) : static_cast<const void*>(L.sh.bgu);
    seg.s = L.sh.gs, seg.n = gn, seg.y = gv, seg.ldy = gn;
    glm::gemm(x, H, M, H, &seg, 1, glm::GemvOut::kF32, 4, st);  // (gemm() forwards its rows to gemv() sixteen at a time)
  }
  // the step's end (model.cu:343): h = bf16(resid16 + yr2) in place, xn = the next layer's RMSNorm of h
  uint16_t* res16 = static_cast<uint16_t*>(upload(slurp(dir + "res16.bin")));
  const uint16_t* normw = static_cast<const uint16_t*>(upload(slurp(dir + "normw.bin")));
  uint16_t* xn = static_cast<uint16_t*>(dalloc((size_t)M * H * 2, 0xFF));
  comm::glm::allreduce_add_norm(comm::DevChannel{}, yr2, M, H, res16, res16, normw, 1e-5f, xn, st);
  HIPOK(hipStreamSynchronize(st));
  dump(dir + "o_idx.bin", idx, (size_t)M * topk * 4);
  dump(dir + "o_w.bin", w, (size_t)M * topk * 4);
  dump(dir + "o_yr.bin", yr, (size_t)M * H * 4);
  dump(dir + "o_ys.bin", ys, (size_t)M * H * 4);
  dump(dir + "o_out.bin", out, (size_t)M * H * 2);
  dump(dir + "o_yr2.bin", yr2, (size_t)M * H * 4);
  dump(dir + "o_ys2.bin", ys2, (size_t)M * H * 4);
  if (gv) dump(dir + "o_gemv.bin", gv, (size_t)M * gn * 4);
  dump(dir + "o_h.bin", res16, (size_t)M * H * 2);
  dump(dir + "o_xn.bin", xn, (size_t)M * H * 2);
  std::printf("CHECK mirror_run ok  ws %zu bytes\n", wsb);
  return 0;
}
