// Test program: drives include/dsk/dsk.h on the GPU the way the reference's runner calls its DeepSeek MoE operators
// (ds41f-4xgx10-switchless/engine/kernels/dsk.h:171-241, 284-295): tile_fp4 / tile_fp8 at load time, experts stacked by id
// in MoeWeights, then router_topk -> moe, moe_routed with idx_out / wts_out, moe_prefill (the grouped GEMMs) and moe_prefill_rows (moe() sixteen rows at a time) over the same rows. Inputs are
// raw files written by tests/test_gpu_mirror.py; outputs go back as raw files and the test compares them bit for bit with
// the ctypes binding of the C ABI on a pooled layer of the same weights.
//   mirror_run_dsk <dir> <H> <I> <E> <M> <route scale> <shared 0|1>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "dsk/dsk.h"

#define HIPOK(x)                                                    \
  do {                                                              \
    hipError_t e_ = (x);                                            \
    if (e_ != hipSuccess) die("%s: %s", #x, hipGetErrorString(e_)); \
  } while (0)

static std::vector<char> slurp(const std::string& p) {
  std::vector<char> b;
  FILE* f = std::fopen(p.c_str(), "rb");
  if (!f) die("cannot read %s", p.c_str());
  std::fseek(f, 0, SEEK_END);
  b.resize((size_t)std::ftell(f));
  std::fseek(f, 0, SEEK_SET);
  if (!b.empty() && std::fread(b.data(), 1, b.size(), f) != b.size()) die("short read of %s", p.c_str());
  std::fclose(f);
  return b;
}
template <class T>
static T* upload(const std::vector<char>& b) {
  void* d = nullptr;
  HIPOK(hipMalloc(&d, b.size()));
  HIPOK(hipMemcpy(d, b.data(), b.size(), hipMemcpyHostToDevice));
  return static_cast<T*>(d);
}
template <class T>
static T* dalloc(size_t n, int fill) {
  void* d = nullptr;
  HIPOK(hipMalloc(&d, n));
  HIPOK(hipMemset(d, fill, n));
  return static_cast<T*>(d);
}
static void dump(const std::string& p, const void* d, size_t n) {
  std::vector<char> b(n);
  HIPOK(hipMemcpy(b.data(), d, n, hipMemcpyDeviceToHost));
  FILE* f = std::fopen(p.c_str(), "wb");
  if (!f || std::fwrite(b.data(), 1, n, f) != n) die("cannot write %s", p.c_str());
  std::fclose(f);
}

int main(int argc, char** argv) {
  if (argc != 8) die("usage: mirror_run_dsk dir H I E M scale shared");
  const std::string dir = std::string(argv[1]) + "/";
  const int H = std::atoi(argv[2]), I = std::atoi(argv[3]), E = std::atoi(argv[4]), M = std::atoi(argv[5]);
  const float scale = (float)std::atof(argv[6]);
  const bool shared = std::atoi(argv[7]) != 0;
  hipStream_t st;
  HIPOK(hipStreamCreate(&st));
  dsk::set_shape(H, I, E);

  // load time: every expert's matrices through tile_fp4 into the stacked tensors, the shared expert's through tile_fp8
  const size_t gu = (size_t)I * H, dn = (size_t)H * I;
  dsk::MoeWeights w{};
  uint8_t *w1 = dalloc<uint8_t>(E * gu / 2, 0), *s1 = dalloc<uint8_t>(E * gu / 32, 0), *w3 = dalloc<uint8_t>(E * gu / 2, 0),
          *s3 = dalloc<uint8_t>(E * gu / 32, 0), *w2 = dalloc<uint8_t>(E * dn / 2, 0), *s2 = dalloc<uint8_t>(E * dn / 32, 0);
  const uint8_t *src_w1 = upload<uint8_t>(slurp(dir + "w1.bin")), *src_s1 = upload<uint8_t>(slurp(dir + "s1.bin")),
                *src_w3 = upload<uint8_t>(slurp(dir + "w3.bin")), *src_s3 = upload<uint8_t>(slurp(dir + "s3.bin")),
                *src_w2 = upload<uint8_t>(slurp(dir + "w2.bin")), *src_s2 = upload<uint8_t>(slurp(dir + "s2.bin"));
  for (int e = 0; e < E; ++e) {
    dsk::tile_fp4(src_w1 + e * gu / 2, src_s1 + e * gu / 32, w1 + e * gu / 2, s1 + e * gu / 32, I, H, st);
    dsk::tile_fp4(src_w3 + e * gu / 2, src_s3 + e * gu / 32, w3 + e * gu / 2, s3 + e * gu / 32, I, H, st);
    dsk::tile_fp4(src_w2 + e * dn / 2, src_s2 + e * dn / 32, w2 + e * dn / 2, s2 + e * dn / 32, H, I, st);
  }
  w.w1 = w1, w.s1 = s1, w.w3 = w3, w.s3 = s3, w.w2 = w2, w.s2 = s2;
  if (shared) {
    uint8_t *a = dalloc<uint8_t>(gu, 0), *as = dalloc<uint8_t>(gu / 1024, 0), *b = dalloc<uint8_t>(gu, 0), *bs = dalloc<uint8_t>(gu / 1024, 0),
            *c = dalloc<uint8_t>(dn, 0), *cs = dalloc<uint8_t>(dn / 1024, 0);
    dsk::tile_fp8(upload<uint8_t>(slurp(dir + "sh_w1.bin")), upload<uint8_t>(slurp(dir + "sh_s1.bin")), a, as, I, H, st);
    dsk::tile_fp8(upload<uint8_t>(slurp(dir + "sh_w3.bin")), upload<uint8_t>(slurp(dir + "sh_s3.bin")), b, bs, I, H, st);
    dsk::tile_fp8(upload<uint8_t>(slurp(dir + "sh_w2.bin")), upload<uint8_t>(slurp(dir + "sh_s2.bin")), c, cs, H, I, st);
    w.sh_w1 = a, w.sh_s1 = as, w.sh_w3 = b, w.sh_s3 = bs, w.sh_w2 = c, w.sh_s2 = cs;
  }
  const uint8_t* xq = upload<uint8_t>(slurp(dir + "xq.bin"));
  const uint8_t* xs = upload<uint8_t>(slurp(dir + "xs.bin"));
  const float* logits = upload<float>(slurp(dir + "logits.bin"));
  const float* bias = upload<float>(slurp(dir + "bias.bin"));

  void* ws = dalloc<uint8_t>(dsk::moe_workspace_bytes(), 0);
  int* idx = dalloc<int>((size_t)M * dsk::kTopK * 4, 0xFF);
  float* wts = dalloc<float>((size_t)M * dsk::kTopK * 4, 0xFF);
  int* idx2 = dalloc<int>((size_t)M * dsk::kTopK * 4, 0xFF);
  float* wts2 = dalloc<float>((size_t)M * dsk::kTopK * 4, 0xFF);
  float* y = dalloc<float>((size_t)M * H * 4, 0xFF);
  float* y2 = dalloc<float>((size_t)M * H * 4, 0xFF);
  float* y3 = dalloc<float>((size_t)M * H * 4, 0xFF);

  dsk::router_topk(logits, bias, M, E, idx, wts, scale, st);
  dsk::moe(xq, xs, M, idx, wts, w, ws, y, dsk::MoeCfg{}, st);
  dsk::moe_routed(xq, xs, M, logits, bias, E, scale, w, ws, y2, dsk::MoeCfg{}, st, idx2, wts2);
  void* pws = dalloc<uint8_t>(dsk::moe_prefill_workspace_bytes(M, E), 0);
  dsk::moe_prefill(xq, xs, M, idx, wts, E, w, pws, y3, st);
  float* y4 = dalloc<float>((size_t)M * H * 4, 0xFF);
  dsk::moe_prefill_rows(xq, xs, M, idx, wts, w, ws, y4, st);
  HIPOK(hipStreamSynchronize(st));
  dump(dir + "o_idx.bin", idx, (size_t)M * dsk::kTopK * 4);
  dump(dir + "o_w.bin", wts, (size_t)M * dsk::kTopK * 4);
  dump(dir + "o_idx2.bin", idx2, (size_t)M * dsk::kTopK * 4);
  dump(dir + "o_w2.bin", wts2, (size_t)M * dsk::kTopK * 4);
  dump(dir + "o_y.bin", y, (size_t)M * H * 4);
  dump(dir + "o_y2.bin", y2, (size_t)M * H * 4);
  dump(dir + "o_y3.bin", y3, (size_t)M * H * 4);
  dump(dir + "o_y4.bin", y4, (size_t)M * H * 4);
  std::printf("CHECK mirror_run_dsk ok  ws %zu bytes\n", dsk::moe_workspace_bytes());
  return 0;
}
