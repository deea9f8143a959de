// The router's selection: the gfx950 counterpart of the reference's gx::route (altar1-4xgx10-switchless/engine/experts/
// route.cu:11-33) and dsk::router_topk (ds41f-4xgx10-switchless/engine/kernels/norm_router.cu:24-34).
// One wavefront a row (common.cuh route_row); ids and weight bits equal the CPU routing reference for the sigmoid score.
#include "abi_internal.h"
#include "common.cuh"

namespace dsgx {
namespace {

__global__ void __launch_bounds__(256) k_route(const float* __restrict__ logits, const float* __restrict__ bias, int M, int E, int topk,
                                               float scale, int score_fn, int* __restrict__ idx, float* __restrict__ wout) {
  const int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, lane = threadIdx.x & 63;
  if (row >= M) return;
  int id;
  float w;
  float lg[kRouteRJ], bs[kRouteRJ];
  route_fetch(logits + (size_t)row * E, E, lane, lg);
  route_fetch(bias, E, lane, bs);
  route_row(lg, bs, E, topk, scale, score_fn, lane, id, w);
  if (lane < topk) idx[row * topk + lane] = id, wout[row * topk + lane] = w;
}

}  // namespace
}  // namespace dsgx

using namespace dsgx;

extern "C" int dsgx_route(const float* logits, const float* bias, int M, int E, int topk, float route_scale, int score_fn, int* idx,
                          float* w, void* stream) {
  if (!logits || !idx || !w) return fail(DSGX_EINVAL, "route: null logits, idx or w");
  if (M < 1 || E < 1 || E > DSGX_MAX_EXPERTS || topk < 1 || topk > DSGX_MAX_TOPK || topk > E)
    return fail(DSGX_EINVAL, "route: M %d, E %d (<= %d), top-k %d (<= %d)", M, E, DSGX_MAX_EXPERTS, topk, DSGX_MAX_TOPK);
  if (score_fn != 0 && score_fn != 1) return fail(DSGX_EINVAL, "route: score function %d", score_fn);
  hipLaunchKernelGGL(k_route, dim3((M + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream), logits, bias, M, E, topk, route_scale,
                     score_fn, idx, w);
  DSGX_HIP(hipGetLastError());
  return DSGX_OK;
}
