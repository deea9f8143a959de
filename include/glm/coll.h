// comm::glm:: - the residual add and RMSNorm that end an MoE (or MLP) step, with the reference's names and argument order
// (altar1-4xgx10-switchless/engine/comm/glmcoll.h:34-62). The reference sums the partials of its four ranks before the add;
// this build runs one GPU, so the channel names a world of one and the "all-reduce" is the identity: the arithmetic after
// it (the rounding order, the norm) is the reference's. A channel of more than one rank dies.
#pragma once
#include <cstdint>

#include "../gx/check.h"

namespace comm {
struct DevChannel {
  int world = 1, rank = 0;
};
namespace glm {

// glmcoll.h:55-57: h = bf16(f32(res) + part) -> res_out (may be res); xn = bf16(w * bf16(h * rsqrt(mean(h^2) + eps))).
// round2: h = bf16(res + bf16(part)). R rows of H values (the reference's form has H = 6144 built in: the 11-argument call).
inline void allreduce_add_norm(const DevChannel& ch, const float* part, int R, int H, const uint16_t* res, uint16_t* res_out,
                               const uint16_t* w, float eps, uint16_t* xn, void* st, bool pdl = false, int slices = 0,
                               bool round2 = false) {
  (void)pdl, (void)slices;
  if (ch.world != 1) die("allreduce_add_norm: a world of %d ranks (one GPU here)", ch.world);
  DSGX_DIE_ON(dsgx_add_norm(part, nullptr, R, H, res, res_out, w, eps, xn, round2 ? 1 : 0, st));
}
inline void allreduce_add_norm(const DevChannel& ch, const float* part, int R, const uint16_t* res, uint16_t* res_out,
                               const uint16_t* w, float eps, uint16_t* xn, void* st, bool pdl = false, int slices = 0,
                               bool round2 = false) {
  allreduce_add_norm(ch, part, R, 6144, res, res_out, w, eps, xn, st, pdl, slices, round2);
}
// glmcoll.h:62-64: two partials (yr and ys), y = bf16(bf16(part) + bf16(part2)), h = bf16(res + y), then the norm
inline void allreduce2_add_norm(const DevChannel& ch, const float* part, const float* part2, int R, int H, const uint16_t* res,
                                uint16_t* res_out, const uint16_t* w, float eps, uint16_t* xn, void* st, bool pdl = false,
                                int slices = 0, bool round2 = false) {
  (void)pdl, (void)slices, (void)round2;
  if (ch.world != 1) die("allreduce2_add_norm: a world of %d ranks (one GPU here)", ch.world);
  if (!part2) die("allreduce2_add_norm: the second partial is null");
  DSGX_DIE_ON(dsgx_add_norm(part, part2, R, H, res, res_out, w, eps, xn, 0, st));
}
inline void allreduce2_add_norm(const DevChannel& ch, const float* part, const float* part2, int R, const uint16_t* res,
                                uint16_t* res_out, const uint16_t* w, float eps, uint16_t* xn, void* st, bool pdl = false,
                                int slices = 0, bool round2 = false) {
  allreduce2_add_norm(ch, part, part2, R, 6144, res, res_out, w, eps, xn, st, pdl, slices, round2);
}

}  // namespace glm
}  // namespace comm
