// Pieces shared by the router kernels (route.hip) and the loss / bookkeeping kernels (losses.hip):
// the lane-group decomposition of a token's experts and the score helpers.
#pragma once

#include "gmoe_common.h"

namespace gmoe {

constexpr int kVpt = 8;            // experts per lane
constexpr int kRouteThreads = 256;  // 4 wavefronts
constexpr int kRouteMaxBlocks = 512;

// Order-preserving map fp32 -> u32 with NaN above +inf and -0 == +0.
__device__ __forceinline__ uint32_t score_key(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // NaN
  if (u == 0x80000000u) u = 0;                              // -0 -> +0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_score(uint32_t k) {
  if (k == 0xffffffffu) return __uint_as_float(0x7fc00000u);
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}
__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

static inline int route_group_lanes(int E, int num_groups) {
  int need = (E + kVpt - 1) / kVpt;
  if (num_groups > need) need = num_groups;  // lane s also holds the score of routing group s
  int G = 1;
  while (G < need) G <<= 1;
  return G;
}

// One wavefront per statistic: lane l adds the partials of workgroups l, l + 64, ... in order, then
// the 64 lane sums meet in a fixed butterfly, so the result depends only on the launch's grid.  (One
// thread per statistic walking all workgroups took 63 us at 64 experts: 2048 dependent loads.)
static __global__ __launch_bounds__(GMOE_WAVE) void route_stats_reduce_kernel(const float* ws, int nblocks,
                                                                       int E, float* stats) {
  const int e = blockIdx.x;
  float a = 0.f;
  for (int b = threadIdx.x; b < nblocks; b += GMOE_WAVE) a += ws[(int64_t)b * (E + 1) + e];
  a = wave_sum_f32(a);
  if (threadIdx.x == 0) stats[e] = a;
}

// Workgroups of a kernel that walks T tokens with G lanes per token.
static int route_grid(int64_t T, int G) {
  const int tpb = (GMOE_WAVE / G) * (kRouteThreads / GMOE_WAVE);
  int64_t tiles = (T + tpb - 1) / tpb;
  if (tiles < 1) tiles = 1;
  return (int)(tiles < kRouteMaxBlocks ? tiles : kRouteMaxBlocks);
}

}  // namespace gmoe
