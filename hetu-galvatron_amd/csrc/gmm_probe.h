// Timing probes of the grouped-GEMM kernel.  The library is built without GMOE_PROBE: then this
// header defines three false constants and five empty macros and the kernel reads without them.
// A probe build (-DGMOE_PROBE=n, never shipped) selects:
//   1  the main loop without its global loads (stale register pieces are still staged through LDS;
//      results are wrong): what the operand stream into the CU costs under the power limit;
//   2  ... without the LDS staging stores as well;
//   4  every main-loop load fetches K tile 0 again (all loads hit in L2; results are wrong): what the
//      L2 misses cost;
//   8  (results stay right) every workgroup adds the time its tiles spend in the prologue, the main
//      loop and the epilogue to device-side sums that gmoe_probe_read() returns, and leaves its start
//      and end time, the XCD and CU it ran on and its tile count for gmoe_probe_read_wg().
#pragma once

#ifndef GMOE_PROBE
#define GMOE_PROBE 0
#endif

namespace gmoe {
constexpr bool kProbeNoLoads = (GMOE_PROBE & 1) != 0;
constexpr bool kProbeNoStaging = (GMOE_PROBE & 2) != 0;
constexpr bool kProbeLoadsHitL2 = GMOE_PROBE == 4;
}  // namespace gmoe

#if GMOE_PROBE & 8
// prologue, main loop, epilogue (100 MHz ticks of lane 0, summed over workgroups), tiles
__device__ unsigned long long gmoe_phase_ticks[4];
extern "C" int gmoe_probe_read(unsigned long long* out4, int reset) {
  if (hipMemcpyFromSymbol(out4, HIP_SYMBOL(gmoe_phase_ticks), 32) != hipSuccess) return -1;
  if (reset) {
    const unsigned long long z[4] = {0, 0, 0, 0};
    if (hipMemcpyToSymbol(HIP_SYMBOL(gmoe_phase_ticks), z, 32) != hipSuccess) return -1;
  }
  return 0;
}
// per workgroup of the last launch: start, end (100 MHz ticks), XCC_ID << 32 | HW_ID, tiles
__device__ unsigned long long gmoe_wg_ticks[1024 * 4];
extern "C" int gmoe_probe_read_wg(unsigned long long* out) {
  return hipMemcpyFromSymbol(out, HIP_SYMBOL(gmoe_wg_ticks), sizeof(gmoe_wg_ticks)) == hipSuccess ? 0 : -1;
}

#define GMOE_PROBE_WORKGROUP_BEGIN()                                                       \
  const unsigned long long pt_wg0 = wall_clock64();                                         \
  unsigned long long pt_pro = 0, pt_main = 0, pt_epi = 0, pt_tiles = 0, pt_a = 0, pt_1 = 0, pt_2 = 0
#define GMOE_PROBE_TILE_BEGIN()                       \
  do {                                                \
    const unsigned long long now = wall_clock64();    \
    if (pt_tiles) pt_epi += now - pt_2;               \
    pt_a = now;                                       \
    ++pt_tiles;                                       \
  } while (0)
#define GMOE_PROBE_MAIN_LOOP_BEGIN() \
  do {                               \
    pt_1 = wall_clock64();           \
    pt_pro += pt_1 - pt_a;           \
  } while (0)
#define GMOE_PROBE_MAIN_LOOP_END() \
  do {                             \
    pt_2 = wall_clock64();         \
    pt_main += pt_2 - pt_1;        \
  } while (0)
#define GMOE_PROBE_WORKGROUP_END()                                                  \
  do {                                                                              \
    if (threadIdx.x == 0 && pt_tiles) {                                             \
      pt_epi += wall_clock64() - pt_2;                                              \
      atomicAdd(&gmoe_phase_ticks[0], pt_pro);                                      \
      atomicAdd(&gmoe_phase_ticks[1], pt_main);                                     \
      atomicAdd(&gmoe_phase_ticks[2], pt_epi);                                      \
      atomicAdd(&gmoe_phase_ticks[3], pt_tiles);                                    \
    }                                                                               \
    if (threadIdx.x == 0 && blockIdx.x < 1024) {                                    \
      unsigned xcc, hwid;                                                           \
      asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));            \
      asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hwid));            \
      gmoe_wg_ticks[blockIdx.x * 4] = pt_wg0;                                       \
      gmoe_wg_ticks[blockIdx.x * 4 + 1] = wall_clock64();                           \
      gmoe_wg_ticks[blockIdx.x * 4 + 2] = ((unsigned long long)xcc << 32) | hwid;   \
      gmoe_wg_ticks[blockIdx.x * 4 + 3] = pt_tiles;                                 \
    }                                                                               \
  } while (0)
#else
#define GMOE_PROBE_WORKGROUP_BEGIN() (void)0
#define GMOE_PROBE_TILE_BEGIN() (void)0
#define GMOE_PROBE_MAIN_LOOP_BEGIN() (void)0
#define GMOE_PROBE_MAIN_LOOP_END() (void)0
#define GMOE_PROBE_WORKGROUP_END() (void)0
#endif
