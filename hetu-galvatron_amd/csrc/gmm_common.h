// Shared pieces of the grouped-GEMM kernels: MFMA wrappers, parameters, tile order.
#pragma once

#include <type_traits>

#include "gmoe_common.h"

namespace gmoe {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

enum { MODE_NN = 0, MODE_NT = 1, MODE_TN = 2 };

constexpr int kGemmThreads = 256;
constexpr int kRowPad = 144;    // bytes per LDS row: 128 data + 16 pad
constexpr int kStripTiles = 8;  // column tiles per strip
constexpr int kMaxGroupsLds = 1024;
constexpr uint32_t kOob = 0x80000000u;  // a buffer offset beyond any resource: reads as zero

#define GMOE_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// Compile-time loop: f(std::integral_constant<int, I>) for I in [B, E).
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

template <int DT>
struct Mma;
template <>
struct Mma<GMOE_BF16> {
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, f32x16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b),
                                                  __builtin_bit_cast(bf16x8, a), acc, 0, 0, 0);
  }
};
template <>
struct Mma<GMOE_F16> {
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, f32x16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b),
                                                 __builtin_bit_cast(f16x8, a), acc, 0, 0, 0);
  }
};
template <>
struct Mma<GMOE_F32> {
  // A lane's 16 bytes are 4 consecutive reduction elements; MFMA q pairs element q of the two
  // lane halves, so 4 MFMAs of depth 2 consume the 8 elements one fragment load covers.
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, f32x16& acc) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(b[q]), __uint_as_float(a[q]), acc,
                                                 0, 0, 0);
  }
};

struct GmmParams {
  const unsigned char* a;
  const unsigned char* b;
  unsigned char* c;
  const long long* offsets;  // [E+1]
  int E;
  int64_t N, K, M;
};

// Position q inside an expert's mt_cnt x nt_cnt tile grid, walked in strips of kStripTiles columns.
__device__ __forceinline__ void strip_order(int64_t q, int mt_cnt, int nt_cnt, int& mt, int& nt) {
  const int64_t per_strip = (int64_t)mt_cnt * kStripTiles;
  const int strip = (int)(q / per_strip);
  const int rem = (int)(q - strip * per_strip);
  const int n0 = strip * kStripTiles;
  const int width = (nt_cnt - n0) < kStripTiles ? (nt_cnt - n0) : kStripTiles;
  mt = rem / width;
  nt = n0 + rem % width;
}


// Launches the LDS-DMA variant (gmm_dtl.hip) for 16-bit operands with large groups.
int launch_gmm_dtl(const GmmParams& p, int mode, int dtype, int out_dtype, hipStream_t st);

}  // namespace gmoe
