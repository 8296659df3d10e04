// Shared device helpers for the gfx950 MoE kernels (64-wide wavefronts).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/galvatron_moe.h"

#define GMOE_WAVE 64

#define GMOE_CHECK_ARG(cond) \
  do {                       \
    if (!(cond)) return GMOE_ERR_INVALID; \
  } while (0)

static inline int gmoe_launch_status() {
  return hipGetLastError() == hipSuccess ? GMOE_OK : GMOE_ERR_LAUNCH;
}

static inline bool gmoe_aligned(const void* p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

// Host-side facts that do not change while the process runs are asked of the runtime once per
// device, not once per launch.
static inline int gmoe_current_device() {
  int dev = 0;
  return hipGetDevice(&dev) == hipSuccess && dev >= 0 ? dev : 0;
}
// Compute units of the current device (256 when the runtime cannot tell).
static inline int gmoe_cu_count() {
  static std::atomic<int> cached[64];
  const int dev = gmoe_current_device();
  if (dev >= 64) return 256;
  int v = cached[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    int q = 0;
    v = (hipDeviceGetAttribute(&q, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && q > 0) ? q : 256;
    cached[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}
// Runs `f` (returning success) the first time it is reached on each device; `mask` has one bit per
// device.  Two threads may both run it the first time, which is harmless for idempotent set-up.
template <typename F>
static inline bool gmoe_once_per_device(std::atomic<uint64_t>& mask, F&& f) {
  const int dev = gmoe_current_device();
  const uint64_t bit = dev < 64 ? (1ull << dev) : 0ull;
  if (bit && (mask.load(std::memory_order_acquire) & bit)) return true;
  if (!f()) return false;
  if (bit) mask.fetch_or(bit, std::memory_order_release);
  return true;
}

namespace gmoe {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---- 16-bit float <-> fp32 -------------------------------------------------------------------
// Conversions to 16 bits use the hardware converts (v_cvt_pk_bf16_f32, v_cvt_f16_f32): round to
// nearest even, NaN stays NaN.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  _Float16 h = __builtin_bit_cast(_Float16, static_cast<uint16_t>(b));
  return static_cast<float>(h);
}
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  _Float16 h = static_cast<_Float16>(f);
  return __builtin_bit_cast(uint16_t, h);
}

template <int DT>
struct Elem;  // DT = gmoe_dtype
template <>
struct Elem<GMOE_F32> {
  typedef float storage;
  static constexpr int bytes = 4;
  __device__ static __forceinline__ float load(const void* p, int64_t i) {
    return static_cast<const float*>(p)[i];
  }
  __device__ static __forceinline__ void store(void* p, int64_t i, float v) {
    static_cast<float*>(p)[i] = v;
  }
  __device__ static __forceinline__ float round(float v) { return v; }
};
template <>
struct Elem<GMOE_BF16> {
  typedef uint16_t storage;
  static constexpr int bytes = 2;
  __device__ static __forceinline__ float load(const void* p, int64_t i) {
    return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  }
  __device__ static __forceinline__ void store(void* p, int64_t i, float v) {
    static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(f32_to_bf16_bits(v));
  }
  __device__ static __forceinline__ float round(float v) {
    return bf16_bits_to_f32(f32_to_bf16_bits(v));
  }
};
template <>
struct Elem<GMOE_F16> {
  typedef uint16_t storage;
  static constexpr int bytes = 2;
  __device__ static __forceinline__ float load(const void* p, int64_t i) {
    return f16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  }
  __device__ static __forceinline__ void store(void* p, int64_t i, float v) {
    static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(f32_to_f16_bits(v));
  }
  __device__ static __forceinline__ float round(float v) {
    return f16_bits_to_f32(f32_to_f16_bits(v));
  }
};

// Unpack / pack a 16-byte vector of DT elements to / from fp32 lanes.
template <int DT>
struct Vec16;
template <>
struct Vec16<GMOE_F32> {
  static constexpr int n = 4;
  __device__ static __forceinline__ void unpack(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
  }
  __device__ static __forceinline__ u32x4 pack(const float* f) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(f[i]);
    return v;
  }
};
template <>
struct Vec16<GMOE_BF16> {
  static constexpr int n = 8;
  __device__ static __forceinline__ void unpack(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(v[i] << 16);
      f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float* f) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      v[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
    return v;
  }
};
template <>
struct Vec16<GMOE_F16> {
  static constexpr int n = 8;
  __device__ static __forceinline__ void unpack(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = f16_bits_to_f32(v[i] & 0xffffu);
      f[2 * i + 1] = f16_bits_to_f32(v[i] >> 16);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float* f) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      v[i] = pack_f16x2(f[2 * i], f[2 * i + 1]);
    return v;
  }
};

// ---- gated-activation math, shared by the activation kernels and the GEMM epilogues so that both
// give the same bits.  The logistic function uses the hardware exp2 and reciprocal (1 ulp each:
// relative error ~1e-6, far below the 16-bit storage and the fp32 test tolerance of 1e-4): a quarter
// of the instructions of expf and an IEEE division, which matters where the activation runs inside
// a GEMM epilogue with the matrix cores waiting.
__device__ __forceinline__ float logistic(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
// gelu = false: SiLU (x * logistic(x)); true: the exact (erf) GELU that F.gelu uses
__device__ __forceinline__ float glu_act(float x, bool gelu) {
  if (!gelu) return x * logistic(x);
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
}
// d act(x) / dx
__device__ __forceinline__ float glu_act_grad(float x, bool gelu) {
  if (!gelu) {
    const float s = logistic(x);
    return s * (1.0f + x * (1.0f - s));
  }
  return 0.5f * (1.0f + erff(x * 0.70710678118654752f)) + x * 0.3989422804014327f * expf(-0.5f * x * x);
}

// ---- wavefront helpers -----------------------------------------------------------------------
__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// DPP row operations (rows are 16 lanes).  quad_perm [1,0,3,2] / [2,3,0,1] exchange lanes at
// distance 1 / 2; row_half_mirror / row_mirror reverse 8 / 16 lanes, which exchanges quads /
// half-rows once the values inside them already agree.
#define GMOE_DPP_XOR1 0xB1
#define GMOE_DPP_XOR2 0x4E
#define GMOE_DPP_HALF_MIRROR 0x141
#define GMOE_DPP_MIRROR 0x140

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __uint_as_float(dpp_u32<CTRL>(__float_as_uint(v)));
}
template <int CTRL>
__device__ __forceinline__ uint64_t dpp_u64(uint64_t v) {
  uint32_t lo = dpp_u32<CTRL>(static_cast<uint32_t>(v));
  uint32_t hi = dpp_u32<CTRL>(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int m) {
  uint32_t lo = __shfl_xor(static_cast<int>(static_cast<uint32_t>(v)), m);
  uint32_t hi = __shfl_xor(static_cast<int>(static_cast<uint32_t>(v >> 32)), m);
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// All-reduce over aligned groups of G consecutive lanes (G a power of two <= 64).
template <int G>
__device__ __forceinline__ uint64_t group_max_u64(uint64_t v) {
  if (G >= 2) { uint64_t o = dpp_u64<GMOE_DPP_XOR1>(v); v = o > v ? o : v; }
  if (G >= 4) { uint64_t o = dpp_u64<GMOE_DPP_XOR2>(v); v = o > v ? o : v; }
  if (G >= 8) { uint64_t o = dpp_u64<GMOE_DPP_HALF_MIRROR>(v); v = o > v ? o : v; }
  if (G >= 16) { uint64_t o = dpp_u64<GMOE_DPP_MIRROR>(v); v = o > v ? o : v; }
  if (G >= 32) { uint64_t o = shfl_xor_u64(v, 16); v = o > v ? o : v; }
  if (G >= 64) { uint64_t o = shfl_xor_u64(v, 32); v = o > v ? o : v; }
  return v;
}
template <int G>
__device__ __forceinline__ float group_max_f32(float v) {
  if (G >= 2) v = fmaxf(v, dpp_f32<GMOE_DPP_XOR1>(v));
  if (G >= 4) v = fmaxf(v, dpp_f32<GMOE_DPP_XOR2>(v));
  if (G >= 8) v = fmaxf(v, dpp_f32<GMOE_DPP_HALF_MIRROR>(v));
  if (G >= 16) v = fmaxf(v, dpp_f32<GMOE_DPP_MIRROR>(v));
  if (G >= 32) v = fmaxf(v, __shfl_xor(v, 16));
  if (G >= 64) v = fmaxf(v, __shfl_xor(v, 32));
  return v;
}
// Sum all-reduce.  The order of the additions is the same in every lane of the group (each step
// adds the partner's partial), so all lanes end with bit-identical results.
template <int G>
__device__ __forceinline__ float group_sum_f32(float v) {
  if (G >= 2) v += dpp_f32<GMOE_DPP_XOR1>(v);
  if (G >= 4) v += dpp_f32<GMOE_DPP_XOR2>(v);
  if (G >= 8) v += dpp_f32<GMOE_DPP_HALF_MIRROR>(v);
  if (G >= 16) v += dpp_f32<GMOE_DPP_MIRROR>(v);
  if (G >= 32) v += __shfl_xor(v, 16);
  if (G >= 64) v += __shfl_xor(v, 32);
  return v;
}
__device__ __forceinline__ float wave_sum_f32(float v) { return group_sum_f32<64>(v); }

// 16-byte global accesses.
__device__ __forceinline__ u32x4 ld16(const void* p) { return *static_cast<const u32x4*>(p); }
__device__ __forceinline__ void st16(void* p, const u32x4& v) { *static_cast<u32x4*>(p) = v; }
// Streaming variants for data that is touched once: keep it from displacing reusable lines.
__device__ __forceinline__ u32x4 ld16_nt(const void* p) {
  return __builtin_nontemporal_load(static_cast<const u32x4*>(p));
}
__device__ __forceinline__ void st16_nt(void* p, const u32x4& v) {
  __builtin_nontemporal_store(v, static_cast<u32x4*>(p));
}

// Defined in norm.hip: out[c] = sum over `parts` rows of the fp32 matrix partial[parts][cols], in
// row order within fixed slices (deterministic), rounded to `dtype`; cols a multiple of 4.
void sum_partial_rows(const float* partial, int parts, int64_t cols, void* out, int dtype,
                      hipStream_t st);

}  // namespace gmoe
