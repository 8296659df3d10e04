// Gated activation of the expert MLP for gfx950: out = act(y[:, :F]) * y[:, F:] and its backward,
// fp32 math on 16-byte vectors.  Follows the `glu` closure (moe/mlp.py:52-57) and swiglu /
// swiglu_back (transformer/fused_kernels.py:142-162); GELU is the exact (erf) form F.gelu uses.
#include "gmoe_common.h"

namespace gmoe {

template <int ACT>
__device__ __forceinline__ float act_fwd(float x) {
  return glu_act(x, ACT == GMOE_ACT_GELU);
}
template <int ACT>
__device__ __forceinline__ float act_grad(float x) {
  return glu_act_grad(x, ACT == GMOE_ACT_GELU);
}

// ---- the activation input kept as fp8 (e4m3fn) for the backward --------------------------------
// `input.to(torch.float8_e4m3fn)` (transformer/fused_kernels.py:175, 193): round to nearest even
// on 3 mantissa bits; what rounds beyond 448 (|x| > 464) and NaN become the NaN code 0x7f, the
// sign bit is kept.  The hardware conversion does the rounding of the values clamped to +-448.
__device__ __forceinline__ uint32_t e4m3fn_fix(uint32_t code, float x) {
  const uint32_t sign = (__float_as_uint(x) >> 24) & 0x80u;
  const uint32_t mag = !(fabsf(x) <= 464.f) ? 0x7fu : (code & 0x7fu);
  return sign | mag;
}
// two values -> two bytes (low 16 bits)
__device__ __forceinline__ uint32_t e4m3fn_pair(float a, float b) {
  const float ca = fminf(fmaxf(a, -448.f), 448.f), cb = fminf(fmaxf(b, -448.f), 448.f);
  const uint32_t w = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, 0, false);
  return e4m3fn_fix(w & 0xffu, a) | (e4m3fn_fix((w >> 8) & 0xffu, b) << 8);
}
__device__ __forceinline__ float e4m3fn_to_f32(uint32_t byte) {
  const float v = __builtin_amdgcn_cvt_f32_fp8((int)byte, 0);
  return (byte & 0x7fu) == 0x7fu ? __uint_as_float(0x7fc00000u | ((byte & 0x80u) << 24)) : v;
}
// NV values -> NV bytes at dst (NV = 4 or 8)
template <int NV>
__device__ __forceinline__ void store_e4m3fn(unsigned char* dst, const float (&v)[NV]) {
  uint32_t w[(NV + 3) / 4];
#pragma unroll
  for (int q = 0; q < NV / 4; ++q)
    w[q] = e4m3fn_pair(v[4 * q], v[4 * q + 1]) | (e4m3fn_pair(v[4 * q + 2], v[4 * q + 3]) << 16);
  if (NV == 8)
    *reinterpret_cast<u32x2*>(dst) = u32x2{w[0], w[(NV + 3) / 4 - 1]};
  else
    *reinterpret_cast<uint32_t*>(dst) = w[0];
}
template <int NV>
__device__ __forceinline__ void load_e4m3fn(const unsigned char* src, float (&v)[NV]) {
  uint32_t w[(NV + 3) / 4];
  if (NV == 8) {
    const u32x2 t = *reinterpret_cast<const u32x2*>(src);
    w[0] = t[0];
    w[(NV + 3) / 4 - 1] = t[1];
  } else {
    w[0] = *reinterpret_cast<const uint32_t*>(src);
  }
#pragma unroll
  for (int q = 0; q < NV; ++q) v[q] = e4m3fn_to_f32((w[q / 4] >> (8 * (q & 3))) & 0xffu);
}

// y8 (optional): y as e4m3fn, [N,2F] bytes
template <int DT, int ACT, bool VEC>
__global__ __launch_bounds__(256) void glu_fwd_kernel(const unsigned char* y, int64_t N, int64_t F,
                                                      unsigned char* out, unsigned char* y8) {
  constexpr int NV = VEC ? Vec16<DT>::n : 1;
  const int64_t per_row = F / NV;
  const int64_t total = N * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / per_row, c = i % per_row;
    if (VEC) {
      const unsigned char* yr = y + r * (2 * F) * Elem<DT>::bytes;
      float a[NV], b[NV], o[NV];
      Vec16<DT>::unpack(ld16_nt(yr + c * 16), a);
      Vec16<DT>::unpack(ld16_nt(yr + F * Elem<DT>::bytes + c * 16), b);
#pragma unroll
      for (int q = 0; q < NV; ++q) o[q] = act_fwd<ACT>(a[q]) * b[q];
      st16_nt(out + (r * F) * Elem<DT>::bytes + c * 16, Vec16<DT>::pack(o));
      if (y8) {
        store_e4m3fn<NV>(y8 + r * 2 * F + c * NV, a);
        store_e4m3fn<NV>(y8 + r * 2 * F + F + c * NV, b);
      }
    } else {
      const float a = Elem<DT>::load(y, r * 2 * F + c), b = Elem<DT>::load(y, r * 2 * F + F + c);
      Elem<DT>::store(out, r * F + c, act_fwd<ACT>(a) * b);
      if (y8) {
        y8[r * 2 * F + c] = (unsigned char)(e4m3fn_pair(a, a) & 0xffu);
        y8[r * 2 * F + F + c] = (unsigned char)(e4m3fn_pair(b, b) & 0xffu);
      }
    }
  }
}

// IN8: y holds e4m3fn bytes (what the forward stored); they widen exactly to any dtype here
template <int DT, int ACT, bool VEC, bool IN8>
__global__ __launch_bounds__(256) void glu_bwd_kernel(const unsigned char* g, const unsigned char* y,
                                                      int64_t N, int64_t F, unsigned char* dy) {
  constexpr int NV = VEC ? Vec16<DT>::n : 1;
  const int64_t per_row = F / NV;
  const int64_t total = N * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / per_row, c = i % per_row;
    if (VEC) {
      const unsigned char* yr = y + r * (2 * F) * Elem<DT>::bytes;
      unsigned char* dr = dy + r * (2 * F) * Elem<DT>::bytes;
      float a[NV], b[NV], go[NV], da[NV], db[NV];
      if constexpr (IN8) {
        load_e4m3fn<NV>(y + r * 2 * F + c * NV, a);
        load_e4m3fn<NV>(y + r * 2 * F + F + c * NV, b);
      } else {
        Vec16<DT>::unpack(ld16_nt(yr + c * 16), a);
        Vec16<DT>::unpack(ld16_nt(yr + F * Elem<DT>::bytes + c * 16), b);
      }
      Vec16<DT>::unpack(ld16_nt(g + (r * F) * Elem<DT>::bytes + c * 16), go);
#pragma unroll
      for (int q = 0; q < NV; ++q) {
        da[q] = go[q] * act_grad<ACT>(a[q]) * b[q];
        db[q] = go[q] * act_fwd<ACT>(a[q]);
      }
      st16_nt(dr + c * 16, Vec16<DT>::pack(da));
      st16_nt(dr + F * Elem<DT>::bytes + c * 16, Vec16<DT>::pack(db));
    } else {
      const float a = IN8 ? e4m3fn_to_f32(y[r * 2 * F + c]) : Elem<DT>::load(y, r * 2 * F + c);
      const float b = IN8 ? e4m3fn_to_f32(y[r * 2 * F + F + c]) : Elem<DT>::load(y, r * 2 * F + F + c);
      const float go = Elem<DT>::load(g, r * F + c);
      Elem<DT>::store(dy, r * 2 * F + c, go * act_grad<ACT>(a) * b);
      Elem<DT>::store(dy, r * 2 * F + F + c, go * act_fwd<ACT>(a));
    }
  }
}

static inline unsigned glu_grid(int64_t total) {
  int64_t b = (total + 255) / 256;
  const int64_t cap = 256 * 64;  // a few waves of blocks per CU, grid-stride beyond that
  return (unsigned)(b < 1 ? 1 : (b > cap ? cap : b));
}

template <int DT, int ACT>
static void launch_glu(bool bwd, bool vec, const void* g, const void* y, int64_t N, int64_t F,
                       void* out, void* y8, bool in8, hipStream_t st) {
  const int64_t total = N * (F / (vec ? Vec16<DT>::n : 1));
  const dim3 grid(glu_grid(total)), block(256);
  const unsigned char* yy = static_cast<const unsigned char*>(y);
  const unsigned char* gg = static_cast<const unsigned char*>(g);
  unsigned char* oo = static_cast<unsigned char*>(out);
  if (!bwd) {
    unsigned char* y8p = static_cast<unsigned char*>(y8);
    if (vec)
      hipLaunchKernelGGL((glu_fwd_kernel<DT, ACT, true>), grid, block, 0, st, yy, N, F, oo, y8p);
    else
      hipLaunchKernelGGL((glu_fwd_kernel<DT, ACT, false>), grid, block, 0, st, yy, N, F, oo, y8p);
  } else {
    auto kern = in8 ? (vec ? glu_bwd_kernel<DT, ACT, true, true> : glu_bwd_kernel<DT, ACT, false, true>)
                    : (vec ? glu_bwd_kernel<DT, ACT, true, false> : glu_bwd_kernel<DT, ACT, false, false>);
    hipLaunchKernelGGL(kern, grid, block, 0, st, gg, yy, N, F, oo);
  }
}

static int glu_dispatch(bool bwd, const void* g, const void* y, int dtype, int64_t N, int64_t F,
                        int act, void* out, void* stream, void* y8 = nullptr, bool in8 = false) {
  GMOE_CHECK_ARG(N >= 0 && F >= 1);
  GMOE_CHECK_ARG(act == GMOE_ACT_SILU || act == GMOE_ACT_GELU);
  if (N == 0) return GMOE_OK;
  GMOE_CHECK_ARG(y && out && (!bwd || g));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int es = dtype == GMOE_F32 ? 4 : 2;
  // 16-byte pieces of the dtype's tensors; the fp8 tensor then moves in 4- or 8-byte pieces
  const bool vec = ((F * es) & 15) == 0 && gmoe_aligned(y, in8 ? 8 : 16) && gmoe_aligned(out, 16) &&
                   (!bwd || gmoe_aligned(g, 16)) && gmoe_aligned(y8, 8);
#define GMOE_GLU_CASE(DT)                                                       \
  case DT:                                                                      \
    if (act == GMOE_ACT_SILU)                                                   \
      launch_glu<DT, GMOE_ACT_SILU>(bwd, vec, g, y, N, F, out, y8, in8, st);             \
    else                                                                        \
      launch_glu<DT, GMOE_ACT_GELU>(bwd, vec, g, y, N, F, out, y8, in8, st);             \
    break;
  switch (dtype) {
    GMOE_GLU_CASE(GMOE_F32)
    GMOE_GLU_CASE(GMOE_BF16)
    GMOE_GLU_CASE(GMOE_F16)
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
#undef GMOE_GLU_CASE
  return gmoe_launch_status();
}

}  // namespace gmoe

extern "C" int gmoe_glu_fwd(const void* y, int dtype, int64_t N, int64_t F, int act, void* out,
                            void* stream) {
  return gmoe::glu_dispatch(false, nullptr, y, dtype, N, F, act, out, stream);
}

extern "C" int gmoe_glu_bwd(const void* grad_out, const void* y, int dtype, int64_t N, int64_t F,
                            int act, void* grad_y, void* stream) {
  return gmoe::glu_dispatch(true, grad_out, y, dtype, N, F, act, grad_y, stream);
}

extern "C" int gmoe_glu_fwd_fp8store(const void* y, int dtype, int64_t N, int64_t F, int act, void* out,
                                     void* y_fp8, void* stream) {
  GMOE_CHECK_ARG(y_fp8 != nullptr || N == 0);
  return gmoe::glu_dispatch(false, nullptr, y, dtype, N, F, act, out, stream, y_fp8, false);
}

extern "C" int gmoe_glu_bwd_fp8in(const void* grad_out, const void* y_fp8, int dtype, int64_t N,
                                  int64_t F, int act, void* grad_y, void* stream) {
  return gmoe::glu_dispatch(true, grad_out, y_fp8, dtype, N, F, act, grad_y, stream, nullptr, true);
}
