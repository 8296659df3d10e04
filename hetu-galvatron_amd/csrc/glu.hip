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

template <int DT, int ACT, bool VEC>
__global__ __launch_bounds__(256) void glu_fwd_kernel(const unsigned char* y, int64_t N, int64_t F,
                                                      unsigned char* out) {
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
    } else {
      const float a = Elem<DT>::load(y, r * 2 * F + c), b = Elem<DT>::load(y, r * 2 * F + F + c);
      Elem<DT>::store(out, r * F + c, act_fwd<ACT>(a) * b);
    }
  }
}

template <int DT, int ACT, bool VEC>
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
      Vec16<DT>::unpack(ld16_nt(yr + c * 16), a);
      Vec16<DT>::unpack(ld16_nt(yr + F * Elem<DT>::bytes + c * 16), b);
      Vec16<DT>::unpack(ld16_nt(g + (r * F) * Elem<DT>::bytes + c * 16), go);
#pragma unroll
      for (int q = 0; q < NV; ++q) {
        da[q] = go[q] * act_grad<ACT>(a[q]) * b[q];
        db[q] = go[q] * act_fwd<ACT>(a[q]);
      }
      st16_nt(dr + c * 16, Vec16<DT>::pack(da));
      st16_nt(dr + F * Elem<DT>::bytes + c * 16, Vec16<DT>::pack(db));
    } else {
      const float a = Elem<DT>::load(y, r * 2 * F + c), b = Elem<DT>::load(y, r * 2 * F + F + c);
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
                       void* out, hipStream_t st) {
  const int64_t total = N * (F / (vec ? Vec16<DT>::n : 1));
  const dim3 grid(glu_grid(total)), block(256);
  const unsigned char* yy = static_cast<const unsigned char*>(y);
  const unsigned char* gg = static_cast<const unsigned char*>(g);
  unsigned char* oo = static_cast<unsigned char*>(out);
  if (!bwd) {
    if (vec)
      hipLaunchKernelGGL((glu_fwd_kernel<DT, ACT, true>), grid, block, 0, st, yy, N, F, oo);
    else
      hipLaunchKernelGGL((glu_fwd_kernel<DT, ACT, false>), grid, block, 0, st, yy, N, F, oo);
  } else {
    if (vec)
      hipLaunchKernelGGL((glu_bwd_kernel<DT, ACT, true>), grid, block, 0, st, gg, yy, N, F, oo);
    else
      hipLaunchKernelGGL((glu_bwd_kernel<DT, ACT, false>), grid, block, 0, st, gg, yy, N, F, oo);
  }
}

static int glu_dispatch(bool bwd, const void* g, const void* y, int dtype, int64_t N, int64_t F,
                        int act, void* out, void* stream) {
  GMOE_CHECK_ARG(N >= 0 && F >= 1);
  GMOE_CHECK_ARG(act == GMOE_ACT_SILU || act == GMOE_ACT_GELU);
  if (N == 0) return GMOE_OK;
  GMOE_CHECK_ARG(y && out && (!bwd || g));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int es = dtype == GMOE_F32 ? 4 : 2;
  const bool vec = ((F * es) & 15) == 0 && gmoe_aligned(y, 16) && gmoe_aligned(out, 16) &&
                   (!bwd || gmoe_aligned(g, 16));
#define GMOE_GLU_CASE(DT)                                                       \
  case DT:                                                                      \
    if (act == GMOE_ACT_SILU)                                                   \
      launch_glu<DT, GMOE_ACT_SILU>(bwd, vec, g, y, N, F, out, st);             \
    else                                                                        \
      launch_glu<DT, GMOE_ACT_GELU>(bwd, vec, g, y, N, F, out, st);             \
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
