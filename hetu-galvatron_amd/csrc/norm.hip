// RMS normalisation in front of the router for gfx950 (HBM-bound): y = x * rstd * w with
// rstd = 1 / sqrt(mean(x^2) + eps), fp32 math, one rounding to the storage type.  Stands in for
// the RMSNorm that GalvatronNorm builds (transformer/norm.py:20-26) and GalvatronMoEAttention
// applies as pre_router_norm (models/moe_modules.py:24-30).
//
// Layout of the work: a workgroup of 256 lanes takes R rows at a time; a lane owns the same NV
// 16-byte column vectors in every row (vector index tid + 256 j), so the weight stays in registers
// and, in the backward, the weight gradient accumulates per lane without any exchange.  The R row
// sums are reduced inside each wavefront and combined across the four wavefronts through a
// double-buffered LDS slot: one barrier per R rows.  R * NV = 8 in the forward (8 vector loads in
// flight per lane); the backward takes R * NV = 4 for 16-bit types (8 to 12 loads in flight).  Workgroups walk the row groups with a grid stride; the
// backward leaves one partial weight gradient per workgroup, summed in a fixed order by a second
// kernel (deterministic for a given T and H).
#include <type_traits>

#include "gmoe_common.h"

namespace gmoe {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / GMOE_WAVE;
constexpr int kNormMaxParts = 512;   // upper bound of the backward grid = rows of the workspace

// Sums of R per-lane values over the workgroup; `slot` holds kNormWaves * R floats and must not be
// the slot the previous call used.
template <int R>
__device__ __forceinline__ void block_sums(float (&v)[R], float* slot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int r = 0; r < R; ++r) v[r] = wave_sum_f32(v[r]);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) slot[wave * R + r] = v[r];
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float s = slot[r];
#pragma unroll
    for (int w = 1; w < kNormWaves; ++w) s += slot[w * R + r];
    v[r] = s;
  }
}

template <int DT, int NV, int R>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_fwd_kernel(
    const unsigned char* __restrict__ x, const unsigned char* __restrict__ w, int64_t T, int H,
    float eps, unsigned char* __restrict__ y, float* __restrict__ rstd) {
  constexpr int EPV = Vec16<DT>::n;
  __shared__ float slots[2][kNormWaves * R];
  const int tid = threadIdx.x;
  const int nvec = H / EPV;
  const int64_t row_bytes = (int64_t)H * Elem<DT>::bytes;
  const float inv_h = 1.0f / (float)H;

  float wf[NV][EPV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = tid + kNormThreads * j;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (c < nvec) v = ld16(w + (int64_t)c * 16);
    Vec16<DT>::unpack(v, wf[j]);
  }

  const int64_t groups = (T + R - 1) / R;
  int parity = 0;
  for (int64_t g = blockIdx.x; g < groups; g += gridDim.x, parity ^= 1) {
    const int64_t r0 = g * R;
    u32x4 xv[R][NV];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = tid + kNormThreads * j;
        xv[r][j] = u32x4{0u, 0u, 0u, 0u};
        if (r0 + r < T && c < nvec) xv[r][j] = ld16_nt(x + (r0 + r) * row_bytes + (int64_t)c * 16);
      }
    float ss[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      ss[r] = 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        float f[EPV];
        Vec16<DT>::unpack(xv[r][j], f);
#pragma unroll
        for (int q = 0; q < EPV; ++q) ss[r] = fmaf(f[q], f[q], ss[r]);
      }
    }
    block_sums<R>(ss, slots[parity]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r0 + r >= T) continue;
      const float rs = 1.0f / sqrtf(ss[r] * inv_h + eps);
      if (tid == 0) rstd[r0 + r] = rs;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = tid + kNormThreads * j;
        if (c >= nvec) continue;
        float f[EPV];
        Vec16<DT>::unpack(xv[r][j], f);
#pragma unroll
        for (int q = 0; q < EPV; ++q) f[q] = (f[q] * rs) * wf[j][q];
        st16(y + (r0 + r) * row_bytes + (int64_t)c * 16, Vec16<DT>::pack(f));
      }
    }
  }
}

// dx = rstd * (dy*w - xhat * mean(dy*w*xhat)) (+ dres), xhat = x * rstd; partial[blockIdx.x][:] =
// sum over this workgroup's rows of dy * xhat.
template <int DT, int NV, int R>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_bwd_kernel(
    const unsigned char* __restrict__ dy, const unsigned char* __restrict__ x,
    const unsigned char* __restrict__ w, const float* __restrict__ rstd,
    const unsigned char* __restrict__ dres, int64_t T, int H, unsigned char* __restrict__ dx,
    float* __restrict__ partial) {
  constexpr int EPV = Vec16<DT>::n;
  __shared__ float slots[2][kNormWaves * R];
  const int tid = threadIdx.x;
  const int nvec = H / EPV;
  const int64_t row_bytes = (int64_t)H * Elem<DT>::bytes;
  const float inv_h = 1.0f / (float)H;

  float wf[NV][EPV], dw[NV][EPV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = tid + kNormThreads * j;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (c < nvec) v = ld16(w + (int64_t)c * 16);
    Vec16<DT>::unpack(v, wf[j]);
#pragma unroll
    for (int q = 0; q < EPV; ++q) dw[j][q] = 0.f;
  }

  const int64_t groups = (T + R - 1) / R;
  int parity = 0;
  for (int64_t g = blockIdx.x; g < groups; g += gridDim.x, parity ^= 1) {
    const int64_t r0 = g * R;
    // the residual branch's gradient is requested with the other two rows, not after the row sums
    u32x4 xv[R][NV], gv[R][NV], dv[R][NV];
    float rs[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const bool row = r0 + r < T;
      rs[r] = row ? rstd[r0 + r] : 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = tid + kNormThreads * j;
        xv[r][j] = u32x4{0u, 0u, 0u, 0u};
        gv[r][j] = u32x4{0u, 0u, 0u, 0u};
        if (row && c < nvec) {
          xv[r][j] = ld16_nt(x + (r0 + r) * row_bytes + (int64_t)c * 16);
          gv[r][j] = ld16_nt(dy + (r0 + r) * row_bytes + (int64_t)c * 16);
          if (dres != nullptr) dv[r][j] = ld16_nt(dres + (r0 + r) * row_bytes + (int64_t)c * 16);
        }
      }
    }
    float c1[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      c1[r] = 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        float xf[EPV], gf[EPV];
        Vec16<DT>::unpack(xv[r][j], xf);
        Vec16<DT>::unpack(gv[r][j], gf);
#pragma unroll
        for (int q = 0; q < EPV; ++q) {
          const float xh = xf[q] * rs[r];
          c1[r] = fmaf(xh, gf[q] * wf[j][q], c1[r]);
          dw[j][q] = fmaf(gf[q], xh, dw[j][q]);
        }
        // keep the unpacked values of one vector at a time: without the fence the scheduler
        // unpacks every row first and the kernel loses half its occupancy to registers
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    block_sums<R>(c1, slots[parity]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r0 + r >= T) continue;
      const float m = c1[r] * inv_h;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = tid + kNormThreads * j;
        if (c >= nvec) continue;
        float xf[EPV], gf[EPV];
        Vec16<DT>::unpack(xv[r][j], xf);
        Vec16<DT>::unpack(gv[r][j], gf);
#pragma unroll
        for (int q = 0; q < EPV; ++q) {
          const float xh = xf[q] * rs[r];
          // one fused multiply-add, written out: the compiler may otherwise contract this
          // expression differently in the two versions of the loop it makes for dres
          xf[q] = fmaf(-xh, m, gf[q] * wf[j][q]) * rs[r];
        }
        if (dres != nullptr) {
          // dx + dres with the two roundings of a separate add kernel
          float rf[EPV];
          Vec16<DT>::unpack(dv[r][j], rf);
          // (an addition of its own: for fp32 nothing else keeps it from contracting with the
          // product above into one fused operation with a single rounding)
#pragma unroll
          for (int q = 0; q < EPV; ++q) {
            float v = Elem<DT>::round(xf[q]);
            asm volatile("" : "+v"(v));
            xf[q] = v + rf[q];
          }
        }
        st16(dx + (r0 + r) * row_bytes + (int64_t)c * 16, Vec16<DT>::pack(xf));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  float* mine = partial + (int64_t)blockIdx.x * H;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = tid + kNormThreads * j;
    if (c >= nvec) continue;
#pragma unroll
    for (int q = 0; q < EPV; q += 4) {
      const f32x4 v = {dw[j][q], dw[j][q + 1], dw[j][q + 2], dw[j][q + 3]};
      *reinterpret_cast<f32x4*>(mine + (int64_t)c * EPV + q) = v;
    }
  }
}

// dweight[h] = sum over the `parts` partial rows, in a fixed order.  A workgroup owns 64 columns:
// 16 lanes x 4 columns read one 256-byte piece of a row, the 64 groups of 16 lanes take every
// 64th row and meet in LDS.
constexpr int kDwThreads = 1024;
constexpr int kDwCols = 64;
template <int DT>
__global__ __launch_bounds__(kDwThreads) void rmsnorm_dw_kernel(const float* __restrict__ partial,
                                                                 int parts, int H,
                                                                 unsigned char* __restrict__ dweight) {
  constexpr int SLICES = kDwThreads / 16;
  __shared__ f32x4 acc[SLICES][16];
  const int sub = threadIdx.x & 15, slice = threadIdx.x >> 4;
  const int col = blockIdx.x * kDwCols + sub * 4;
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  if (col < H)
    for (int p = slice; p < parts; p += SLICES)
      s += *reinterpret_cast<const f32x4*>(partial + (int64_t)p * H + col);
  acc[slice][sub] = s;
  __syncthreads();
  // the first 64 lanes sum one column each over the slices
  if (threadIdx.x < kDwCols) {
    const int c = blockIdx.x * kDwCols + threadIdx.x;
    if (c < H) {
      float t = 0.f;
      for (int k = 0; k < SLICES; ++k) t += reinterpret_cast<const float*>(&acc[k][0])[threadIdx.x];
      Elem<DT>::store(dweight, c, t);
    }
  }
}

// out[c] = sum over the `parts` rows of partial[., c] (cols a multiple of 4), rounded to `dtype`.
void sum_partial_rows(const float* partial, int parts, int64_t cols, void* out, int dtype,
                      hipStream_t st) {
  const unsigned grid = (unsigned)((cols + kDwCols - 1) / kDwCols);
  unsigned char* o = static_cast<unsigned char*>(out);
  if (dtype == GMOE_F32)
    hipLaunchKernelGGL((rmsnorm_dw_kernel<GMOE_F32>), dim3(grid), dim3(kDwThreads), 0, st, partial, parts, (int)cols, o);
  else if (dtype == GMOE_BF16)
    hipLaunchKernelGGL((rmsnorm_dw_kernel<GMOE_BF16>), dim3(grid), dim3(kDwThreads), 0, st, partial, parts, (int)cols, o);
  else
    hipLaunchKernelGGL((rmsnorm_dw_kernel<GMOE_F16>), dim3(grid), dim3(kDwThreads), 0, st, partial, parts, (int)cols, o);
}

// Rows per step of the backward kernel: R * NV = 8 for fp32, 4 for the 16-bit types, whose 8
// elements per vector double the live registers (beyond 256 a CU holds one workgroup, not two).
static constexpr int norm_bwd_rows(int nv, int dtype) {
  const int r = (dtype == GMOE_F32 ? 8 : 4) / nv;
  return r < 1 ? 1 : r;
}

static int norm_parts(int64_t T, int R) {
  const int64_t groups = (T + R - 1) / R;
  return (int)(groups < kNormMaxParts ? groups : kNormMaxParts);
}

// NV = vectors per lane (power of two covering H), R = 8 / NV rows per step.
static int norm_nv(int64_t H, int dtype) {
  const int epv = dtype == GMOE_F32 ? 4 : 8;
  const int64_t nvec = H / epv;
  for (int nv = 1; nv <= 8; nv *= 2)
    if (nvec <= (int64_t)kNormThreads * nv) return nv;
  return 0;
}

template <int DT, int NV>
static void launch_fwd(const void* x, const void* w, int64_t T, int H, float eps, void* y, float* rstd,
                       hipStream_t st) {
  constexpr int R = 8 / NV;
  const int64_t groups = (T + R - 1) / R;
  const unsigned grid = (unsigned)(groups < 4096 ? groups : 4096);
  hipLaunchKernelGGL((rmsnorm_fwd_kernel<DT, NV, R>), dim3(grid), dim3(kNormThreads), 0, st,
                     static_cast<const unsigned char*>(x), static_cast<const unsigned char*>(w), T, H,
                     eps, static_cast<unsigned char*>(y), rstd);
}

template <int DT, int NV>
static void launch_bwd(const void* dy, const void* x, const void* w, const float* rstd,
                       const void* dres, int64_t T, int H, void* dx, void* dweight, float* partial,
                       hipStream_t st) {
  constexpr int R = norm_bwd_rows(NV, DT);
  const int parts = norm_parts(T, R);
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<DT, NV, R>), dim3((unsigned)parts), dim3(kNormThreads), 0, st,
                     static_cast<const unsigned char*>(dy), static_cast<const unsigned char*>(x),
                     static_cast<const unsigned char*>(w), rstd,
                     static_cast<const unsigned char*>(dres), T, H, static_cast<unsigned char*>(dx),
                     partial);
  const unsigned grid = (unsigned)((H + kDwCols - 1) / kDwCols);
  hipLaunchKernelGGL((rmsnorm_dw_kernel<DT>), dim3(grid), dim3(kDwThreads), 0, st, partial, parts, H,
                     static_cast<unsigned char*>(dweight));
}

template <int DT, typename F>
static bool by_nv(int nv, F&& f) {
  switch (nv) {
    case 1: f(std::integral_constant<int, 1>{}); return true;
    case 2: f(std::integral_constant<int, 2>{}); return true;
    case 4: f(std::integral_constant<int, 4>{}); return true;
    case 8: f(std::integral_constant<int, 8>{}); return true;
  }
  return false;
}

static int norm_shape_status(int64_t T, int64_t H, int dtype) {
  if (dtype != GMOE_F32 && dtype != GMOE_BF16 && dtype != GMOE_F16) return GMOE_ERR_UNSUPPORTED;
  if (T < 0 || H < 1) return GMOE_ERR_INVALID;
  const int epv = dtype == GMOE_F32 ? 4 : 8;
  if (H % epv != 0) return GMOE_ERR_INVALID;
  if (norm_nv(H, dtype) == 0) return GMOE_ERR_UNSUPPORTED;
  return GMOE_OK;
}

}  // namespace gmoe

extern "C" int gmoe_rmsnorm_fwd(const void* x, const void* weight, int64_t T, int64_t H, float eps,
                                int dtype, void* y, float* rstd, void* stream) {
  using namespace gmoe;
  const int stt = norm_shape_status(T, H, dtype);
  if (stt != GMOE_OK) return stt;
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(x && weight && y && rstd);
  GMOE_CHECK_ARG(gmoe_aligned(x, 16) && gmoe_aligned(weight, 16) && gmoe_aligned(y, 16));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nv = norm_nv(H, dtype);
  auto go = [&](auto dt) {
    constexpr int DT = decltype(dt)::value;
    by_nv<DT>(nv, [&](auto n) {
      launch_fwd<DT, decltype(n)::value>(x, weight, T, (int)H, eps, y, rstd, st);
    });
  };
  if (dtype == GMOE_F32) go(std::integral_constant<int, GMOE_F32>{});
  else if (dtype == GMOE_BF16) go(std::integral_constant<int, GMOE_BF16>{});
  else go(std::integral_constant<int, GMOE_F16>{});
  return gmoe_launch_status();
}

extern "C" int64_t gmoe_rmsnorm_bwd_workspace_rows(int64_t T, int64_t H, int dtype) {
  using namespace gmoe;
  if (norm_shape_status(T, H, dtype) != GMOE_OK) return -1;
  return norm_parts(T, norm_bwd_rows(norm_nv(H, dtype), dtype));
}

extern "C" int gmoe_rmsnorm_bwd(const void* dy, const void* x, const void* weight, const float* rstd,
                                const void* dresidual, int64_t T, int64_t H, int dtype, void* dx,
                                void* dweight, float* workspace, int64_t workspace_rows,
                                void* stream) {
  using namespace gmoe;
  const int stt = norm_shape_status(T, H, dtype);
  if (stt != GMOE_OK) return stt;
  GMOE_CHECK_ARG(dweight && weight);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nv = norm_nv(H, dtype);
  if (T > 0) {
    GMOE_CHECK_ARG(dy && x && rstd && dx && workspace);
    GMOE_CHECK_ARG(gmoe_aligned(dy, 16) && gmoe_aligned(x, 16) && gmoe_aligned(weight, 16) &&
                   gmoe_aligned(dx, 16) && gmoe_aligned(workspace, 16) && gmoe_aligned(dresidual, 16));
    GMOE_CHECK_ARG(workspace_rows >= norm_parts(T, norm_bwd_rows(nv, dtype)));
  }
  auto go = [&](auto dt) {
    constexpr int DT = decltype(dt)::value;
    if (T == 0) {  // no rows: the weight gradient is zero
      const unsigned grid = (unsigned)((H + kDwCols - 1) / kDwCols);
      hipLaunchKernelGGL((rmsnorm_dw_kernel<DT>), dim3(grid), dim3(kDwThreads), 0, st,
                         static_cast<const float*>(nullptr), 0, (int)H,
                         static_cast<unsigned char*>(dweight));
      return;
    }
    by_nv<DT>(nv, [&](auto n) {
      launch_bwd<DT, decltype(n)::value>(dy, x, weight, rstd, dresidual, T, (int)H, dx, dweight,
                                         workspace, st);
    });
  };
  if (dtype == GMOE_F32) go(std::integral_constant<int, GMOE_F32>{});
  else if (dtype == GMOE_BF16) go(std::integral_constant<int, GMOE_BF16>{});
  else go(std::integral_constant<int, GMOE_F16>{});
  return gmoe_launch_status();
}
