// Per-expert bias rows for gfx950: out[r] = x[r] + bias[expert of row r] and the bias gradient
// (column sums over each expert's rows).  The reference's experts with `add_bias_linear` add the
// fc1 bias before the activation (transformer/mlp.py:104-135: bias_swiglu_impl / `intermediate +
// bias`) and hand the fc2 bias on as rows, `output_bias.expand_as(output)` (moe/mlp.py:200-207).
#include "gmoe_common.h"

namespace gmoe {

// group of row r in a table of G+1 ascending offsets; G for a row past the last offset
__device__ __forceinline__ int group_of_row(const int64_t* __restrict__ offsets, int G, int64_t r) {
  if (offsets == nullptr) return 0;
  if (r >= offsets[G]) return G;
  int lo = 0, hi = G;  // offsets[lo] <= r < offsets[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (offsets[mid] <= r)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

// x may be null (the bias alone is expanded to rows) or equal to out; rows past the last group keep
// x (or zero)
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void bias_rows_kernel(const unsigned char* x,
                                                        const unsigned char* __restrict__ bias,
                                                        const int64_t* __restrict__ offsets, int G,
                                                        int64_t N, int64_t M, unsigned char* out) {
  constexpr int NV = VEC ? Vec16<DT>::n : 1;
  const int64_t per_row = M / NV;
  const int64_t total = N * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / per_row, c = i % per_row;
    const int g = group_of_row(offsets, G, r);
    if (VEC) {
      float a[NV], b[NV];
#pragma unroll
      for (int q = 0; q < NV; ++q) a[q] = b[q] = 0.f;
      if (x) Vec16<DT>::unpack(ld16_nt(x + (r * M) * Elem<DT>::bytes + c * 16), a);
      if (g < G) Vec16<DT>::unpack(*reinterpret_cast<const u32x4*>(bias + ((int64_t)g * M) * Elem<DT>::bytes + c * 16), b);
#pragma unroll
      for (int q = 0; q < NV; ++q) a[q] += b[q];
      st16_nt(out + (r * M) * Elem<DT>::bytes + c * 16, Vec16<DT>::pack(a));
    } else {
      const float a = x ? Elem<DT>::load(x, r * M + c) : 0.f;
      const float b = g < G ? Elem<DT>::load(bias, (int64_t)g * M + c) : 0.f;
      Elem<DT>::store(out, r * M + c, a + b);
    }
  }
}

// grad_bias[g][c] = sum over the rows of group g of grad[r][c]: 64 columns per workgroup, the rows
// dealt to four lanes per column, fp32 partial sums added in a fixed order (no atomics)
template <int DT>
__global__ __launch_bounds__(256) void bias_rows_bwd_kernel(const unsigned char* __restrict__ grad,
                                                            const int64_t* __restrict__ offsets,
                                                            int64_t N, int64_t M,
                                                            unsigned char* grad_bias) {
  __shared__ float part[4][64];
  const int g = blockIdx.y;
  const int col = threadIdx.x & 63, phase = threadIdx.x >> 6;
  const int64_t c = (int64_t)blockIdx.x * 64 + col;
  const int64_t r0 = offsets ? offsets[g] : 0, r1 = offsets ? offsets[g + 1] : N;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < M) {
    // four independent chains per lane so that the loads overlap; their order of addition is fixed
    int64_t r = r0 + phase;
    for (; r + 12 < r1; r += 16) {
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] += Elem<DT>::load(grad, (r + 4 * u) * M + c);
    }
    for (int u = 0; r < r1; r += 4, ++u) acc[u & 3] += Elem<DT>::load(grad, r * M + c);
  }
  part[phase][col] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  __syncthreads();
  if (phase == 0 && c < M)
    Elem<DT>::store(grad_bias, (int64_t)g * M + c,
                    (part[0][col] + part[1][col]) + (part[2][col] + part[3][col]));
}

static int bias_grid(int64_t total) {
  const int64_t blocks = (total + 255) / 256;
  return (int)(blocks < 1 ? 1 : (blocks > 256 * 16 ? 256 * 16 : blocks));
}

template <int DT>
static void launch_bias_rows(bool vec, const void* x, const void* bias, const int64_t* offsets, int G,
                             int64_t N, int64_t M, void* out, hipStream_t st) {
  const int64_t total = N * (M / (vec ? Vec16<DT>::n : 1));
  const dim3 grid(bias_grid(total)), block(256);
  auto kern = vec ? bias_rows_kernel<DT, true> : bias_rows_kernel<DT, false>;
  hipLaunchKernelGGL(kern, grid, block, 0, st, static_cast<const unsigned char*>(x),
                     static_cast<const unsigned char*>(bias), offsets, G, N, M,
                     static_cast<unsigned char*>(out));
}

}  // namespace gmoe

extern "C" int gmoe_bias_rows(const void* x, const void* bias, int dtype, int64_t N, int64_t M,
                              const int64_t* expert_offsets, int E, void* out, void* stream) {
  GMOE_CHECK_ARG(N >= 0 && M >= 1 && E >= 1);
  GMOE_CHECK_ARG(expert_offsets != nullptr || E == 1);
  if (N == 0) return GMOE_OK;
  GMOE_CHECK_ARG(bias && out);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int es = dtype == GMOE_F32 ? 4 : 2;
  const bool vec = ((M * es) & 15) == 0 && gmoe_aligned(x, 16) && gmoe_aligned(bias, 16) &&
                   gmoe_aligned(out, 16);
  switch (dtype) {
    case GMOE_F32: gmoe::launch_bias_rows<GMOE_F32>(vec, x, bias, expert_offsets, E, N, M, out, st); break;
    case GMOE_BF16: gmoe::launch_bias_rows<GMOE_BF16>(vec, x, bias, expert_offsets, E, N, M, out, st); break;
    case GMOE_F16: gmoe::launch_bias_rows<GMOE_F16>(vec, x, bias, expert_offsets, E, N, M, out, st); break;
    default: return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}

extern "C" int gmoe_bias_rows_bwd(const void* grad, int dtype, int64_t N, int64_t M,
                                  const int64_t* expert_offsets, int E, void* grad_bias,
                                  void* stream) {
  GMOE_CHECK_ARG(N >= 0 && M >= 1 && E >= 1 && E <= 65535);
  GMOE_CHECK_ARG(expert_offsets != nullptr || E == 1);
  GMOE_CHECK_ARG(grad_bias && (grad || N == 0));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((M + 63) / 64), (unsigned)E), block(256);
  const unsigned char* g = static_cast<const unsigned char*>(grad);
  unsigned char* o = static_cast<unsigned char*>(grad_bias);
  switch (dtype) {
    case GMOE_F32: hipLaunchKernelGGL(gmoe::bias_rows_bwd_kernel<GMOE_F32>, grid, block, 0, st, g, expert_offsets, N, M, o); break;
    case GMOE_BF16: hipLaunchKernelGGL(gmoe::bias_rows_bwd_kernel<GMOE_BF16>, grid, block, 0, st, g, expert_offsets, N, M, o); break;
    case GMOE_F16: hipLaunchKernelGGL(gmoe::bias_rows_bwd_kernel<GMOE_F16>, grid, block, 0, st, g, expert_offsets, N, M, o); break;
    default: return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}
