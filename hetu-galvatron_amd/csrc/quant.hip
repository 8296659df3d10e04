// Block-scaled fp8 (e4m3fn) quantisation for gfx950.  The reference keeps its fp8 expert path
// commented out (moe/mlp.py:164-184), so the formats are defined here.
//   * Expert weights: one bf16 scale per 128x128 tile of each [K, M] matrix, scale = bf16(amax / 448)
//     (1 for an all-zero tile), q = rne(w / scale) saturated to +-448; consumed by gmoe_gmm_fp8w and
//     gmoe_gmm_fp8a.
//   * Activations: one power-of-two scale per row and 128 reduction elements, 2^e with the smallest
//     e for which amax * 2^-e <= 448 (e = -127 for an all-zero block), q = rne(x * 2^-e); the scale is
//     stored as its E8M0 byte (e + 127) in all four bytes of a dword of a table [K/128][N], the form
//     the block-scaled fp8 MFMA takes as its scale operand; consumed by gmoe_gmm_fp8a.
#include "gmoe_common.h"

namespace gmoe {

constexpr int kQBlock = 128;
constexpr float kFp8Max = 448.0f;

// One workgroup of 256 threads per tile; thread t covers columns 8*(t%16)..+7 of rows t/16 + 16*i.
template <int DT>
__global__ __launch_bounds__(256) void quantize_fp8_block_kernel(const unsigned char* w, int64_t K,
                                                                 int64_t M, unsigned char* q,
                                                                 uint16_t* scale) {
  const int mb = blockIdx.x, kb = blockIdx.y;
  const int64_t b = blockIdx.z;
  const int kbs = gridDim.y, mbs = gridDim.x;
  const int tid = threadIdx.x, c8 = tid & 15, r0 = tid >> 4;
  const unsigned char* wm = w + b * K * M * Elem<DT>::bytes;
  unsigned char* qm = q + b * K * M;
  const int64_t col = (int64_t)mb * kQBlock + c8 * 8;

  float v[8][8];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t row = (int64_t)kb * kQBlock + r0 + 16 * i;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool ok = row < K && col + j < M;
      v[i][j] = ok ? Elem<DT>::load(wm, row * M + col + j) : 0.f;
      amax = fmaxf(amax, fabsf(v[i][j]));
    }
  }
  __shared__ float part[4];
  amax = group_max_f32<64>(amax);
  if ((tid & 63) == 0) part[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
  uint32_t sbits = f32_to_bf16_bits(amax / kFp8Max);
  if (bf16_bits_to_f32(sbits) == 0.f) sbits = 0x3f80u;  // 1.0
  if (tid == 0) scale[(b * kbs + kb) * mbs + mb] = (uint16_t)sbits;
  const float s = bf16_bits_to_f32(sbits);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t row = (int64_t)kb * kQBlock + r0 + 16 * i;
    if (row >= K) continue;
    uint32_t lo = 0, hi = 0;
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = fminf(fmaxf(v[i][j] / s, -kFp8Max), kFp8Max);
    lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], (int)lo, false);
    lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], (int)lo, true);
    hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], (int)hi, false);
    hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], (int)hi, true);
    if (col + 8 <= M) {
      *reinterpret_cast<u32x2*>(qm + row * M + col) = u32x2{lo, hi};
    } else {
      for (int j = 0; j < 8 && col + j < M; ++j)
        qm[row * M + col + j] = (unsigned char)(((j < 4 ? lo : hi) >> (8 * (j & 3))) & 0xffu);
    }
  }
}

// One wavefront per row; a group of 16 lanes owns a 128-element block, 8 elements per lane, four
// blocks per pass.  The 16-byte loads of kRowPasses passes are requested before the first block is
// reduced (a pass alone keeps 1 KiB per wavefront in flight, far too little for HBM).
constexpr int kRowPasses = 8;

// The 16 lanes that own a block agree on its scale, write it (lane c == 0) and their 8 codes each.
__device__ __forceinline__ void quantize_block_of_row(const float (&v)[8], int c, bool in_table, bool in_row,
                                                      int32_t* scale_slot, unsigned char* q8) {
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
#pragma unroll
  for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
  // smallest e with amax * 2^-e <= 448 = 0.875 * 2^9: amax = m * 2^ex, m in [0.5, 1)
  int e = -127;
  if (amax > 0.f) {
    int ex;
    const float m = frexpf(amax, &ex);
    e = m <= 0.875f ? ex - 9 : ex - 8;
    e = e < -127 ? -127 : (e > 127 ? 127 : e);
  }
  if (in_table && c == 0) {
    const uint32_t b = (uint32_t)(e + 127);
    *scale_slot = (int32_t)(b | (b << 8) | (b << 16) | (b << 24));
  }
  if (!in_row) return;
  float f[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = ldexpf(v[j], -e);
  uint32_t lo = 0, hi = 0;
  lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], (int)lo, false);
  lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], (int)lo, true);
  hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], (int)hi, false);
  hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], (int)hi, true);
  *reinterpret_cast<u32x2*>(q8) = u32x2{lo, hi};
}

// Rounds a product to DT's storage type.  The value is pinned in a register first: left to itself the
// compiler folds the multiply into the fp16 conversion as fma(a, b, +0) (v_fma_mixlo_f16), which turns
// a product of -0 into +0, and the activation kernels store -0.
template <int DT>
__device__ __forceinline__ float round_product(float t) {
  asm volatile("" : "+v"(t));
  return Elem<DT>::round(t);
}

template <int DT>
__device__ __forceinline__ void load8(const unsigned char* p, float (&v)[8]) {
  if constexpr (Elem<DT>::bytes == 2) {
    Vec16<DT>::unpack(ld16_nt(p), v);
  } else {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(p);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(p + 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = lo[j];
      v[4 + j] = hi[j];
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void quantize_fp8_rows_kernel(const unsigned char* x, int64_t N,
                                                                int64_t K, unsigned char* q,
                                                                int32_t* scale) {
  constexpr int ES = Elem<DT>::bytes;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= N) return;
  const int g = lane >> 4, c = lane & 15;
  const int64_t kbs = (K + kQBlock - 1) / kQBlock;
  const unsigned char* xr = x + row * K * ES;
  for (int64_t kb0 = 0; kb0 < kbs; kb0 += 4 * kRowPasses) {
    // K is a multiple of 8, so a lane's 8 elements are all inside the row or all outside
    float v[kRowPasses][8];
#pragma unroll
    for (int p = 0; p < kRowPasses; ++p) {
      const int64_t k0 = (kb0 + 4 * p + g) * kQBlock + c * 8;
      if (k0 < K) {
        load8<DT>(xr + k0 * ES, v[p]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[p][j] = 0.f;
      }
    }
#pragma unroll
    for (int p = 0; p < kRowPasses; ++p) {
      const int64_t kb = kb0 + 4 * p + g;
      const int64_t k0 = kb * kQBlock + c * 8;
      quantize_block_of_row(v[p], c, kb < kbs, k0 < K, scale + kb * N + row, q + row * K + k0);
    }
  }
}

// The gated activation and the quantiser in one pass: the rows that enter the second product, act(y[:,
// :F]) * y[:, F:] rounded to DT as the activation kernel stores it, leave as fp8 codes and scales
// only.  Same lane layout as above over the F columns of the result.
template <int DT, int ACT>
__global__ __launch_bounds__(256) void glu_fwd_quantize_rows_kernel(const unsigned char* y, int64_t N,
                                                                    int64_t F, unsigned char* q,
                                                                    int32_t* scale) {
  constexpr int ES = Elem<DT>::bytes;
  constexpr int PASSES = 4;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= N) return;
  const int g = lane >> 4, c = lane & 15;
  const int64_t kbs = (F + kQBlock - 1) / kQBlock;
  const unsigned char* yr = y + row * 2 * F * ES;
  for (int64_t kb0 = 0; kb0 < kbs; kb0 += 4 * PASSES) {
    float a[PASSES][8], b[PASSES][8];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int64_t k0 = (kb0 + 4 * p + g) * kQBlock + c * 8;
      if (k0 < F) {
        load8<DT>(yr + k0 * ES, a[p]);
        load8<DT>(yr + (F + k0) * ES, b[p]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) a[p][j] = b[p][j] = 0.f;
      }
    }
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int64_t kb = kb0 + 4 * p + g;
      const int64_t k0 = kb * kQBlock + c * 8;
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = round_product<DT>(glu_act(a[p][j], ACT == GMOE_ACT_GELU) * b[p][j]);
      quantize_block_of_row(v, c, kb < kbs, k0 < F, scale + kb * N + row, q + row * F + k0);
    }
  }
}

// The activation backward and the quantiser in one pass: the rows that enter the input-gradient
// product, [d * act'(gate) * up | d * act(gate)] rounded to DT as the backward kernel stores them, as
// codes and scales only ([N, 2F] codes, scale blocks 0 .. F/128-1 of the first half, F/128 .. of the
// second).  A lane loads d, gate and up of its 8 columns once and quantises its block of either half.
// F is a multiple of 128.
template <int DT, int ACT>
__global__ __launch_bounds__(256) void glu_bwd_quantize_rows_kernel(const unsigned char* d,
                                                                    const unsigned char* y, int64_t N,
                                                                    int64_t F, unsigned char* q,
                                                                    int32_t* scale) {
  constexpr int ES = Elem<DT>::bytes;
  constexpr int PASSES = 2;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= N) return;
  const int g = lane >> 4, c = lane & 15;
  const int64_t kbs = F / kQBlock;
  const unsigned char* yr = y + row * 2 * F * ES;
  const unsigned char* dr = d + row * F * ES;
  for (int64_t kb0 = 0; kb0 < kbs; kb0 += 4 * PASSES) {
    float a[PASSES][8], b[PASSES][8], go[PASSES][8];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int64_t k0 = (kb0 + 4 * p + g) * kQBlock + c * 8;
      if (k0 < F) {
        load8<DT>(yr + k0 * ES, a[p]);
        load8<DT>(yr + (F + k0) * ES, b[p]);
        load8<DT>(dr + k0 * ES, go[p]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) a[p][j] = b[p][j] = go[p][j] = 0.f;
      }
    }
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int64_t kb = kb0 + 4 * p + g;
      const int64_t k0 = kb * kQBlock + c * 8;
      const bool in = kb < kbs;
      float da[8], db[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        da[j] = round_product<DT>(go[p][j] * glu_act_grad(a[p][j], ACT == GMOE_ACT_GELU) * b[p][j]);
        db[j] = round_product<DT>(go[p][j] * glu_act(a[p][j], ACT == GMOE_ACT_GELU));
      }
      quantize_block_of_row(da, c, in, in, scale + kb * N + row, q + row * 2 * F + k0);
      quantize_block_of_row(db, c, in, in, scale + (kbs + kb) * N + row, q + row * 2 * F + F + k0);
    }
  }
}

}  // namespace gmoe

extern "C" int gmoe_quantize_fp8_block(const void* w, int dtype, int64_t batch, int64_t K, int64_t M,
                                       void* q, void* scale, void* stream) {
  using namespace gmoe;
  GMOE_CHECK_ARG(batch >= 0 && K >= 1 && M >= 1);
  if (batch == 0) return GMOE_OK;
  GMOE_CHECK_ARG(w && q && scale);
  if ((M % 8) != 0) return GMOE_ERR_UNSUPPORTED;
  if (!gmoe_aligned(q, 8)) return GMOE_ERR_INVALID;
  const int64_t kbs = (K + kQBlock - 1) / kQBlock, mbs = (M + kQBlock - 1) / kQBlock;
  if (kbs > 65535 || batch > 65535) return GMOE_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)mbs, (unsigned)kbs, (unsigned)batch), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned char* ww = static_cast<const unsigned char*>(w);
  unsigned char* qq = static_cast<unsigned char*>(q);
  uint16_t* ss = static_cast<uint16_t*>(scale);
  switch (dtype) {
    case GMOE_F32:
      hipLaunchKernelGGL((quantize_fp8_block_kernel<GMOE_F32>), grid, block, 0, st, ww, K, M, qq, ss);
      break;
    case GMOE_BF16:
      hipLaunchKernelGGL((quantize_fp8_block_kernel<GMOE_BF16>), grid, block, 0, st, ww, K, M, qq, ss);
      break;
    case GMOE_F16:
      hipLaunchKernelGGL((quantize_fp8_block_kernel<GMOE_F16>), grid, block, 0, st, ww, K, M, qq, ss);
      break;
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}

extern "C" int gmoe_quantize_fp8_rows(const void* x, int dtype, int64_t N, int64_t K, void* q,
                                      int32_t* scales, void* stream) {
  using namespace gmoe;
  GMOE_CHECK_ARG(N >= 0 && K >= 1);
  if (N == 0) return GMOE_OK;
  GMOE_CHECK_ARG(x && q && scales);
  if ((K % 8) != 0) return GMOE_ERR_UNSUPPORTED;
  if (!gmoe_aligned(q, 8) || !gmoe_aligned(x, 16)) return GMOE_ERR_INVALID;
  const dim3 grid((unsigned)((N + 3) / 4)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned char* xx = static_cast<const unsigned char*>(x);
  unsigned char* qq = static_cast<unsigned char*>(q);
  switch (dtype) {
    case GMOE_F32:
      hipLaunchKernelGGL((quantize_fp8_rows_kernel<GMOE_F32>), grid, block, 0, st, xx, N, K, qq, scales);
      break;
    case GMOE_BF16:
      hipLaunchKernelGGL((quantize_fp8_rows_kernel<GMOE_BF16>), grid, block, 0, st, xx, N, K, qq, scales);
      break;
    case GMOE_F16:
      hipLaunchKernelGGL((quantize_fp8_rows_kernel<GMOE_F16>), grid, block, 0, st, xx, N, K, qq, scales);
      break;
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}

namespace gmoe {
template <int DT>
static void launch_glu_quantize(bool bwd, int act, const unsigned char* d, const unsigned char* y, int64_t N,
                                int64_t F, unsigned char* q, int32_t* scales, hipStream_t st) {
  const dim3 grid((unsigned)((N + 3) / 4)), block(256);
  const bool gelu = act == GMOE_ACT_GELU;
  if (!bwd) {
    auto kern = gelu ? glu_fwd_quantize_rows_kernel<DT, GMOE_ACT_GELU> : glu_fwd_quantize_rows_kernel<DT, GMOE_ACT_SILU>;
    hipLaunchKernelGGL(kern, grid, block, 0, st, y, N, F, q, scales);
  } else {
    auto kern = gelu ? glu_bwd_quantize_rows_kernel<DT, GMOE_ACT_GELU> : glu_bwd_quantize_rows_kernel<DT, GMOE_ACT_SILU>;
    hipLaunchKernelGGL(kern, grid, block, 0, st, d, y, N, F, q, scales);
  }
}

static int glu_quantize_dispatch(bool bwd, const void* grad_out, const void* y, int dtype, int64_t N,
                                 int64_t F, int act, void* q, int32_t* scales, void* stream) {
  GMOE_CHECK_ARG(N >= 0 && F >= 1);
  GMOE_CHECK_ARG(act == GMOE_ACT_SILU || act == GMOE_ACT_GELU);
  if (N == 0) return GMOE_OK;
  GMOE_CHECK_ARG(y && q && scales && (!bwd || grad_out));
  if ((F % (bwd ? kQBlock : 8)) != 0) return GMOE_ERR_UNSUPPORTED;
  if (!gmoe_aligned(q, 8) || !gmoe_aligned(y, 16) || !gmoe_aligned(grad_out, 16)) return GMOE_ERR_INVALID;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned char* dd = static_cast<const unsigned char*>(grad_out);
  const unsigned char* yy = static_cast<const unsigned char*>(y);
  unsigned char* qq = static_cast<unsigned char*>(q);
  switch (dtype) {
    case GMOE_F32: launch_glu_quantize<GMOE_F32>(bwd, act, dd, yy, N, F, qq, scales, st); break;
    case GMOE_BF16: launch_glu_quantize<GMOE_BF16>(bwd, act, dd, yy, N, F, qq, scales, st); break;
    case GMOE_F16: launch_glu_quantize<GMOE_F16>(bwd, act, dd, yy, N, F, qq, scales, st); break;
    default: return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}
}  // namespace gmoe

extern "C" int gmoe_glu_fwd_quantize_fp8_rows(const void* y, int dtype, int64_t N, int64_t F, int act,
                                              void* q, int32_t* scales, void* stream) {
  return gmoe::glu_quantize_dispatch(false, nullptr, y, dtype, N, F, act, q, scales, stream);
}

extern "C" int gmoe_glu_bwd_quantize_fp8_rows(const void* grad_out, const void* y, int dtype, int64_t N,
                                              int64_t F, int act, void* q, int32_t* scales,
                                              void* stream) {
  return gmoe::glu_quantize_dispatch(true, grad_out, y, dtype, N, F, act, q, scales, stream);
}
