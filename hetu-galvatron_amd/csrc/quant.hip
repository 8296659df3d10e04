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
        if constexpr (ES == 2) {
          Vec16<DT>::unpack(ld16_nt(xr + k0 * 2), v[p]);
        } else {
          const f32x4 lo = *reinterpret_cast<const f32x4*>(xr + k0 * 4);
          const f32x4 hi = *reinterpret_cast<const f32x4*>(xr + k0 * 4 + 16);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[p][j] = lo[j];
            v[p][4 + j] = hi[j];
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[p][j] = 0.f;
      }
    }
#pragma unroll
    for (int p = 0; p < kRowPasses; ++p) {
      const int64_t kb = kb0 + 4 * p + g;
      const int64_t k0 = kb * kQBlock + c * 8;
      float amax = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[p][j]));
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
      if (kb < kbs && c == 0) {
        const uint32_t b = (uint32_t)(e + 127);
        scale[kb * N + row] = (int32_t)(b | (b << 8) | (b << 16) | (b << 24));
      }
      if (k0 >= K) continue;
      float f[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = ldexpf(v[p][j], -e);
      uint32_t lo = 0, hi = 0;
      lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], (int)lo, false);
      lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], (int)lo, true);
      hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], (int)hi, false);
      hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], (int)hi, true);
      *reinterpret_cast<u32x2*>(q + row * K + k0) = u32x2{lo, hi};
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
