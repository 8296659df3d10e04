// Expert-capacity selection for gfx950: keep at most `capacity` tokens per expert
// (topk_softmax_with_capacity, moe/moe_utils.py:519-544).  The reference takes a top-`capacity`
// along the token axis of the dense gate matrix ("probs" policy) or of the 0/1 routing map
// ("position" policy) with torch.topk, whose order among equal values is unspecified; here the
// rule is fixed: among equal keys the lowest token index wins.
//
// One workgroup per expert column.  The capacity-th largest key is found by a 4-pass, 8-bit radix
// selection with an LDS histogram; a last pass in token order keeps every key above the threshold
// and the first `need` keys equal to it (ballot ranks inside a wavefront, a 16-entry scan across
// the wavefronts of the block).
#include "gmoe_common.h"

namespace gmoe {

constexpr int kCapThreads = 1024;

// Order-preserving image of an fp32 value in unsigned integers.
__device__ __forceinline__ uint32_t f32_sort_key(float v) {
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

template <int PDT>
__global__ __launch_bounds__(kCapThreads) void capacity_select_kernel(
    const unsigned char* probs, const uint8_t* routing_map, int64_t T, int E, int64_t capacity,
    int by_position, int pad, unsigned char* out_probs, uint8_t* out_map) {
  __shared__ unsigned int hist[256];
  __shared__ unsigned int sel[2];       // chosen byte, remaining count
  __shared__ unsigned int wave_cnt[kCapThreads / 64];
  const int e = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  auto key_of = [&](int64_t t) -> uint32_t {
    if (by_position) return routing_map[t * E + e] ? 1u : 0u;
    return f32_sort_key(Elem<PDT>::load(probs, t * E + e));
  };

  // ---- threshold: the capacity-th largest key -------------------------------------------------
  uint32_t prefix = 0, known = 0;
  unsigned int need = (unsigned int)capacity;  // 1 <= capacity <= T (checked by the host)
  for (int pass = 3; pass >= 0; --pass) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int64_t t = tid; t < T; t += kCapThreads) {
      const uint32_t k = key_of(t);
      if ((k & known) == prefix) atomicAdd(&hist[(k >> (8 * pass)) & 255u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      unsigned int cum = 0;
      int b = 255;
      for (; b > 0; --b) {
        if (cum + hist[b] >= need) break;
        cum += hist[b];
      }
      sel[0] = (unsigned int)b;
      sel[1] = need - cum;
    }
    __syncthreads();
    prefix |= sel[0] << (8 * pass);
    known |= 0xffu << (8 * pass);
    need = sel[1];
    __syncthreads();
  }
  const uint32_t thr = prefix;  // `need` keys equal to thr are kept, in token order

  // ---- selection in token order -----------------------------------------------------------------
  unsigned int eq_before = 0;
  for (int64_t t0 = 0; t0 < T; t0 += kCapThreads) {
    const int64_t t = t0 + tid;
    const bool in = t < T;
    const uint32_t k = in ? key_of(t) : 0u;
    const bool eq = in && k == thr;
    const uint64_t bal = __ballot(eq);
    if (lane == 0) wave_cnt[wave] = (unsigned int)__popcll(bal);
    __syncthreads();
    unsigned int before = eq_before, total = 0;
    for (int w = 0; w < kCapThreads / 64; ++w) {
      const unsigned int c = wave_cnt[w];
      if (w < wave) before += c;
      total += c;
    }
    const unsigned int rank = before + (unsigned int)__popcll(bal & ((1ull << lane) - 1ull));
    if (in) {
      const bool chosen = k > thr || (eq && rank < need);
      const bool keep = pad ? chosen : (chosen && routing_map[t * E + e] != 0);
      out_map[t * E + e] = keep ? 1 : 0;
      Elem<PDT>::store(out_probs, t * E + e, keep ? Elem<PDT>::load(probs, t * E + e) : 0.f);
    }
    eq_before += total;
    __syncthreads();
  }
}

}  // namespace gmoe

extern "C" int gmoe_capacity_select(const void* probs, int probs_dtype, const uint8_t* routing_map,
                                    int64_t T, int E, int64_t capacity, int by_position, int pad,
                                    void* out_probs, uint8_t* out_map, void* stream) {
  using namespace gmoe;
  GMOE_CHECK_ARG(T >= 0 && E >= 1 && capacity >= 1);
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(probs && routing_map && out_probs && out_map);
  if (capacity > T) capacity = T;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)E), block(kCapThreads);
  const unsigned char* pp = static_cast<const unsigned char*>(probs);
  unsigned char* op = static_cast<unsigned char*>(out_probs);
  switch (probs_dtype) {
    case GMOE_F32:
      hipLaunchKernelGGL((capacity_select_kernel<GMOE_F32>), grid, block, 0, st, pp, routing_map, T, E,
                         capacity, by_position, pad, op, out_map);
      break;
    case GMOE_BF16:
      hipLaunchKernelGGL((capacity_select_kernel<GMOE_BF16>), grid, block, 0, st, pp, routing_map, T, E,
                         capacity, by_position, pad, op, out_map);
      break;
    case GMOE_F16:
      hipLaunchKernelGGL((capacity_select_kernel<GMOE_F16>), grid, block, 0, st, pp, routing_map, T, E,
                         capacity, by_position, pad, op, out_map);
      break;
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}
