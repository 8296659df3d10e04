// Token permute / unpermute for gfx950.
//
// Plan kernels turn the boolean routing map [T,E] into the expert-major, token-ascending (stable)
// permutation the reference builds with transpose + arange + masked_select
// (moe/moe_utils.py:264-272) / `triton_make_row_id_map` (moe/fused_kernels.py:514-605):
//   plan_count  per 256-token chunk and expert: number of routed tokens (wavefront ballots)
//   plan_scan   one exclusive scan over the (expert-major) chunk counts
//   plan_fill   rank inside the chunk from the ballots + chunk base -> destination rows
// The plan is kept token-major (dst_map [T,E] int32) so that the row kernels, which run one
// wavefront per token, find all destinations of a token in one coalesced load.
//
// Row kernels move whole rows with 16-byte accesses per lane (a wavefront covers 1 KiB per
// instruction), with streaming (nontemporal) hints on data that is touched once: scatter (permute), gather-reduce in fp32 (unpermute; also permute's backward) and
// the backward of the weighted unpermute including the gate gradients.
#include <mutex>

#include "gmoe_common.h"

namespace gmoe {

constexpr int kChunkTokens = 256;  // tokens per plan chunk == threads per block

// ------------------------------------------------------------------------------------------
// Plan
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kChunkTokens) void plan_count_kernel(const uint8_t* map, int64_t T,
                                                                   int E, int NC, int vec8,
                                                                   int* counts) {
  extern __shared__ int wc[];  // [4][E]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t t = (int64_t)blockIdx.x * kChunkTokens + tid;
  const bool valid = t < T;
  const uint8_t* row = map + (valid ? t : 0) * (int64_t)E;
  if (vec8) {  // E % 8 == 0 and an 8-byte aligned map: one load covers 8 experts
    for (int eb = 0; eb < E; eb += 8) {
      const uint64_t bits = valid ? *reinterpret_cast<const uint64_t*>(row + eb) : 0ull;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint64_t b = __ballot(((bits >> (8 * j)) & 0xffull) != 0);
        if (lane == 0) wc[wave * E + eb + j] = __popcll(b);
      }
    }
  } else {
    for (int e = 0; e < E; ++e) {
      const uint64_t b = __ballot(valid && row[e] != 0);
      if (lane == 0) wc[wave * E + e] = __popcll(b);
    }
  }
  __syncthreads();
  for (int e = tid; e < E; e += kChunkTokens)
    counts[(int64_t)e * NC + blockIdx.x] = wc[e] + wc[E + e] + wc[2 * E + e] + wc[3 * E + e];
}

constexpr int kScanThreads = 1024;

// Exclusive scan of counts[E*NC] (expert-major) into base[E*NC]; per-expert totals and offsets.
__global__ __launch_bounds__(kScanThreads) void plan_scan_kernel(const int* counts, int E, int NC,
                                                                  int64_t capacity, int* base,
                                                                  long long* tokens_per_expert,
                                                                  long long* expert_offsets) {
  __shared__ int wsum[kScanThreads / 64];
  __shared__ int carry_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t total = (int64_t)E * NC;
  if (NC == 0) {  // no tokens: every expert is empty (or an all-padding block)
    for (int e = tid; e <= E; e += kScanThreads) {
      if (e < E) tokens_per_expert[e] = capacity > 0 ? capacity : 0;
      expert_offsets[e] = capacity > 0 ? (long long)e * capacity : 0;
    }
    return;
  }
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int64_t start = 0; start < total; start += kScanThreads) {
    const int64_t i = start + tid;
    const int c = i < total ? counts[i] : 0;
    int incl = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(incl, d);
      if (lane >= d) incl += o;
    }
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    int wbase = 0;
    for (int w = 0; w < wave; ++w) wbase += wsum[w];
    const int carry = carry_s;
    if (i < total) base[i] = carry + wbase + incl - c;
    __syncthreads();
    if (tid == kScanThreads - 1) carry_s = carry + wbase + incl;
    __syncthreads();
  }
  const int grand = carry_s;
  __syncthreads();
  // per-expert totals from the flat prefix
  for (int e = tid; e < E; e += kScanThreads) {
    const int first = base[(int64_t)e * NC];
    const int next = (e + 1 < E) ? base[(int64_t)(e + 1) * NC] : grand;
    if (capacity > 0) {
      tokens_per_expert[e] = capacity;
      expert_offsets[e] = (long long)e * capacity;
    } else {
      tokens_per_expert[e] = next - first;
      expert_offsets[e] = first;
    }
  }
  if (tid == 0) expert_offsets[E] = capacity > 0 ? (long long)E * capacity : grand;
  if (capacity > 0) {
    // rebase every expert's chunk prefixes onto its fixed-size block
    __syncthreads();
    for (int e = 0; e < E; ++e) {
      const int first = base[(int64_t)e * NC];
      __syncthreads();
      for (int c = tid; c < NC; c += kScanThreads) {
        const int64_t i = (int64_t)e * NC + c;
        base[i] = base[i] - first;  // rank of the chunk's first token inside expert e
      }
      __syncthreads();
    }
  }
}

// Workgroup (chunk, slice): the destination rows of 256 tokens for kFillExperts consecutive experts.
// Slicing the experts keeps the grid at chunks x E / 8 workgroups (a 64-expert router over 8192
// tokens has only 32 chunks) and lets a lane write its token's 8 destinations as two 16-byte stores.
constexpr int kFillExperts = 8;

__global__ __launch_bounds__(kChunkTokens) void plan_fill_kernel(
    const uint8_t* map, int64_t T, int E, int NC, int vec8, int64_t capacity, const int* base,
    int32_t* dst_map, long long* sorted_indices, int64_t sorted_cap, long long* row_id_map) {
  __shared__ unsigned long long bal[kChunkTokens / 64][kFillExperts];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t t = (int64_t)blockIdx.x * kChunkTokens + tid;
  const bool valid = t < T;
  const int e_begin = blockIdx.y * kFillExperts;
  const int e_cnt = E - e_begin < kFillExperts ? E - e_begin : kFillExperts;
  const uint8_t* row = map + (valid ? t : 0) * (int64_t)E + e_begin;
  if (vec8) {  // E % 8 == 0 and an 8-byte aligned map: one load covers the slice
    const uint64_t bits = valid ? *reinterpret_cast<const uint64_t*>(row) : 0ull;
#pragma unroll
    for (int j = 0; j < kFillExperts; ++j) {
      const uint64_t b = __ballot(((bits >> (8 * j)) & 0xffull) != 0);
      if (lane == 0) bal[wave][j] = b;
    }
  } else {
#pragma unroll
    for (int j = 0; j < kFillExperts; ++j) {
      const uint64_t b = __ballot(valid && j < e_cnt && row[j] != 0);
      if (lane == 0) bal[wave][j] = b;
    }
  }
  __syncthreads();
  const uint64_t lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int32_t d[kFillExperts];
#pragma unroll
  for (int j = 0; j < kFillExperts; ++j) {
    d[j] = -1;
    if (j >= e_cnt) continue;
    const int e = e_begin + j;
    int before = 0;
    for (int w = 0; w < wave; ++w) before += __popcll(bal[w][j]);
    const uint64_t b = bal[wave][j];
    const bool pred = (b >> lane) & 1ull;
    int64_t rank = (int64_t)base[(int64_t)e * NC + blockIdx.x] + before + __popcll(b & lt);
    int64_t dst;
    if (capacity > 0)
      dst = rank < capacity ? (int64_t)e * capacity + rank : -1;
    else
      dst = rank;
    if (!pred || dst >= sorted_cap) dst = -1;
    d[j] = (int32_t)dst;
    if (valid) {
      if (row_id_map) row_id_map[(int64_t)e * T + t] = dst;
      if (dst >= 0 && sorted_indices) sorted_indices[dst] = t;
    }
  }
  if (!valid) return;
  int32_t* out = dst_map + t * E + e_begin;
  if (e_cnt == kFillExperts && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
    reinterpret_cast<i32x4*>(out)[0] = i32x4{d[0], d[1], d[2], d[3]};
    reinterpret_cast<i32x4*>(out)[1] = i32x4{d[4], d[5], d[6], d[7]};
  } else {
#pragma unroll
    for (int j = 0; j < kFillExperts; ++j)
      if (j < e_cnt) out[j] = d[j];
  }
}

// ------------------------------------------------------------------------------------------
// Row movers.  One wavefront per token; a row is walked in pieces of CH chunks per lane.
// Loads are streaming (nontemporal): every row is read once.  Stores of rows that the next kernel
// reads (the permuted rows, the gradient rows of the combine's backward) are ordinary stores:
// measured 14 % (permute) and 7 % (backward) faster than nontemporal ones; the combine's output row
// shows no difference and stays nontemporal.
// ------------------------------------------------------------------------------------------
constexpr int kRowThreads = 256;
constexpr int kCH = 8;  // 16-byte chunks per lane held in registers (8 KiB of row per wavefront)

__device__ __forceinline__ float load_prob(const void* p, int64_t i, int pdt) {
  if (pdt == GMOE_F32) return static_cast<const float*>(p)[i];
  if (pdt == GMOE_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  return f16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
}
__device__ __forceinline__ void store_prob(void* p, int64_t i, int pdt, float v) {
  if (pdt == GMOE_F32)
    static_cast<float*>(p)[i] = v;
  else if (pdt == GMOE_BF16)
    static_cast<uint16_t*>(p)[i] = (uint16_t)f32_to_bf16_bits(v);
  else
    static_cast<uint16_t*>(p)[i] = (uint16_t)f32_to_f16_bits(v);
}
__device__ __forceinline__ void copy_prob(const void* src, int64_t si, void* dst, int64_t di,
                                          int pdt) {
  if (pdt == GMOE_F32)
    static_cast<uint32_t*>(dst)[di] = static_cast<const uint32_t*>(src)[si];
  else
    static_cast<uint16_t*>(dst)[di] = static_cast<const uint16_t*>(src)[si];
}

// permuted[dst] = tokens[t]; row_chunks = row bytes / 16.
__global__ __launch_bounds__(kRowThreads) void permute_rows_kernel(
    const unsigned char* tokens, int64_t T, int64_t row_chunks, int E, const int32_t* dst_map,
    int64_t n_out, unsigned char* permuted, const void* probs, int pdt, void* permuted_probs) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (kRowThreads / 64) + (threadIdx.x >> 6);
  if (t >= T) return;  // whole wavefront leaves together
  const int64_t row_bytes = row_chunks * 16;
  const unsigned char* src = tokens + t * row_bytes;
  for (int64_t c0 = 0; c0 < row_chunks; c0 += 64 * kCH) {
    u32x4 r[kCH];
#pragma unroll
    for (int i = 0; i < kCH; ++i) {
      const int64_t c = c0 + i * 64 + lane;
      if (c < row_chunks) r[i] = ld16_nt(src + c * 16);
    }
    for (int eb = 0; eb < E; eb += 64) {
      const int e = eb + lane;
      const int d = e < E ? dst_map[t * E + e] : -1;
      uint64_t m = __ballot(d >= 0 && d < n_out);
      while (m) {
        const int j = __builtin_ctzll(m);
        m &= m - 1;
        const int64_t dst = __builtin_amdgcn_readlane(d, j);
        unsigned char* out = permuted + dst * row_bytes;
#pragma unroll
        for (int i = 0; i < kCH; ++i) {
          const int64_t c = c0 + i * 64 + lane;
          if (c < row_chunks) st16(out + c * 16, r[i]);
        }
        if (permuted_probs && c0 == 0 && lane == 0)
          copy_prob(probs, t * E + eb + j, permuted_probs, dst, pdt);
      }
    }
  }
}

// Element-granular fallback for rows that are not a multiple of 16 bytes.
__global__ __launch_bounds__(kRowThreads) void permute_rows_generic_kernel(
    const unsigned char* tokens, int64_t T, int64_t H, int es, int E, const int32_t* dst_map,
    int64_t n_out, unsigned char* permuted, const void* probs, int pdt, void* permuted_probs) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (kRowThreads / 64) + (threadIdx.x >> 6);
  if (t >= T) return;
  for (int e = 0; e < E; ++e) {
    const int d = dst_map[t * E + e];
    if (d < 0 || d >= n_out) continue;
    if (es == 2) {
      const uint16_t* s = reinterpret_cast<const uint16_t*>(tokens) + t * H;
      uint16_t* o = reinterpret_cast<uint16_t*>(permuted) + (int64_t)d * H;
      for (int64_t h = lane; h < H; h += 64) o[h] = s[h];
    } else {
      const uint32_t* s = reinterpret_cast<const uint32_t*>(tokens) + t * H;
      uint32_t* o = reinterpret_cast<uint32_t*>(permuted) + (int64_t)d * H;
      for (int64_t h = lane; h < H; h += 64) o[h] = s[h];
    }
    if (permuted_probs && lane == 0) copy_prob(probs, t * E + e, permuted_probs, d, pdt);
  }
}

// The value as it is, but opaque to the compiler: what is unpacked from it is unpacked again at the
// next use instead of being kept (a row piece held as fp32 takes twice to four times the registers).
__device__ __forceinline__ u32x4 keep_packed(u32x4 v) {
  asm volatile("" : "+v"(v));
  return v;
}

// out[t] = sum_e permuted[dst_map[t,e]] * p[t,e]  (fp32 accumulation, ascending e)
// EXTRA: an addend and / or a residual row may follow (their registers cost a wavefront per SIMD).
template <int DT, bool VEC, bool EXTRA>
__global__ __launch_bounds__(kRowThreads) void unpermute_rows_kernel(
    const unsigned char* permuted, int64_t T, int64_t H, int E, const int32_t* dst_map,
    int64_t n_out, const void* mprobs, int pdt, unsigned char* out, const void* pprobs_in,
    void* uprobs_out, const unsigned char* addend, const unsigned char* residual) {
  constexpr int N = VEC ? Vec16<DT>::n : 1;
  constexpr int ES = Elem<DT>::bytes;
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (kRowThreads / 64) + (threadIdx.x >> 6);
  if (t >= T) return;
  const int64_t row_chunks = H / N;
  const int64_t row_bytes = H * ES;
  // destination rows of the first 64 experts: read once, before the rounds over the row
  const int d_first = lane < E ? dst_map[t * E + lane] : -1;
  for (int64_t c0 = 0; c0 < row_chunks; c0 += 64 * kCH) {
    float acc[kCH][N];
#pragma unroll
    for (int i = 0; i < kCH; ++i)
#pragma unroll
      for (int q = 0; q < N; ++q) acc[i][q] = 0.f;
    // the rows added after the sum are requested first: their loads are in flight with the
    // source rows' instead of starting a second round trip when the sum is complete
    u32x4 radd[VEC && EXTRA ? kCH : 1], rres[VEC && EXTRA ? kCH : 1];
    if constexpr (VEC && EXTRA) {
#pragma unroll
      for (int i = 0; i < kCH; ++i) {
        const int64_t c = c0 + i * 64 + lane;
        if (c < row_chunks) {
          if (addend) radd[i] = ld16_nt(addend + t * row_bytes + c * 16);
          if (residual) rres[i] = ld16_nt(residual + t * row_bytes + c * 16);
        }
      }
    }
    for (int eb = 0; eb < E; eb += 64) {
      const int e = eb + lane;
      const int d = eb == 0 ? d_first : (e < E ? dst_map[t * E + e] : -1);
      const bool ok = d >= 0 && d < n_out;
      uint64_t m = __ballot(ok);
      if (uprobs_out && c0 == 0 && e < E) {
        if (ok)
          copy_prob(pprobs_in, d, uprobs_out, t * E + e, pdt);
        else
          store_prob(uprobs_out, t * E + e, pdt, 0.f);
      }
      while (m) {
        // two source rows per round: both rows' loads are in flight before either is consumed
        const int j0 = __builtin_ctzll(m);
        m &= m - 1;
        const bool two = m != 0;
        const int j1 = two ? __builtin_ctzll(m) : j0;
        if (two) m &= m - 1;
        const int64_t srow0 = __builtin_amdgcn_readlane(d, j0);
        const int64_t srow1 = __builtin_amdgcn_readlane(d, j1);
        const float pr0 = mprobs ? load_prob(mprobs, t * E + eb + j0, pdt) : 1.f;
        const float pr1 = mprobs ? load_prob(mprobs, t * E + eb + j1, pdt) : 1.f;
        const unsigned char* src0 = permuted + srow0 * row_bytes;
        const unsigned char* src1 = permuted + srow1 * row_bytes;
        if (VEC) {
          u32x4 r0[kCH], r1[kCH];
#pragma unroll
          for (int i = 0; i < kCH; ++i) {
            const int64_t c = c0 + i * 64 + lane;
            if (c < row_chunks) r0[i] = ld16_nt(src0 + c * 16);
          }
          if (two) {
#pragma unroll
            for (int i = 0; i < kCH; ++i) {
              const int64_t c = c0 + i * 64 + lane;
              if (c < row_chunks) r1[i] = ld16_nt(src1 + c * 16);
            }
          }
#pragma unroll
          for (int i = 0; i < kCH; ++i) {
            const int64_t c = c0 + i * 64 + lane;
            if (c < row_chunks) {
              float f[N];
              Vec16<DT>::unpack(r0[i], f);
#pragma unroll
              for (int q = 0; q < N; ++q) acc[i][q] = fmaf(f[q], pr0, acc[i][q]);
            }
          }
          if (two) {
#pragma unroll
            for (int i = 0; i < kCH; ++i) {
              const int64_t c = c0 + i * 64 + lane;
              if (c < row_chunks) {
                float f[N];
                Vec16<DT>::unpack(r1[i], f);
#pragma unroll
                for (int q = 0; q < N; ++q) acc[i][q] = fmaf(f[q], pr1, acc[i][q]);
              }
            }
          }
        } else {
#pragma unroll
          for (int i = 0; i < kCH; ++i) {
            const int64_t c = c0 + i * 64 + lane;
            if (c < row_chunks) {
              acc[i][0] = fmaf(Elem<DT>::load(src0, c), pr0, acc[i][0]);
              if (two) acc[i][0] = fmaf(Elem<DT>::load(src1, c), pr1, acc[i][0]);
            }
          }
        }
      }
    }
    unsigned char* o = out + t * row_bytes;
    // out = round(round(round(sum) + addend) + residual): the roundings of the separate adds
    // `output += shared_expert_output` and `... + mlp_residual`, each term optional
#pragma unroll
    for (int term = 0; term < (EXTRA ? 2 : 0); ++term) {
      const unsigned char* base = term == 0 ? addend : residual;
      if (base == nullptr) continue;
      const unsigned char* rs = base + t * row_bytes;
#pragma unroll
      for (int i = 0; i < kCH; ++i) {
        const int64_t c = c0 + i * 64 + lane;
        if (c < row_chunks) {
          if (VEC) {
            float f[N];
            Vec16<DT>::unpack(term == 0 ? radd[i] : rres[i], f);
#pragma unroll
            for (int q = 0; q < N; ++q) acc[i][q] = Elem<DT>::round(acc[i][q]) + f[q];
          } else {
            acc[i][0] = Elem<DT>::round(acc[i][0]) + Elem<DT>::load(rs, c);
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kCH; ++i) {
      const int64_t c = c0 + i * 64 + lane;
      if (c < row_chunks) {
        if (VEC)
          st16_nt(o + c * 16, Vec16<DT>::pack(acc[i]));
        else
          Elem<DT>::store(o, c, acc[i][0]);
      }
    }
  }
}

// grad_permuted[dst] = grad_out[t] * p[t,e];  grad_probs[t,e] = <fwd_input[dst], grad_out[t]>
// A piece of the token's gradient row (8 KiB) is loaded once and serves all of the token's experts,
// two at a time: both forward-input rows are requested before either is consumed (24 KiB in flight
// per wavefront).
template <int DT, bool VEC>
__global__ __launch_bounds__(kRowThreads) void unpermute_rows_bwd_kernel(
    const unsigned char* grad_out, const unsigned char* fwd_in, int64_t T, int64_t H, int E,
    const int32_t* dst_map, int64_t n_out, const void* mprobs, int pdt, unsigned char* grad_perm,
    void* grad_probs) {
  constexpr int N = VEC ? Vec16<DT>::n : 1;
  constexpr int ES = Elem<DT>::bytes;
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * (kRowThreads / 64) + (threadIdx.x >> 6);
  if (t >= T) return;
  const int64_t row_chunks = H / N;
  const int64_t row_bytes = H * ES;
  const unsigned char* g = grad_out + t * row_bytes;
  for (int eb = 0; eb < E; eb += 64) {
    const int e = eb + lane;
    const int d = e < E ? dst_map[t * E + e] : -1;
    uint64_t m = __ballot(d >= 0 && d < n_out);
    float mine = 0.f;  // gate gradient of expert eb+lane
    if (VEC) {
      // a piece of the gradient row stays in registers while all of the token's experts use it
      for (int64_t c0 = 0; c0 < row_chunks; c0 += 64 * kCH) {
        u32x4 rg[kCH];
#pragma unroll
        for (int i = 0; i < kCH; ++i) {
          const int64_t c = c0 + i * 64 + lane;
          if (c < row_chunks) rg[i] = ld16_nt(g + c * 16);
        }
        uint64_t mm = m;
        while (mm) {
          const int j0 = __builtin_ctzll(mm);
          mm &= mm - 1;
          const bool two = mm != 0;
          const int j1 = two ? __builtin_ctzll(mm) : j0;
          if (two) mm &= mm - 1;
          const int64_t drow0 = __builtin_amdgcn_readlane(d, j0);
          const int64_t drow1 = __builtin_amdgcn_readlane(d, j1);
          const float pr0 = load_prob(mprobs, t * E + eb + j0, pdt);
          const float pr1 = load_prob(mprobs, t * E + eb + j1, pdt);
          const unsigned char* fin0 = fwd_in + drow0 * row_bytes;
          const unsigned char* fin1 = fwd_in + drow1 * row_bytes;
          unsigned char* gp0 = grad_perm + drow0 * row_bytes;
          unsigned char* gp1 = grad_perm + drow1 * row_bytes;
          u32x4 rf0[kCH], rf1[kCH];
#pragma unroll
          for (int i = 0; i < kCH; ++i) {
            const int64_t c = c0 + i * 64 + lane;
            if (c < row_chunks) rf0[i] = ld16_nt(fin0 + c * 16);
          }
          if (two) {
#pragma unroll
            for (int i = 0; i < kCH; ++i) {
              const int64_t c = c0 + i * 64 + lane;
              if (c < row_chunks) rf1[i] = ld16_nt(fin1 + c * 16);
            }
          }
          float dot0 = 0.f, dot1 = 0.f;
#pragma unroll
          for (int i = 0; i < kCH; ++i) {
            const int64_t c = c0 + i * 64 + lane;
            if (c < row_chunks) {
              float fg[N], ff[N], fo[N];
              Vec16<DT>::unpack(keep_packed(rg[i]), fg);
              Vec16<DT>::unpack(rf0[i], ff);
#pragma unroll
              for (int q = 0; q < N; ++q) {
                fo[q] = fg[q] * pr0;
                dot0 = fmaf(ff[q], fg[q], dot0);
              }
              st16(gp0 + c * 16, Vec16<DT>::pack(fo));
            }
          }
          if (two) {
#pragma unroll
            for (int i = 0; i < kCH; ++i) {
              const int64_t c = c0 + i * 64 + lane;
              if (c < row_chunks) {
                float fg[N], ff[N], fo[N];
                Vec16<DT>::unpack(keep_packed(rg[i]), fg);
                Vec16<DT>::unpack(rf1[i], ff);
#pragma unroll
                for (int q = 0; q < N; ++q) {
                  fo[q] = fg[q] * pr1;
                  dot1 = fmaf(ff[q], fg[q], dot1);
                }
                st16(gp1 + c * 16, Vec16<DT>::pack(fo));
              }
            }
          }
          // the piece's share of <fwd_input[row], grad>, added in piece order
          dot0 = wave_sum_f32(dot0);
          if (lane == j0) mine += dot0;
          if (two) {
            dot1 = wave_sum_f32(dot1);
            if (lane == j1) mine += dot1;
          }
        }
      }
    } else {
      while (m) {
        const int j0 = __builtin_ctzll(m);
        m &= m - 1;
        const int64_t drow0 = __builtin_amdgcn_readlane(d, j0);
        const float pr0 = load_prob(mprobs, t * E + eb + j0, pdt);
        const unsigned char* fin0 = fwd_in + drow0 * row_bytes;
        unsigned char* gp0 = grad_perm + drow0 * row_bytes;
        float dot0 = 0.f;
        for (int64_t c = lane; c < row_chunks; c += 64) {
          const float fg = Elem<DT>::load(g, c);
          Elem<DT>::store(gp0, c, fg * pr0);
          dot0 = fmaf(Elem<DT>::load(fin0, c), fg, dot0);
        }
        dot0 = wave_sum_f32(dot0);
        if (lane == j0) mine = dot0;
      }
    }
    if (e < E) store_prob(grad_probs, t * E + e, pdt, mine);
  }
}

// acc[sorted_indices[r]] += permuted[r] * pp[r]   (fp32 atomics)
template <int DT>
__global__ __launch_bounds__(kRowThreads) void scatter_add_rows_kernel(
    const void* permuted, int64_t n_rows, int64_t H, const long long* sorted_indices,
    const void* pprobs, int pdt, int64_t T, float* acc) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (kRowThreads / 64) + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  const long long t = sorted_indices[r];
  if (t < 0 || t >= T) return;
  const float pr = pprobs ? load_prob(pprobs, r, pdt) : 1.f;
  for (int64_t h = lane; h < H; h += 64)
    atomicAdd(&acc[t * H + h], Elem<DT>::load(permuted, r * H + h) * pr);
}

template <int DT>
__global__ void cast_rows_kernel(const float* src, int64_t n, void* dst) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) Elem<DT>::store(dst, i, src[i]);
}

// ---- chunk sort ---------------------------------------------------------------------------
// One block computes the chunk -> output offset table in LDS, then wavefronts copy rows.
__global__ __launch_bounds__(kRowThreads) void sort_chunks_map_kernel(
    const long long* split_sizes, const long long* sorted_idxs, int num_splits, int64_t n_rows,
    long long* row_map) {
  // row_map[dst] = src.  Serial prefix sums over the (small) split tables by thread 0, then a
  // block-wide fill; num_splits is at most a few thousand.
  extern __shared__ long long tab[];  // in_off[num_splits+1], out_off[num_splits+1]
  long long* in_off = tab;
  long long* out_off = tab + num_splits + 1;
  // An index outside [0, num_splits) names no chunk: it contributes no rows.  Rows of the output
  // that no chunk covers (the sizes sum to less than n_rows) get -1, which the row mover skips.
  if (threadIdx.x == 0) {
    long long a = 0;
    for (int i = 0; i < num_splits; ++i) {
      in_off[i] = a;
      a += split_sizes[i];
    }
    in_off[num_splits] = a;
    long long b = 0;
    for (int i = 0; i < num_splits; ++i) {
      out_off[i] = b;
      const long long j = sorted_idxs[i];
      b += (j >= 0 && j < num_splits) ? split_sizes[j] : 0;
    }
    out_off[num_splits] = b;
  }
  __syncthreads();
  const long long tid0 = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (int i = 0; i < num_splits; ++i) {
    const long long j = sorted_idxs[i];
    if (j < 0 || j >= num_splits) continue;
    const long long src0 = in_off[j];
    const long long len = out_off[i + 1] - out_off[i];
    const long long dst0 = out_off[i];
    for (long long r = tid0; r < len; r += stride)
      if (dst0 + r < n_rows) row_map[dst0 + r] = src0 + r < n_rows ? src0 + r : -1;
  }
  for (long long r = out_off[num_splits] + tid0; r < n_rows; r += stride) row_map[r] = -1;
}

// out[dst] = inp[row_map[dst]] (GATHER) or out[row_map[src]] = inp[src] (!GATHER)
template <bool GATHER>
__global__ __launch_bounds__(kRowThreads) void move_rows_by_map_kernel(
    const unsigned char* inp, int64_t n_rows, int64_t row_bytes, const long long* row_map,
    unsigned char* out) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (kRowThreads / 64) + (threadIdx.x >> 6);
  if (r >= n_rows) return;
  const long long o = row_map[r];
  if (o < 0 || o >= n_rows) return;
  const unsigned char* s = inp + (GATHER ? o : r) * row_bytes;
  unsigned char* d = out + (GATHER ? r : o) * row_bytes;
  if ((row_bytes & 15) == 0) {
    for (int64_t c = lane; c < row_bytes / 16; c += 64) st16(d + c * 16, ld16(s + c * 16));
  } else {
    for (int64_t c = lane; c < row_bytes / 2; c += 64)
      reinterpret_cast<uint16_t*>(d)[c] = reinterpret_cast<const uint16_t*>(s)[c];
  }
}

static inline int dtype_bytes(int dt) {
  switch (dt) {
    case GMOE_F32: return 4;
    case GMOE_BF16:
    case GMOE_F16: return 2;
    default: return 0;
  }
}
static inline bool prob_dtype_ok(int dt) { return dt == GMOE_F32 || dt == GMOE_BF16 || dt == GMOE_F16; }

}  // namespace gmoe

using namespace gmoe;

extern "C" int64_t gmoe_permute_plan_workspace_bytes(int64_t T, int E) {
  const int64_t NC = (T + kChunkTokens - 1) / kChunkTokens;
  return 2 * (int64_t)E * (NC > 0 ? NC : 1) * (int64_t)sizeof(int);
}

// Argument checks and the three plan launches; counts / base are E * max(NC, 1) ints each.
static int permute_plan_launch(const uint8_t* routing_map, int64_t T, int E, int64_t capacity,
                               int32_t* dst_map, int64_t* sorted_indices, int64_t sorted_cap,
                               int64_t* row_id_map, int64_t* tokens_per_expert,
                               int64_t* expert_offsets, int* counts, int* base, hipStream_t st) {
  const int NC = (int)((T + kChunkTokens - 1) / kChunkTokens);
  const int vec8 = ((E & 7) == 0 && gmoe_aligned(routing_map, 8)) ? 1 : 0;
  if (NC > 0)
    hipLaunchKernelGGL(plan_count_kernel, dim3(NC), dim3(kChunkTokens), (size_t)E * 4 * sizeof(int),
                       st, routing_map, T, E, NC, vec8, counts);
  hipLaunchKernelGGL(plan_scan_kernel, dim3(1), dim3(kScanThreads), 0, st, counts, E, NC, capacity,
                     base, reinterpret_cast<long long*>(tokens_per_expert),
                     reinterpret_cast<long long*>(expert_offsets));
  if (NC > 0)
    hipLaunchKernelGGL(plan_fill_kernel, dim3(NC, (E + kFillExperts - 1) / kFillExperts),
                       dim3(kChunkTokens), 0, st, routing_map, T, E, NC,
                       vec8, capacity, base, dst_map, reinterpret_cast<long long*>(sorted_indices),
                       sorted_cap, reinterpret_cast<long long*>(row_id_map));
  return gmoe_launch_status();
}

static int permute_plan_check(const uint8_t* routing_map, int64_t T, int E, int32_t* dst_map,
                              int64_t sorted_cap, int64_t* tokens_per_expert,
                              int64_t* expert_offsets) {
  GMOE_CHECK_ARG(T >= 0 && E >= 1 && tokens_per_expert && expert_offsets);
  GMOE_CHECK_ARG(T == 0 || (routing_map && dst_map));
  GMOE_CHECK_ARG(T * (int64_t)E < (1ll << 31));  // destination rows are int32
  GMOE_CHECK_ARG(sorted_cap >= 0 && sorted_cap < (1ll << 31));
  if ((size_t)E * 32 > 64 * 1024) return GMOE_ERR_UNSUPPORTED;
  return GMOE_OK;
}

extern "C" int gmoe_permute_plan(const uint8_t* routing_map, int64_t T, int E, int64_t capacity,
                                 int32_t* dst_map, int64_t* sorted_indices, int64_t sorted_cap,
                                 int64_t* row_id_map, int64_t* tokens_per_expert,
                                 int64_t* expert_offsets, void* workspace, void* stream) {
  GMOE_CHECK_ARG(workspace != nullptr);
  const int rc = permute_plan_check(routing_map, T, E, dst_map, sorted_cap, tokens_per_expert,
                                    expert_offsets);
  if (rc != GMOE_OK) return rc;
  const int64_t NC = (T + kChunkTokens - 1) / kChunkTokens;
  int* counts = static_cast<int*>(workspace);
  int* base = counts + (int64_t)E * (NC > 0 ? NC : 1);
  return permute_plan_launch(routing_map, T, E, capacity, dst_map, sorted_indices, sorted_cap,
                             row_id_map, tokens_per_expert, expert_offsets, counts, base,
                             static_cast<hipStream_t>(stream));
}

// ---- the plan without a workspace argument ------------------------------------------------------
// The chunk counts and their prefix live in a device array of the library itself, for callers that
// cannot allocate.  Every GPU holds its own copy of the array at its own address: the address is
// looked up once per device (with that device current) and kept; host code only ever uses that
// pointer, never the array's name.
constexpr int64_t kPlanStaticSlots = 65536;  // E * ceil(T / 256) at most
static __device__ __align__(256) int scratch[2 * kPlanStaticSlots];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static int* g_scratch_ptr[kMaxDevices];  // per device; nullptr until looked up

// Device pointer of `scratch` on the current device, or nullptr on an error.
static int* plan_scratch_for_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    int* ptr = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

extern "C" int64_t gmoe_permute_plan_static_max_slots(void) { return kPlanStaticSlots; }

extern "C" int gmoe_permute_plan_static(const uint8_t* routing_map, int64_t T, int E,
                                        int64_t capacity, int32_t* dst_map,
                                        int64_t* sorted_indices, int64_t sorted_cap,
                                        int64_t* row_id_map, int64_t* tokens_per_expert,
                                        int64_t* expert_offsets, void* stream) {
  const int rc = permute_plan_check(routing_map, T, E, dst_map, sorted_cap, tokens_per_expert,
                                    expert_offsets);
  if (rc != GMOE_OK) return rc;
  const int64_t NC = (T + kChunkTokens - 1) / kChunkTokens;
  const int64_t slots = (int64_t)E * (NC > 0 ? NC : 1);
  if (slots > kPlanStaticSlots) return GMOE_ERR_TOO_LARGE;
  int* ptr = plan_scratch_for_current_device();
  if (ptr == nullptr) return GMOE_ERR_LAUNCH;
  // Nothing in the array has to start at zero: the count pass writes all E * NC counts before the
  // scan reads them, and the scan writes every prefix the fill pass reads.
  return permute_plan_launch(routing_map, T, E, capacity, dst_map, sorted_indices, sorted_cap,
                             row_id_map, tokens_per_expert, expert_offsets, ptr, ptr + slots,
                             static_cast<hipStream_t>(stream));
}

extern "C" int gmoe_permute_rows(const void* tokens, int dtype, int64_t T, int64_t H, int E,
                                 const int32_t* dst_map, int64_t n_out, void* permuted,
                                 const void* probs, int probs_dtype, void* permuted_probs,
                                 void* stream) {
  const int es = dtype_bytes(dtype);
  GMOE_CHECK_ARG(es != 0 && T >= 0 && H >= 1 && E >= 1 && n_out >= 0);
  GMOE_CHECK_ARG(permuted_probs == nullptr || (probs != nullptr && prob_dtype_ok(probs_dtype)));
  if (T == 0 || n_out == 0) return GMOE_OK;
  GMOE_CHECK_ARG(tokens && dst_map && permuted);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((T + 3) / 4)), block(kRowThreads);
  const int64_t row_bytes = H * es;
  if ((row_bytes & 15) == 0 && gmoe_aligned(tokens, 16) && gmoe_aligned(permuted, 16)) {
    hipLaunchKernelGGL(permute_rows_kernel, grid, block, 0, st,
                       static_cast<const unsigned char*>(tokens), T, row_bytes / 16, E, dst_map,
                       n_out, static_cast<unsigned char*>(permuted), probs, probs_dtype,
                       permuted_probs);
  } else {
    hipLaunchKernelGGL(permute_rows_generic_kernel, grid, block, 0, st,
                       static_cast<const unsigned char*>(tokens), T, H, es, E, dst_map, n_out,
                       static_cast<unsigned char*>(permuted), probs, probs_dtype, permuted_probs);
  }
  return gmoe_launch_status();
}

template <int DT>
static void launch_unpermute(bool vec, dim3 grid, hipStream_t st, const void* permuted, int64_t T,
                             int64_t H, int E, const int32_t* dst_map, int64_t n_out,
                             const void* mp, int pdt, void* out, const void* ppin, void* upout,
                             const void* addend, const void* residual) {
  const unsigned char* ad = static_cast<const unsigned char*>(addend);
  const unsigned char* rs = static_cast<const unsigned char*>(residual);
  auto kern = vec ? ((ad || rs) ? unpermute_rows_kernel<DT, true, true> : unpermute_rows_kernel<DT, true, false>)
                  : unpermute_rows_kernel<DT, false, true>;
  hipLaunchKernelGGL(kern, grid, dim3(kRowThreads), 0, st, static_cast<const unsigned char*>(permuted),
                     T, H, E, dst_map, n_out, mp, pdt, static_cast<unsigned char*>(out), ppin, upout,
                     ad, rs);
}

extern "C" int gmoe_unpermute_rows(const void* permuted, int dtype, int64_t T, int64_t H, int E,
                                   const int32_t* dst_map, int64_t n_out, const void* merging_probs,
                                   int probs_dtype, void* out, const void* permuted_probs_in,
                                   void* unpermuted_probs, const void* addend, const void* residual,
                                   void* stream) {
  const int es = dtype_bytes(dtype);
  GMOE_CHECK_ARG(es != 0 && T >= 0 && H >= 1 && E >= 1 && n_out >= 0);
  GMOE_CHECK_ARG((merging_probs == nullptr && unpermuted_probs == nullptr) ||
                 prob_dtype_ok(probs_dtype));
  GMOE_CHECK_ARG(unpermuted_probs == nullptr || permuted_probs_in != nullptr || n_out == 0);
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(dst_map && out && (permuted || n_out == 0));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((T + 3) / 4));
  const bool vec = ((H * es) & 15) == 0 && gmoe_aligned(permuted, 16) && gmoe_aligned(out, 16) &&
                   gmoe_aligned(addend, 16) && gmoe_aligned(residual, 16);
  switch (dtype) {
    case GMOE_F32:
      launch_unpermute<GMOE_F32>(vec, grid, st, permuted, T, H, E, dst_map, n_out, merging_probs,
                                 probs_dtype, out, permuted_probs_in, unpermuted_probs, addend, residual);
      break;
    case GMOE_BF16:
      launch_unpermute<GMOE_BF16>(vec, grid, st, permuted, T, H, E, dst_map, n_out, merging_probs,
                                  probs_dtype, out, permuted_probs_in, unpermuted_probs, addend, residual);
      break;
    case GMOE_F16:
      launch_unpermute<GMOE_F16>(vec, grid, st, permuted, T, H, E, dst_map, n_out, merging_probs,
                                 probs_dtype, out, permuted_probs_in, unpermuted_probs, addend, residual);
      break;
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}

template <int DT>
static void launch_unpermute_bwd(bool vec, dim3 grid, hipStream_t st, const void* go,
                                 const void* fin, int64_t T, int64_t H, int E,
                                 const int32_t* dst_map, int64_t n_out, const void* mp, int pdt,
                                 void* gp, void* gprobs) {
  if (vec)
    hipLaunchKernelGGL((unpermute_rows_bwd_kernel<DT, true>), grid, dim3(kRowThreads), 0, st,
                       static_cast<const unsigned char*>(go), static_cast<const unsigned char*>(fin),
                       T, H, E, dst_map, n_out, mp, pdt, static_cast<unsigned char*>(gp), gprobs);
  else
    hipLaunchKernelGGL((unpermute_rows_bwd_kernel<DT, false>), grid, dim3(kRowThreads), 0, st,
                       static_cast<const unsigned char*>(go), static_cast<const unsigned char*>(fin),
                       T, H, E, dst_map, n_out, mp, pdt, static_cast<unsigned char*>(gp), gprobs);
}

extern "C" int gmoe_unpermute_rows_bwd(const void* grad_out, const void* fwd_input, int dtype,
                                       int64_t T, int64_t H, int E, const int32_t* dst_map,
                                       int64_t n_out, const void* merging_probs, int probs_dtype,
                                       void* grad_permuted, void* grad_probs, void* stream) {
  const int es = dtype_bytes(dtype);
  GMOE_CHECK_ARG(es != 0 && T >= 0 && H >= 1 && E >= 1 && n_out >= 0);
  GMOE_CHECK_ARG(prob_dtype_ok(probs_dtype));
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(grad_out && dst_map && merging_probs && grad_probs);
  GMOE_CHECK_ARG(n_out == 0 || (fwd_input && grad_permuted));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((T + 3) / 4));
  const bool vec = ((H * es) & 15) == 0 && gmoe_aligned(grad_out, 16) &&
                   gmoe_aligned(fwd_input, 16) && gmoe_aligned(grad_permuted, 16);
  switch (dtype) {
    case GMOE_F32:
      launch_unpermute_bwd<GMOE_F32>(vec, grid, st, grad_out, fwd_input, T, H, E, dst_map, n_out,
                                     merging_probs, probs_dtype, grad_permuted, grad_probs);
      break;
    case GMOE_BF16:
      launch_unpermute_bwd<GMOE_BF16>(vec, grid, st, grad_out, fwd_input, T, H, E, dst_map, n_out,
                                      merging_probs, probs_dtype, grad_permuted, grad_probs);
      break;
    case GMOE_F16:
      launch_unpermute_bwd<GMOE_F16>(vec, grid, st, grad_out, fwd_input, T, H, E, dst_map, n_out,
                                     merging_probs, probs_dtype, grad_permuted, grad_probs);
      break;
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}

extern "C" int gmoe_scatter_add_rows(const void* permuted, int dtype, int64_t n_rows, int64_t H,
                                     const int64_t* sorted_indices, const void* permuted_probs,
                                     int probs_dtype, int64_t T, float* acc, void* stream) {
  GMOE_CHECK_ARG(dtype_bytes(dtype) != 0 && n_rows >= 0 && H >= 1 && T >= 0);
  GMOE_CHECK_ARG(permuted_probs == nullptr || prob_dtype_ok(probs_dtype));
  if (n_rows == 0) return GMOE_OK;
  GMOE_CHECK_ARG(permuted && sorted_indices && acc);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((n_rows + 3) / 4)), block(kRowThreads);
  const long long* si = reinterpret_cast<const long long*>(sorted_indices);
  switch (dtype) {
    case GMOE_F32:
      hipLaunchKernelGGL((scatter_add_rows_kernel<GMOE_F32>), grid, block, 0, st, permuted, n_rows, H,
                         si, permuted_probs, probs_dtype, T, acc);
      break;
    case GMOE_BF16:
      hipLaunchKernelGGL((scatter_add_rows_kernel<GMOE_BF16>), grid, block, 0, st, permuted, n_rows,
                         H, si, permuted_probs, probs_dtype, T, acc);
      break;
    case GMOE_F16:
      hipLaunchKernelGGL((scatter_add_rows_kernel<GMOE_F16>), grid, block, 0, st, permuted, n_rows, H,
                         si, permuted_probs, probs_dtype, T, acc);
      break;
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
  return gmoe_launch_status();
}

extern "C" int gmoe_cast_rows(const float* src, int64_t n_elems, int dst_dtype, void* dst,
                              void* stream) {
  GMOE_CHECK_ARG(n_elems >= 0 && dtype_bytes(dst_dtype) != 0);
  if (n_elems == 0) return GMOE_OK;
  GMOE_CHECK_ARG(src && dst);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((n_elems + 255) / 256)), block(256);
  switch (dst_dtype) {
    case GMOE_F32:
      hipLaunchKernelGGL((cast_rows_kernel<GMOE_F32>), grid, block, 0, st, src, n_elems, dst);
      break;
    case GMOE_BF16:
      hipLaunchKernelGGL((cast_rows_kernel<GMOE_BF16>), grid, block, 0, st, src, n_elems, dst);
      break;
    default:
      hipLaunchKernelGGL((cast_rows_kernel<GMOE_F16>), grid, block, 0, st, src, n_elems, dst);
      break;
  }
  return gmoe_launch_status();
}

extern "C" int gmoe_sort_chunks(const void* inp, int dtype, int64_t n_rows, int64_t H,
                                const int64_t* split_sizes, const int64_t* sorted_idxs,
                                int num_splits, void* out, int64_t* row_map, void* stream) {
  const int es = dtype_bytes(dtype);
  GMOE_CHECK_ARG(es != 0 && n_rows >= 0 && H >= 1 && num_splits >= 1);
  GMOE_CHECK_ARG(split_sizes && sorted_idxs && row_map);
  if ((size_t)(num_splits + 1) * 16 > 60 * 1024) return GMOE_ERR_UNSUPPORTED;
  if (n_rows == 0) return GMOE_OK;
  GMOE_CHECK_ARG(inp && out);
  GMOE_CHECK_ARG(((H * es) & 1) == 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(sort_chunks_map_kernel, dim3(64), dim3(kRowThreads),
                     (size_t)(num_splits + 1) * 2 * sizeof(long long), st,
                     reinterpret_cast<const long long*>(split_sizes),
                     reinterpret_cast<const long long*>(sorted_idxs), num_splits, n_rows,
                     reinterpret_cast<long long*>(row_map));
  hipLaunchKernelGGL((move_rows_by_map_kernel<true>), dim3((unsigned)((n_rows + 3) / 4)),
                     dim3(kRowThreads), 0, st, static_cast<const unsigned char*>(inp), n_rows,
                     H * es, reinterpret_cast<const long long*>(row_map),
                     static_cast<unsigned char*>(out));
  return gmoe_launch_status();
}

extern "C" int gmoe_scatter_rows_by_map(const void* inp, int dtype, int64_t n_rows, int64_t H,
                                        const int64_t* row_map, void* out, void* stream) {
  const int es = dtype_bytes(dtype);
  GMOE_CHECK_ARG(es != 0 && n_rows >= 0 && H >= 1);
  if (n_rows == 0) return GMOE_OK;
  GMOE_CHECK_ARG(inp && out && row_map);
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL((move_rows_by_map_kernel<false>), dim3((unsigned)((n_rows + 3) / 4)),
                     dim3(kRowThreads), 0, st, static_cast<const unsigned char*>(inp), n_rows,
                     H * es, reinterpret_cast<const long long*>(row_map),
                     static_cast<unsigned char*>(out));
  return gmoe_launch_status();
}
