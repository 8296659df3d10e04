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
  // fused gated-activation epilogues (see gmoe_gmm_glu / gmoe_gmm_glu_bwd)
  unsigned char* c2;         // forward: activated output [N,F]
  const unsigned char* aux;  // backward: fc1 [N,2F]
  const unsigned char* b_scale;  // fp8 weights: bf16 block scales
  const unsigned char* a_scale;  // fp8 activations: power-of-two row scales, dwords [K/128][N]
  int row_part;              // NN / NT: which rows of every expert this launch covers (ROWS_*)
  int64_t F;
  // split reduction of a launch with few tiles (see SPLIT_* in gmm.hip): fp32 partial tiles
  float* ws;
  int64_t ws_floats;
  int split_slots;           // tiles x splits this launch may spread over; 0 = never split
  int phase;                 // SPLIT_OFF, SPLIT_PARTIAL, SPLIT_REDUCE
  int main_grid;             // ROWS_AUTO_*: workgroups of the launch with 256-row tiles
};
// First row of group e.  A null offset table means one group holding all N rows (dense GEMM on the
// grouped kernels: the gate projection of large expert counts).
__device__ __forceinline__ long long group_begin(const GmmParams& p, int e) {
  return p.offsets ? p.offsets[e] : (e > 0 ? (long long)p.N : 0ll);
}
enum { SPLIT_OFF = 0, SPLIT_PARTIAL = 1, SPLIT_REDUCE = 2 };
constexpr int kMaxSplit = 8;

// A launch with 256-row tiles leaves an expert's last n % 256 rows, when they are at most kRemRows,
// to a second launch with 128-row tiles: a tile that is almost empty costs as much as a full one,
// and with near-uniform routing those tiles alone add a whole round of the persistent grid.
// ROWS_AUTO_*: the pair of launches decides on the device, from the tile counts, whether the split
// into ROWS_MAIN + ROWS_REMAINDER pays (resolve_row_part in gmm.hip); if not, the AUTO_MAIN launch
// takes all rows and the AUTO_REMAINDER launch exits.
enum { ROWS_ALL = 0, ROWS_MAIN = 1, ROWS_REMAINDER = 2, ROWS_AUTO_MAIN = 3, ROWS_AUTO_REMAINDER = 4,
       ROWS_NONE = 5 };
constexpr int kRemRows = 128;
// Workgroups the split remainder launch spreads over: two per CU.
constexpr int kSplitSlots = 512;
// rows [begin, begin + count) of an expert with n rows that belong to `part`
__device__ __forceinline__ void expert_row_part(long long n, int part, long long& begin,
                                                long long& count) {
  const long long full = n / 256 * 256, rem = n - full;
  const bool split = rem > 0 && rem <= kRemRows;
  begin = (part == ROWS_REMAINDER && split) ? full : 0;
  count = part == ROWS_ALL ? n : (part == ROWS_MAIN ? (split ? full : n) : (split ? rem : 0));
}

// TN: rows of an expert one buffer resource may span (both operands, row pitch K and M elements),
// a multiple of every kernel's K tile.
__host__ __device__ __forceinline__ int64_t tn_segment_rows(int64_t K, int64_t M, int es) {
  const int64_t pitch = (K > M ? K : M) * es;
  const int64_t rows = (0x7fffffffll - 1024) / pitch;
  return rows < 64 ? 64 : rows / 64 * 64;
}

enum { EPI_NONE = 0, EPI_GLU_FWD_SILU = 1, EPI_GLU_FWD_GELU = 2, EPI_GLU_BWD_SILU = 3, EPI_GLU_BWD_GELU = 4 };

// pack 4 fp32 into 4 16-bit values of type DT
template <int DT>
__device__ __forceinline__ u32x2 pack4(float v0, float v1, float v2, float v3) {
  u32x2 o;
  if (DT == GMOE_BF16) {
    o[0] = pack_bf16x2(v0, v1);
    o[1] = pack_bf16x2(v2, v3);
  } else {
    o[0] = pack_f16x2(v0, v1);
    o[1] = pack_f16x2(v2, v3);
  }
  return o;
}
template <int DT>
__device__ __forceinline__ void unpack4(const u32x2& w, float* f) {
  if (DT == GMOE_BF16) {
    f[0] = __uint_as_float(w[0] << 16); f[1] = __uint_as_float(w[0] & 0xffff0000u);
    f[2] = __uint_as_float(w[1] << 16); f[3] = __uint_as_float(w[1] & 0xffff0000u);
  } else {
    f[0] = f16_bits_to_f32(w[0] & 0xffffu); f[1] = f16_bits_to_f32(w[0] >> 16);
    f[2] = f16_bits_to_f32(w[1] & 0xffffu); f[3] = f16_bits_to_f32(w[1] >> 16);
  }
}

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

// Epilogue staging: this wavefront's accumulators, rounded to the 16-bit type ODT, go into an LDS
// tile [rows][BN] whose row pitch of BN*2+8 bytes puts the 32 rows one store instruction touches
// on distinct banks.  After a barrier the tile is read back row-contiguously, so global memory
// sees 16-byte accesses that cover whole 128-byte lines.
template <int BN>
struct CTile {
  static constexpr int pitch = BN * 2 + 8;
  static constexpr int chunks = BN / 8;                 // 16-byte chunks per row
  static constexpr int rows_per_pass = kGemmThreads / chunks;
};
template <int ODT, int WTM, int WTN, int BN>
__device__ __forceinline__ void stage_acc_lds(unsigned char* lds, const f32x16 (&acc)[WTM][WTN],
                                              int row_base, int col_base, int lane) {
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int j = 0; j < WTN; ++j)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const int row = row_base + i * 32 + (lane & 31);
        const int col = col_base + j * 32 + 8 * vq + 4 * (lane >> 5);
        *reinterpret_cast<u32x2*>(lds + row * CTile<BN>::pitch + col * 2) =
            pack4<ODT>(acc[i][j][4 * vq], acc[i][j][4 * vq + 1], acc[i][j][4 * vq + 2],
                       acc[i][j][4 * vq + 3]);
      }
}
// 16 bytes of a staged row (8-byte aligned only)
__device__ __forceinline__ u32x4 ctile_read16(const unsigned char* p) {
  const u32x2 lo = *reinterpret_cast<const u32x2*>(p);
  const u32x2 hi = *reinterpret_cast<const u32x2*>(p + 8);
  return u32x4{lo[0], lo[1], hi[0], hi[1]};
}

// ---- LDS-DMA copies (gmm_dtl.hip, gmm_fp8s.hip) ---------------------------------------------------
typedef __attribute__((address_space(3))) unsigned char lds_byte;

__device__ __forceinline__ uint32_t lds_offset_of(const void* p) {
  return (uint32_t)(uintptr_t)(lds_byte*)(p);
}

// One LDS-DMA instruction: lane L copies 16 bytes from rsrc[voff + soff] to LDS[lds_base + 16*L].
__device__ __forceinline__ void dma16(uint32_t lds_base, uint32_t voff, const u32x4& rsrc,
                                      uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_dma_outstanding() {
  // at most N of this wavefront's copies may still be in flight
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ u32x4 make_raw_rsrc(const void* base, int64_t bytes) {
  const uint64_t a = (uint64_t)(uintptr_t)base;
  const uint32_t n = bytes <= 0 ? 0u : (bytes > 0x7fffffffll ? 0x7fffffffu : (uint32_t)bytes);
  u32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
  r[2] = __builtin_amdgcn_readfirstlane(n);
  r[3] = 0x00020000u;
  return r;
}

// ---- fp8 (e4m3) weights with one bf16 scale per 128x128 block (gmm.hip, gmm_fp8s.hip) --------------
// Two fp8 values (the low or the high half of w) as two bf16 in one instruction: the scaled
// conversion with a scale of one.  Every e4m3 value, the denormal codes included, is a bf16 value,
// so the result is exact; through fp32 the pair takes two instructions.
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t w, bool hi) {
  return hi ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true))
            : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
}
struct Fp8Scale {
  const uint16_t* ptr;  // scale of K block 0 for this tile
  int stride;           // elements between consecutive K blocks
  int last;             // index of the last K block
  __device__ __forceinline__ float at(int kt) const {
    int kb = kt >> 1;   // 64-element K tiles, 128-element blocks
    kb = kb > last ? last : kb;
    return bf16_bits_to_f32(ptr[(int64_t)kb * stride]);
  }
};

// Launches the LDS-DMA variant (gmm_dtl.hip) of the dW product (TN) for 16-bit operands.
int launch_gmm_dtl_tn(const GmmParams& p, int dtype, int out_dtype, hipStream_t st);

// Launches the weight-stationary kernel for fp8 weights and few rows per expert (gmm_fp8s.hip);
// whether it applies: gmm_fp8_skinny_applies.
int launch_gmm_fp8_skinny(const GmmParams& p, bool trans_b, hipStream_t st);
bool gmm_fp8_skinny_applies(const GmmParams& p, bool any_row_count = false);

// One dense product on the grouped kernels (gmm.hip): a single group of all N rows, no offset
// table.  mode MODE_NN: c [N,M] = a [N,K] @ b [K,M]; MODE_NT: c = a @ b^T with b [M,K]; MODE_TN:
// c [K,M] = a^T @ b with a [N,K], b [N,M].  K and M multiples of 8.
// ws / ws_floats: optional fp32 workspace of gmm_dense_workspace_floats(N, K, M, mode) floats; with
// it an NN / NT product with few output tiles and a long reduction is split over the idle CUs.
int gmm_dense(const void* a, const void* b, void* c, int64_t N, int64_t K, int64_t M, int mode,
              int dtype, int out_dtype, hipStream_t st, float* ws = nullptr, int64_t ws_floats = 0);
int64_t gmm_dense_workspace_floats(int64_t N, int64_t K, int64_t M, int mode);

// c [groups][K,M] = a_g^T @ b_g over the row ranges [offsets[g], offsets[g+1]) of a [N,K] and
// b [N,M] (offsets: groups + 1 device values): the grouped weight-gradient product, also used to cut
// one long reduction into `groups` partial products.
int gmm_grouped_tn(const void* a, const void* b, void* c, const int64_t* offsets, int groups, int64_t N,
                   int64_t K, int64_t M, int dtype, int out_dtype, hipStream_t st);

}  // namespace gmoe
