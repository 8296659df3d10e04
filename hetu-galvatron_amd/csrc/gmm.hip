// Grouped GEMM for gfx950 (CDNA4): one persistent kernel over a device-side expert-offset table.
// Replaces `grouped_gemm.ops.gmm` (call sites moe/mlp.py:106-112) and its backward.
//
//   NN  c[rows_e]  = a[rows_e] @ b[e]        a [N,K]  b [E,K,M]  c [N,M]    (forward)
//   NT  c[rows_e]  = a[rows_e] @ b[e]^T      a [N,K]  b [E,M,K]  c [N,M]    (dX)
//   TN  c[e]       = a[rows_e]^T @ b[rows_e] a [N,K]  b [N,M]    c [E,K,M]  (dW)
//
// Structure
//   * 256 threads = 4 wavefronts in a 2x2 grid; the block owns a BM x BN tile of C, each wavefront
//     a (BM/2) x (BN/2) sub-tile made of 32x32 MFMA accumulators (fp32).
//   * Operand tiles are staged through LDS in the layout [outer index][BK reduction elements], 128
//     bytes of data per row padded to 144 so that the 16-byte fragment reads of 16 consecutive rows
//     hit disjoint banks.  Two LDS stages; the global loads of tile kt+1 are issued before the MFMAs
//     of tile kt and written to the other stage afterwards (one barrier per K step).
//   * An operand whose reduction index is contiguous in memory is copied as is.  One whose
//     reduction index is the slow dimension (b in NN, both in TN) is loaded as 8x8 (16-bit) or 4x4
//     (fp32) blocks and transposed in registers (v_perm_b32) on its way to LDS, so the MFMA side
//     never sees the difference.
//   * The MFMA is issued with the operands swapped (B fragment as SrcA) so that a lane ends up with
//     4 consecutive columns of one row of C: 8-byte (16-bit) / 16-byte (fp32) stores.
//   * Tiles are numbered expert-major, inside an expert in strips of 8 column tiles, and handed to
//     workgroups so that the 32 workgroups that share an XCD (workgroup id mod 8) work on one
//     4x8 patch of tiles at a time: the A and B panels they stream are shared in that XCD's L2.
#include "gmoe_common.h"

namespace gmoe {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

enum { MODE_NN = 0, MODE_NT = 1, MODE_TN = 2 };

constexpr int kGemmThreads = 256;
constexpr int kRowPad = 144;   // bytes per LDS row: 128 data + 16 pad
constexpr int kStripTiles = 8; // column tiles per strip
constexpr int kMaxGroupsLds = 1024;

template <int DT>
struct Mma;
template <>
struct Mma<GMOE_BF16> {
  static constexpr int EPC = 8;  // elements per 16-byte chunk
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, f32x16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b),
                                                  __builtin_bit_cast(bf16x8, a), acc, 0, 0, 0);
  }
};
template <>
struct Mma<GMOE_F16> {
  static constexpr int EPC = 8;
  __device__ static __forceinline__ void run(const u32x4& a, const u32x4& b, f32x16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b),
                                                 __builtin_bit_cast(f16x8, a), acc, 0, 0, 0);
  }
};
template <>
struct Mma<GMOE_F32> {
  static constexpr int EPC = 4;
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
};

// ---- operand loaders ----------------------------------------------------------------------------
// A tile is R "outer" indices x BK reduction elements (128 bytes per outer index).

// Reduction index contiguous in memory: element (o, k) at src + o*ld + k.
template <int R, int ES>
struct DirectLoader {
  static constexpr int EPC = 16 / ES;
  static constexpr int NL = R / 32;  // 16-byte loads per thread
  u32x4 r[NL];
  // thread t covers chunk t%8 of rows t/8 + 32*i
  __device__ __forceinline__ void load(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k0, int64_t k_lim, int tid) {
    const int c = tid & 7, r0 = tid >> 3;
    const int64_t k = k0 + c * EPC;
    const bool kok = k < k_lim;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int64_t o = o0 + r0 + 32 * i;
      if (kok && o < o_lim)
        r[i] = ld16(src + (o * ld + k) * ES);
      else
        r[i] = u32x4{0, 0, 0, 0};
    }
  }
  __device__ __forceinline__ void store(unsigned char* lds, int tid) const {
    const int c = tid & 7, r0 = tid >> 3;
#pragma unroll
    for (int i = 0; i < NL; ++i)
      *reinterpret_cast<u32x4*>(lds + (r0 + 32 * i) * kRowPad + c * 16) = r[i];
  }
};

// Reduction index is the slow dimension: element (o, k) at src + k*ld + o.  Thread t owns the
// EPC x EPC block(s) at reduction block t%8, outer block t/8 (+32 per pass).
template <int R, int ES>
struct TransposeLoader {
  static constexpr int EPC = 16 / ES;
  static constexpr int OB = R / EPC;                   // outer blocks in the tile
  static constexpr int NP = (OB + 31) / 32;            // passes
  u32x4 r[NP][EPC];
  __device__ __forceinline__ void load(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k0, int64_t k_lim, int tid) {
    const int kb = tid & 7, ob0 = tid >> 3;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int ob = ob0 + 32 * p;
      const int64_t o = o0 + (int64_t)ob * EPC;
      const bool ook = ob < OB && o < o_lim;
#pragma unroll
      for (int i = 0; i < EPC; ++i) {
        const int64_t k = k0 + kb * EPC + i;
        if (ook && k < k_lim)
          r[p][i] = ld16(src + (k * ld + o) * ES);
        else
          r[p][i] = u32x4{0, 0, 0, 0};
      }
    }
  }
  __device__ __forceinline__ void store(unsigned char* lds, int tid) const {
    const int kb = tid & 7, ob0 = tid >> 3;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int ob = ob0 + 32 * p;
      if (ob >= OB) continue;
#pragma unroll
      for (int o = 0; o < EPC; ++o) {
        u32x4 v;
        if (ES == 2) {
          // v.dword[q] = (r[2q] element o) | (r[2q+1] element o) << 16
          const uint32_t sel = (o & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            v[q] = __builtin_amdgcn_perm(r[p][2 * q + 1][o >> 1], r[p][2 * q][o >> 1], sel);
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = r[p][q][o];
        }
        *reinterpret_cast<u32x4*>(lds + (ob * EPC + o) * kRowPad + kb * 16) = v;
      }
    }
  }
};

template <int R, int ES, bool TRANSPOSE>
struct Loader : DirectLoader<R, ES> {};
template <int R, int ES>
struct Loader<R, ES, true> : TransposeLoader<R, ES> {};

// ---- tile schedule ------------------------------------------------------------------------------
struct Tile {
  int e;
  int mt, nt;
};

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

// ---- the kernel -----------------------------------------------------------------------------------
template <int DT, int ODT, int MODE, int BM, int BN>
__global__ __launch_bounds__(kGemmThreads) void gmm_kernel(GmmParams p) {
  constexpr int ES = Elem<DT>::bytes;
  constexpr int BK = 128 / ES;       // reduction elements per LDS row
  constexpr int KSTEPS = 4;          // fragment loads per K tile (32 bytes of each row per step)
  constexpr int WTM = BM / 2 / 32;   // 32x32 accumulators per wavefront, rows
  constexpr int WTN = BN / 2 / 32;   // ... columns
  constexpr bool A_T = (MODE == MODE_TN);
  constexpr bool B_T = (MODE != MODE_NT);
  constexpr int A_BYTES = BM * kRowPad;
  constexpr int B_BYTES = BN * kRowPad;
  constexpr int STAGE = A_BYTES + B_BYTES;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  __shared__ long long tile_cum[kMaxGroupsLds + 1];  // exclusive prefix of tiles per expert

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  const int E = p.E;
  const int64_t K = p.K, M = p.M;
  // C is (rows x cols) per expert: NN/NT rows = tokens of the expert, cols = M;  TN rows = K, cols = M
  const int nt_cnt = (int)((M + BN - 1) / BN);
  const int mt_fixed = (int)((K + BM - 1) / BM);  // TN only

  for (int e = tid; e <= E; e += kGemmThreads) {
    // serial prefix per thread would be O(E^2); E is small, and this runs once per workgroup
    long long acc = 0;
    for (int j = 0; j < e; ++j) {
      const long long n = p.offsets[j + 1] - p.offsets[j];
      const long long mt = MODE == MODE_TN ? mt_fixed : (n + BM - 1) / BM;
      acc += mt * nt_cnt;
    }
    tile_cum[e] = acc;
  }
  __syncthreads();
  const long long total_tiles = tile_cum[E];

  // Workgroup w runs on XCD w%8.  Give XCD x the 32 consecutive positions [32x, 32x+32) of every
  // round of gridDim.x tiles (gridDim.x is a multiple of 8).
  const int per_xcd = gridDim.x / 8;
  const long long first = (long long)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;

  int e = 0;
  for (long long s = first; s < total_tiles; s += gridDim.x) {
    while (tile_cum[e + 1] <= s) ++e;
    const long long row0 = p.offsets[e];
    const long long n_e = p.offsets[e + 1] - row0;
    const int mt_cnt = MODE == MODE_TN ? mt_fixed : (int)((n_e + BM - 1) / BM);
    int mt, nt;
    strip_order(s - tile_cum[e], mt_cnt, nt_cnt, mt, nt);

    // Operand views for this tile.
    const unsigned char* a_src;
    const unsigned char* b_src;
    int64_t a_ld, b_ld, a_o0, a_olim, b_o0, b_olim, k_lim;
    if (MODE == MODE_NN) {
      a_src = p.a + row0 * K * ES;  a_ld = K;  a_o0 = (int64_t)mt * BM;  a_olim = n_e;
      b_src = p.b + (int64_t)e * K * M * ES;  b_ld = M;  b_o0 = (int64_t)nt * BN;  b_olim = M;
      k_lim = K;
    } else if (MODE == MODE_NT) {
      a_src = p.a + row0 * K * ES;  a_ld = K;  a_o0 = (int64_t)mt * BM;  a_olim = n_e;
      b_src = p.b + (int64_t)e * M * K * ES;  b_ld = K;  b_o0 = (int64_t)nt * BN;  b_olim = M;
      k_lim = K;
    } else {
      a_src = p.a + row0 * K * ES;  a_ld = K;  a_o0 = (int64_t)mt * BM;  a_olim = K;
      b_src = p.b + row0 * M * ES;  b_ld = M;  b_o0 = (int64_t)nt * BN;  b_olim = M;
      k_lim = n_e;
    }

    f32x16 acc[WTM][WTN];
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WTN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int kt_cnt = (int)((k_lim + BK - 1) / BK);
    Loader<BM, ES, A_T> la;
    Loader<BN, ES, B_T> lb;
    if (kt_cnt > 0) {
      la.load(a_src, a_ld, a_o0, a_olim, 0, k_lim, tid);
      lb.load(b_src, b_ld, b_o0, b_olim, 0, k_lim, tid);
      la.store(lds, tid);
      lb.store(lds + A_BYTES, tid);
    }
    __syncthreads();
    for (int kt = 0; kt < kt_cnt; ++kt) {
      const bool more = kt + 1 < kt_cnt;
      if (more) {
        la.load(a_src, a_ld, a_o0, a_olim, (int64_t)(kt + 1) * BK, k_lim, tid);
        lb.load(b_src, b_ld, b_o0, b_olim, (int64_t)(kt + 1) * BK, k_lim, tid);
      }
      const unsigned char* sa = lds + (kt & 1) * STAGE;
      const unsigned char* sb = sa + A_BYTES;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        u32x4 fa[WTM], fb[WTN];
        const int coff = (ks * 2 + (lane >> 5)) * 16;
#pragma unroll
        for (int i = 0; i < WTM; ++i)
          fa[i] = *reinterpret_cast<const u32x4*>(
              sa + (wm * (BM / 2) + i * 32 + (lane & 31)) * kRowPad + coff);
#pragma unroll
        for (int j = 0; j < WTN; ++j)
          fb[j] = *reinterpret_cast<const u32x4*>(
              sb + (wn * (BN / 2) + j * 32 + (lane & 31)) * kRowPad + coff);
#pragma unroll
        for (int i = 0; i < WTM; ++i)
#pragma unroll
          for (int j = 0; j < WTN; ++j) Mma<DT>::run(fa[i], fb[j], acc[i][j]);
      }
      if (more) {
        unsigned char* da = lds + ((kt + 1) & 1) * STAGE;
        la.store(da, tid);
        lb.store(da + A_BYTES, tid);
      }
      __syncthreads();
    }

    // ---- epilogue: lane holds row (lane%32), columns 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 ----
    constexpr int OES = Elem<ODT>::bytes;
    unsigned char* c_base;
    int64_t c_rows;
    if (MODE == MODE_TN) {
      c_base = p.c + (int64_t)e * K * M * OES;
      c_rows = K;
    } else {
      c_base = p.c + row0 * M * OES;
      c_rows = n_e;
    }
#pragma unroll
    for (int i = 0; i < WTM; ++i) {
      const int64_t m = (int64_t)mt * BM + wm * (BM / 2) + i * 32 + (lane & 31);
      if (m >= c_rows) continue;
#pragma unroll
      for (int j = 0; j < WTN; ++j) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int64_t n = (int64_t)nt * BN + wn * (BN / 2) + j * 32 + 8 * vq + 4 * (lane >> 5);
          if (n >= M) continue;
          unsigned char* dst = c_base + (m * M + n) * OES;
          const float v0 = acc[i][j][4 * vq], v1 = acc[i][j][4 * vq + 1];
          const float v2 = acc[i][j][4 * vq + 2], v3 = acc[i][j][4 * vq + 3];
          if (ODT == GMOE_F32) {
            *reinterpret_cast<f32x4*>(dst) = f32x4{v0, v1, v2, v3};
          } else if (ODT == GMOE_BF16) {
            u32x2 o;
            o[0] = pack_bf16x2(v0, v1);
            o[1] = pack_bf16x2(v2, v3);
            *reinterpret_cast<u32x2*>(dst) = o;
          } else {
            u32x2 o;
            o[0] = pack_f16x2(v0, v1);
            o[1] = pack_f16x2(v2, v3);
            *reinterpret_cast<u32x2*>(dst) = o;
          }
        }
      }
    }
  }
}

template <int DT, int ODT, int MODE, int BM, int BN>
static int launch_gmm_cfg(const GmmParams& p, hipStream_t st) {
  constexpr size_t smem = 2 * (size_t)(BM + BN) * kRowPad;
  auto kern = gmm_kernel<DT, ODT, MODE, BM, BN>;
  if (smem > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return GMOE_ERR_LAUNCH;
  }
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      cus = v;
  }
  int grid = (cus / 8) * 8;
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kGemmThreads), smem, st, p);
  return gmoe_launch_status();
}

template <int DT, int ODT, int MODE>
static int launch_gmm_mode(const GmmParams& p, hipStream_t st) {
  // Large tiles once an expert's share of rows (NN/NT) or the output itself (TN) can fill them.
  const int64_t rows_per_expert = MODE == MODE_TN ? p.K : (p.N / (p.E > 0 ? p.E : 1));
  if (rows_per_expert >= 512 && p.M >= 256)
    return launch_gmm_cfg<DT, ODT, MODE, 256, 256>(p, st);
  return launch_gmm_cfg<DT, ODT, MODE, 128, 128>(p, st);
}

template <int DT, int ODT>
static int launch_gmm(const GmmParams& p, int mode, hipStream_t st) {
  switch (mode) {
    case MODE_NN: return launch_gmm_mode<DT, ODT, MODE_NN>(p, st);
    case MODE_NT: return launch_gmm_mode<DT, ODT, MODE_NT>(p, st);
    default: return launch_gmm_mode<DT, ODT, MODE_TN>(p, st);
  }
}

}  // namespace gmoe

using namespace gmoe;

extern "C" int gmoe_gmm(const void* a, const void* b, void* c, const int64_t* expert_offsets, int E,
                        int64_t N, int64_t K, int64_t M, int trans_a, int trans_b, int dtype,
                        int out_dtype, void* stream) {
  GMOE_CHECK_ARG(E >= 1 && N >= 0 && K >= 1 && M >= 1 && expert_offsets);
  GMOE_CHECK_ARG(!(trans_a && trans_b));
  GMOE_CHECK_ARG(c != nullptr && b != nullptr && (a != nullptr || N == 0));
  if (E > kMaxGroupsLds) return GMOE_ERR_UNSUPPORTED;
  if ((K % 8) != 0 || (M % 8) != 0) return GMOE_ERR_UNSUPPORTED;
  if (!gmoe_aligned(a, 16) || !gmoe_aligned(b, 16) || !gmoe_aligned(c, 16)) return GMOE_ERR_INVALID;
  if (!trans_a && N == 0) return GMOE_OK;  // nothing to write
  GmmParams p;
  p.a = static_cast<const unsigned char*>(a);
  p.b = static_cast<const unsigned char*>(b);
  p.c = static_cast<unsigned char*>(c);
  p.offsets = reinterpret_cast<const long long*>(expert_offsets);
  p.E = E;
  p.N = N;
  p.K = K;
  p.M = M;
  const int mode = trans_a ? MODE_TN : (trans_b ? MODE_NT : MODE_NN);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == GMOE_BF16 && out_dtype == GMOE_BF16) return launch_gmm<GMOE_BF16, GMOE_BF16>(p, mode, st);
  if (dtype == GMOE_BF16 && out_dtype == GMOE_F32) return launch_gmm<GMOE_BF16, GMOE_F32>(p, mode, st);
  if (dtype == GMOE_F16 && out_dtype == GMOE_F16) return launch_gmm<GMOE_F16, GMOE_F16>(p, mode, st);
  if (dtype == GMOE_F16 && out_dtype == GMOE_F32) return launch_gmm<GMOE_F16, GMOE_F32>(p, mode, st);
  if (dtype == GMOE_F32 && out_dtype == GMOE_F32) return launch_gmm<GMOE_F32, GMOE_F32>(p, mode, st);
  return GMOE_ERR_UNSUPPORTED;
}

extern "C" int gmoe_gmm_fp8w(const void* a, const void* b_q, const void* b_scale, void* c,
                             const int64_t* expert_offsets, int E, int64_t N, int64_t K, int64_t M,
                             int trans_b, void* stream) {
  (void)a; (void)b_q; (void)b_scale; (void)c; (void)expert_offsets; (void)E; (void)N; (void)K;
  (void)M; (void)trans_b; (void)stream;
  return GMOE_ERR_UNSUPPORTED;
}
