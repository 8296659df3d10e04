// Grouped GEMM, LDS-DMA variant for the dW product (TN) of 16-bit operands (bf16 / fp16) on gfx950:
//   c[e] = a[rows_e]^T @ b[rows_e],  a [N,K], b [N,M], c [E,K,M].
//
// Same contract, tile order and MFMA arrangement as gmm.hip (256x256 block tile, 2x2 wavefronts,
// 32x32x16 MFMAs, operands swapped so a lane owns 4 consecutive columns of C).  What differs is how
// operand tiles reach LDS and how deep the prefetch is:
//
//   * Global memory is copied straight into LDS by `buffer_load_dwordx4 ... lds` (no staging
//     registers, no ds_write).  A wavefront instruction deposits 64 x 16 bytes contiguously, so
//     there is no room for row padding; bank conflicts are avoided by permuting WHICH 16-byte
//     chunk a lane fetches (an XOR swizzle applied on the global side) and undoing it in the
//     fragment addresses.
//   * A K tile is 32 elements deep and LDS holds 4 stages (4 x 32 KiB): the copy of tile t+3 is
//     issued while tile t is multiplied, i.e. a request has about three tiles of MFMAs to land.
//     One barrier per K tile; the copies are tracked by hand (vmcnt), the compiler tracks the
//     LDS reads.
//   * Both operands have the reduction index (the token) as the slow dimension in memory; they are
//     stored in LDS as they are in memory, [k][outer], and the MFMA fragments are read with the
//     transposing LDS load ds_read_b64_tr_b16: a group of 16 lanes reads a 4(k) x 16(outer) block
//     and every lane receives the 4 k-values of its own column.
//
// For NN and NT the register-staged kernel of gmm.hip measured faster: copies of an operand whose
// reduction index is contiguous arrive as 64-byte row pieces here, which the address path handles
// at half the rate of the 128-byte pieces that kernel requests.
#include "gmm_common.h"

namespace gmoe {

namespace dtl {

constexpr int BM = 256, BN = 256;
constexpr int BKT = 32;                 // reduction elements per stage
constexpr int NST = 4;                  // LDS stages
constexpr int OPER_BYTES = 256 * BKT * 2;  // one operand tile: 16 KiB
constexpr int STAGE_BYTES = 2 * OPER_BYTES;
constexpr int LOADS_PER_TILE = 8;       // LDS-DMA instructions per wavefront per K tile (4 per operand)

typedef short s16x4 __attribute__((ext_vector_type(4)));
// ---- operand stored outer-contiguous: LDS tile [32 k][256 outer], 512 bytes per k row ----------
// The 64-byte segment sg of row k sits at segment position sg ^ f(k), f(k) = (k & 3) | ((k >> 1) & 4):
// the 8 rows one transposing read touches (k0..k0+3 and k0+8..k0+11) land in 8 different segments.
struct TransOperand {
  u32x4 rsrc;
  uint32_t voff[4];
  uint32_t row_bytes;
  uint32_t frag_k;       // byte offset of the lane's first k row
  uint32_t frag_seg[4];  // byte offset of the lane's 8 bytes inside a k row, per fragment

  // src: the expert's operand (row 0 = first reduction index); the tile starts at outer index o0.
  __device__ __forceinline__ void init(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t k_limit, int wave, int lane, int sub_col0) {
    rsrc = make_raw_rsrc(src + o0 * 2, k_limit * ld * 2 - o0 * 2);
    row_bytes = (uint32_t)(ld * 2);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int krow = (wave * 4 + q) * 2 + (lane >> 5);
      const int f = (krow & 3) | ((krow >> 1) & 4);
      const int P = lane & 31;                      // 16-byte slot inside the k row
      const int ct = ((((P >> 2) ^ f) << 2) + (P & 3)) * 8;  // tile column this slot holds
      voff[q] = (uint32_t)(((int64_t)krow * ld + ct) * 2);
    }
    const int s = lane & 15, g = lane >> 5, half = (lane >> 4) & 1;
    frag_k = (uint32_t)((8 * g + (s >> 2)) * 512);
    const int f = (s >> 2) | (g << 2);
    const int seg0 = sub_col0 / 32;  // 128-column sub-tile: 0 or 4
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      frag_seg[j] = (uint32_t)((((seg0 + j) ^ f) * 64) + half * 32 + (s & 3) * 8);
    }
  }
  template <int q>
  __device__ __forceinline__ void issue(int kt, uint32_t lds_tile, int wave) const {
    dma16(lds_tile + (uint32_t)((wave * 4 + q) * 1024), voff[q], rsrc,
          (uint32_t)(kt * BKT) * row_bytes);
  }
  static constexpr int READS_PER_FRAG = 2;
  // half h (4 of the 8 k values) of fragment j of K step ks
  template <int j, int ks, int h>
  __device__ __forceinline__ void read(const unsigned char* tile, u32x4& f) const {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(lds_byte*)(tile + frag_k + frag_seg[j] +
                                                               (ks * 16 + h * 4) * 512));
    const u32x2 w = __builtin_bit_cast(u32x2, v);
    f[2 * h] = w[0];
    f[2 * h + 1] = w[1];
  }
};

template <int DT, int ODT>
__global__ __launch_bounds__(kGemmThreads) void gmm_dtl_kernel(GmmParams p) {
  typedef TransOperand OpA;
  typedef TransOperand OpB;
  constexpr int WT = 4;   // 32x32 accumulators per wavefront in each direction
  constexpr int NM = 16;  // MFMAs per K step
  constexpr int RA = OpA::READS_PER_FRAG, RB = OpB::READS_PER_FRAG;
  constexpr int NREAD = WT * RA + WT * RB;  // LDS reads per K step

  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t lds0 = lds_offset_of(lds);

  const int E = p.E;
  const int64_t K = p.K, M = p.M;
  const int nt_cnt = (int)((M + BN - 1) / BN);
  const int mt_cnt = (int)((K + BM - 1) / BM);

  // every expert has the same mt_cnt x nt_cnt grid of output tiles
  const long long per_expert = (long long)mt_cnt * nt_cnt;
  const long long total_tiles = per_expert * E;
  // workgroup w runs on XCD w % 8: XCD x takes the positions [x*G/8, (x+1)*G/8) of every whole round
  // of G = gridDim.x tiles; the last, partial round is dealt to the XCDs in equal consecutive shares
  const int G = gridDim.x;
  const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
  const long long whole = total_tiles / G * G;  // tiles in whole rounds
  auto tail_tile = [&]() -> long long {
    const long long share = (total_tiles - whole + 7) / 8;
    const long long t = whole + xcd * share + slot;
    return (slot < share && t < total_tiles) ? t : -1;
  };
  const long long first = (long long)xcd * (G / 8) + slot;

  for (long long s = first < whole ? first : tail_tile(); s >= 0;
       s = s >= whole ? -1 : (s + G < whole ? s + G : tail_tile())) {
    const int e = (int)(s / per_expert);
    const long long row0 = group_begin(p, e);
    const long long n_e = group_begin(p, e + 1) - row0;
    int mt, nt;
    strip_order(s - e * per_expert, mt_cnt, nt_cnt, mt, nt);

    f32x16 acc[WT][WT];
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
      for (int j = 0; j < WT; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // a buffer resource spans at most 2 GiB: an expert with more rows than that is walked in
    // segments (one segment in all but extreme cases), the accumulators carried across
    const int64_t seg_rows = tn_segment_rows(K, M, 2);
    for (int64_t seg0 = 0; seg0 < n_e; seg0 += seg_rows) {
    OpA oa;
    OpB ob;
    const int64_t k_lim = n_e - seg0 < seg_rows ? n_e - seg0 : seg_rows;
    oa.init(p.a + (row0 + seg0) * K * 2, K, (int64_t)mt * BM, k_lim, wave, lane, wm * 128);
    ob.init(p.b + (row0 + seg0) * M * 2, M, (int64_t)nt * BN, k_lim, wave, lane, wn * 128);

    const int kt_cnt = (int)((k_lim + BKT - 1) / BKT);
    u32x4 fa[2][WT], fb[2][WT];

    // copy K tile kt into its stage (all 8 instructions of this wavefront)
    auto issue_tile = [&](int kt) {
      const uint32_t st = lds0 + (uint32_t)((kt & (NST - 1)) * STAGE_BYTES);
      static_for<0, 4>([&](auto q) { oa.template issue<decltype(q)::value>(kt, st, wave); });
      static_for<0, 4>(
          [&](auto q) { ob.template issue<decltype(q)::value>(kt, st + OPER_BYTES, wave); });
    };
    // read operation r of K step ks of the tile at `stage` into fragment buffer `buf`
    auto frag_read = [&](auto r_c, auto ks_c, auto buf_c, const unsigned char* stage) {
      constexpr int r = decltype(r_c)::value, ks = decltype(ks_c)::value, buf = decltype(buf_c)::value;
      if constexpr (r < WT * RA) {
        oa.template read<r / RA, ks, r % RA>(stage, fa[buf][r / RA]);
      } else {
        constexpr int rb = r - WT * RA;
        ob.template read<rb / RB, ks, rb % RB>(stage + OPER_BYTES, fb[buf][rb / RB]);
      }
    };

    if (kt_cnt > 0) {
      // ---- prologue: tiles 0..2 in flight, wait for tile 0, fragments of its step 0 ------------
      issue_tile(0);
      issue_tile(1);
      issue_tile(2);
      wait_dma_outstanding<2 * LOADS_PER_TILE>();
      __syncthreads();
      static_for<0, NREAD>([&](auto r) {
        frag_read(r, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, lds);
      });

      for (int kt = 0; kt < kt_cnt; ++kt) {
        const unsigned char* cur = lds + (kt & (NST - 1)) * STAGE_BYTES;
        const unsigned char* nxt = lds + ((kt + 1) & (NST - 1)) * STAGE_BYTES;
        const uint32_t st3 = lds0 + (uint32_t)(((kt + 3) & (NST - 1)) * STAGE_BYTES);
        // ---- K step 0: MFMAs on buffer 0; read step 1 into buffer 1; request tile kt+3 ------
        static_for<0, NM>([&](auto m_c) {
          constexpr int m = decltype(m_c)::value;
          // boustrophedon order over the fragments: one operand changes per MFMA
          constexpr int mi = m / WT, mj = (mi & 1) ? WT - 1 - m % WT : m % WT;
          Mma<DT>::run(fa[0][mi], fb[0][mj], acc[mi][mj]);
          GMOE_SCHED_FENCE();
          constexpr int n_ops = NREAD + LOADS_PER_TILE;
          constexpr int op_begin = (m * n_ops + NM - 1) / NM;
          constexpr int op_end = ((m + 1) * n_ops + NM - 1) / NM;
          static_for<op_begin, op_end>([&](auto op_c) {
            constexpr int op = decltype(op_c)::value;
            if constexpr (op < NREAD) {
              frag_read(op_c, std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{}, cur);
            } else if constexpr (op - NREAD < 4) {
              oa.template issue<op - NREAD>(kt + 3, st3, wave);
            } else {
              ob.template issue<op - NREAD - 4>(kt + 3, st3 + OPER_BYTES, wave);
            }
          });
          GMOE_SCHED_FENCE();
        });
        // tile kt+1 must have landed (tiles kt+2 and kt+3 may still be in flight); the barrier
        // also tells everyone that this tile's stage has been read for the last time
        wait_dma_outstanding<2 * LOADS_PER_TILE>();
        __syncthreads();
        GMOE_SCHED_FENCE();
        // ---- K step 1: MFMAs on buffer 1; read step 0 of tile kt+1 into buffer 0 -------------
        static_for<0, NM>([&](auto m_c) {
          constexpr int m = decltype(m_c)::value;
          // boustrophedon order over the fragments: one operand changes per MFMA
          constexpr int mi = m / WT, mj = (mi & 1) ? WT - 1 - m % WT : m % WT;
          Mma<DT>::run(fa[1][mi], fb[1][mj], acc[mi][mj]);
          GMOE_SCHED_FENCE();
          constexpr int op_begin = (m * NREAD + NM - 1) / NM;
          constexpr int op_end = ((m + 1) * NREAD + NM - 1) / NM;
          static_for<op_begin, op_end>([&](auto op_c) {
            frag_read(op_c, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, nxt);
          });
          GMOE_SCHED_FENCE();
        });
      }
      // every copy has landed and every wavefront is done with LDS before the next tile reuses it
      wait_dma_outstanding<0>();
      __syncthreads();
    }
    }

    // ---- epilogue: lane holds row (lane%32), columns 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 ----
    constexpr int OES = Elem<ODT>::bytes;
    unsigned char* c_base = p.c + (int64_t)e * K * M * OES;
    const int64_t c_rows = K;
    if constexpr (ODT != GMOE_F32) {
      using CT = CTile<BN>;
      stage_acc_lds<ODT, WT, WT, BN>(lds, acc, wm * 128, wn * 128, lane);
      __syncthreads();
      const int cc = tid % CT::chunks, r0 = tid / CT::chunks;
      const int64_t n = (int64_t)nt * BN + cc * 8;
#pragma unroll 8
      for (int it = 0; it < BM / CT::rows_per_pass; ++it) {
        const int row = it * CT::rows_per_pass + r0;
        const int64_t m = (int64_t)mt * BM + row;
        if (m < c_rows && n < M)
          st16(c_base + (m * M + n) * OES, ctile_read16(lds + row * CT::pitch + cc * 16));
      }
      __syncthreads();  // the next tile's copies overwrite the staged values
      continue;
    }
#pragma unroll
    for (int i = 0; i < WT; ++i) {
      const int64_t m = (int64_t)mt * BM + wm * 128 + i * 32 + (lane & 31);
      if (m >= c_rows) continue;
#pragma unroll
      for (int j = 0; j < WT; ++j) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int64_t n = (int64_t)nt * BN + wn * 128 + j * 32 + 8 * vq + 4 * (lane >> 5);
          if (n >= M) continue;
          unsigned char* dst = c_base + (m * M + n) * OES;
          const float v0 = acc[i][j][4 * vq], v1 = acc[i][j][4 * vq + 1];
          const float v2 = acc[i][j][4 * vq + 2], v3 = acc[i][j][4 * vq + 3];
          if (ODT == GMOE_F32)
            *reinterpret_cast<f32x4*>(dst) = f32x4{v0, v1, v2, v3};
          else
            *reinterpret_cast<u32x2*>(dst) = pack4<ODT>(v0, v1, v2, v3);
        }
      }
    }
  }
}

template <int DT, int ODT>
static int launch_cfg(const GmmParams& p, hipStream_t st) {
  // the K-tile stages, reused by the epilogue as one 256-row tile of 16-bit results
  constexpr size_t stages = (size_t)NST * STAGE_BYTES, ctile = (size_t)BM * CTile<BN>::pitch;
  constexpr size_t smem = stages > ctile ? stages : ctile;
  auto kern = gmm_dtl_kernel<DT, ODT>;
  static std::atomic<uint64_t> done_mask{0};
  if (!gmoe_once_per_device(done_mask, [&] {
        return hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess;
      }))
    return GMOE_ERR_LAUNCH;
  int grid = (gmoe_cu_count() / 8) * 8;
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kGemmThreads), smem, st, p);
  return gmoe_launch_status();
}

}  // namespace dtl

int launch_gmm_dtl_tn(const GmmParams& p, int dtype, int out_dtype, hipStream_t st) {
  if (dtype == GMOE_BF16 && out_dtype == GMOE_BF16) return dtl::launch_cfg<GMOE_BF16, GMOE_BF16>(p, st);
  if (dtype == GMOE_BF16 && out_dtype == GMOE_F32) return dtl::launch_cfg<GMOE_BF16, GMOE_F32>(p, st);
  if (dtype == GMOE_F16 && out_dtype == GMOE_F16) return dtl::launch_cfg<GMOE_F16, GMOE_F16>(p, st);
  if (dtype == GMOE_F16 && out_dtype == GMOE_F32) return dtl::launch_cfg<GMOE_F16, GMOE_F32>(p, st);
  return GMOE_ERR_UNSUPPORTED;
}

}  // namespace gmoe
