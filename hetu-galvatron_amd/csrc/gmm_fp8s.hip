// Grouped GEMM on block-scaled fp8 (e4m3) expert weights when an expert has few rows (the share of a
// DeepSeek-V3-shape shard one GPU receives: about 128 routed rows per local expert): weight
// streaming.  Same contract as the fp8 form of gmm.hip (gmoe_gmm_fp8w):
//   NN  c[rows_e] = a[rows_e] @ deq(b[e])      a [N,K] bf16  b [E,K,M] fp8  scales [E, K/128, M/128]
//   NT  c[rows_e] = a[rows_e] @ deq(b[e])^T    a [N,K] bf16  b [E,M,K] fp8  scales [E, M/128, K/128]
//
// The 128x128-tile kernel reads an expert's weights once per 128-row tile and widens every weight
// tile on its way into LDS; with 129..256 rows per expert that is two passes over the weights, a
// third of the MFMA work is padding, and the launch is bound by vector instructions and LDS
// traffic, not by HBM.  Here the weights are stationary in the other sense: a workgroup owns all
// rows of an expert (up to 192, in 32-row MFMA fragments; more rows are cut into equal chunks) and a
// strip of 256 columns, and streams that strip's weights from HBM exactly once.
//
//   * 8 wavefronts, two per SIMD: 4 column strips of 64 x 2 halves of the row fragments, so a
//     wavefront holds at most 3 x 2 accumulators and everything (results, partial sums, fragments)
//     lives in the 256 architectural registers a wavefront has at that occupancy: the MFMAs write
//     them directly and the block-scale fold below is one multiply-add per element, without moves
//     between the two register files.
//   * Weights travel global -> LDS as fp8 bytes by LDS-DMA (no staging registers, no conversion on
//     the way), are read as MFMA B fragments (plain 16-byte reads when the reduction index is
//     contiguous in memory, the transposing ds_read_b64_tr_b8 when it is the slow dimension) and
//     widened to bf16 in registers: one conversion instruction per pair, exact; the two wavefronts
//     that share a column strip each widen it.
//   * The activations of the expert (bf16) are copied by LDS-DMA as well and shared by the column
//     strips; a fragment read feeds two MFMAs.
//   * 3 LDS stages of 64 reduction elements (24 KiB of activations + 16 KiB of weights), two stages
//     in flight while one is multiplied.  One barrier per stage.
//   * Block scales stay exact: the products of a stage are accumulated unscaled in a second fp32
//     accumulator (two 32 x 32 sets, alternating), which is multiplied by the block's scale and
//     added to the result while the next 32 x 32 block is multiplied.  A 128-element scale block is
//     two stages, so its scale is applied twice to half of its products: the same real number,
//     another order of the fp32 additions.
//   * Bank conflicts are avoided on the global side, as in gmm_dtl.hip: a DMA instruction writes
//     1 KiB contiguously, so which 16 bytes of memory a lane fetches is permuted (XOR swizzles) and
//     the fragment addresses undo it.
#include "gmm_common.h"

namespace gmoe {

namespace fp8s {

constexpr int THREADS = 512;                     // 8 wavefronts: 2 row halves x 4 column strips
constexpr int BN = 256;                          // columns per workgroup, 64 per strip
constexpr int MAXF = 6;                          // 32-row fragments per row chunk, 3 per row half
constexpr int MAX_ROWS = MAXF * 32;
constexpr int BKS = 64;                          // reduction elements per stage
constexpr int B_BYTES = BN * BKS;                // 16 KiB of weights per stage
constexpr int B_LOADS = B_BYTES / 1024 / 8;      // LDS-DMA instructions per wavefront and stage: 2

// Stage layout.  A8 = false: bf16 activations, [row pairs][256 bytes], 24 KiB, 3 stages.  A8 = true:
// fp8 activations, [rows][64 bytes] (16 KiB: the copies come in whole KiB per wavefront, rows past
// 192 are never read), followed by the rows' power-of-two scales as one dword per row (2 KiB), 4
// stages.
template <bool A8>
struct Cfg {
  static constexpr int A_BYTES = A8 ? 16 * 1024 : MAX_ROWS * BKS * 2;
  static constexpr int A_LOADS = A_BYTES / 1024 / 8;  // per wavefront and stage: 3 (bf16) or 2 (fp8)
  static constexpr int S_BYTES = A8 ? 2048 : 0;
  static constexpr int S_LOADS = A8 ? 1 : 0;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + S_BYTES;
  static constexpr int NST = A8 ? 4 : 3;
  static constexpr int AHEAD = NST - 1;                // stages requested ahead of the one multiplied
  static constexpr int LOADS_PER_STAGE = A_LOADS + B_LOADS + S_LOADS;
  static constexpr int FRAG_BYTES = A8 ? 32 * 64 : 4096;  // LDS bytes of a 32-row fragment
};

typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

// One LDS-DMA instruction of 4 bytes per lane: lane L copies rsrc[voff + soff] to LDS[lds_base + 4*L].
__device__ __forceinline__ void dma4(uint32_t lds_base, uint32_t voff, const u32x4& rsrc, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory", "m0");
}

// Timing probes (results are wrong; the library is built without GMOE_FP8S_PROBE): 1 leaves out the
// fragment reads, conversions, MFMAs and the scale fold (what the copies alone take), 2 the weight
// copies after the first two stages, 4 the activation copies after the first two stages, 8 the
// barrier of a stage.
#ifndef GMOE_FP8S_PROBE
#define GMOE_FP8S_PROBE 0
#endif
constexpr bool kProbeNoCompute = (GMOE_FP8S_PROBE & 1) != 0;
constexpr bool kProbeNoWeightCopies = (GMOE_FP8S_PROBE & 2) != 0;
constexpr bool kProbeNoActivationCopies = (GMOE_FP8S_PROBE & 4) != 0;
constexpr bool kProbeNoBarrier = (GMOE_FP8S_PROBE & 8) != 0;   // with 2 and 4: no barrier per stage

// Row chunks of an expert with n rows: equal parts of at most MAX_ROWS rows, multiples of 32.
__device__ __forceinline__ int chunks_of(long long n) { return (int)((n + MAX_ROWS - 1) / MAX_ROWS); }
__device__ __forceinline__ int chunk_rows(long long n, int chunks) {
  return (int)(((n + chunks - 1) / chunks + 31) / 32 * 32);
}

// What a lane needs to issue its copies and read its fragments; set up once per item.
template <bool NT, bool A8>
struct Lane {
  u32x4 rsrc_a, rsrc_b, rsrc_s;
  uint32_t voff_a[Cfg<A8>::A_LOADS], voff_b[B_LOADS];  // byte offsets of this lane's copies of stage 0
  uint32_t voff_s;            // A8: this lane's dword of the activation scales
  uint32_t b_kstep;           // bytes a stage advances in the weight operand
  uint32_t s_kstep;           // A8: bytes a 128-element block advances in the scale table
  uint32_t a_off[4];          // fragment read offsets inside a stage: bf16 per K step; fp8 the two 16-byte halves
  uint32_t b_off[2];          // NT: per K-step pair (fp8: per half); NN: per column fragment
};

// The block scales of one item's reduction for this wavefront's column strip, kept in registers: lane
// l of register r holds the scale of 128-element block 64*r + l.  A per-stage load from memory would
// share the copy counter with the LDS-DMA copies, and waiting for it would wait for them.
constexpr int kScaleRegs = 4;  // reductions of up to 4 * 64 * 128 elements
struct StripScales {
  float r[kScaleRegs];
  __device__ __forceinline__ float at(int kt) const {  // kt: 64-element stage
    const int kb = kt >> 1;
    float v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, r[0]), kb & 63));
#pragma unroll
    for (int q = 1; q < kScaleRegs; ++q) {
      const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, r[q]), kb & 63));
      v = (kb >> 6) == q ? w : v;
    }
    return v;
  }
};

// One stage's copies of this wavefront: 3 KiB of activations (rows past the chunk read zeros and
// cost no memory traffic) and 2 KiB of weights.
__device__ __forceinline__ u32x4 uniform_rsrc(const u32x4& r) {
  return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane(r[0]), (uint32_t)__builtin_amdgcn_readfirstlane(r[1]),
               (uint32_t)__builtin_amdgcn_readfirstlane(r[2]), (uint32_t)__builtin_amdgcn_readfirstlane(r[3])};
}
template <bool NT, bool A8>
__device__ __forceinline__ void issue_stage(uint32_t lds0, const Lane<NT, A8>& ln, int wave, int kt) {
  using C = Cfg<A8>;
  const uint32_t st = lds0 + (uint32_t)((kt % C::NST) * C::STAGE_BYTES);
  // the resources are wavefront-uniform; the copies take them in scalar registers
  const u32x4 rsrc_a = uniform_rsrc(ln.rsrc_a), rsrc_b = uniform_rsrc(ln.rsrc_b);
  const uint32_t b_kstep = __builtin_amdgcn_readfirstlane(ln.b_kstep);
  static_for<0, C::A_LOADS>([&](auto t_c) {
    constexpr int t = decltype(t_c)::value;
    const uint32_t voff = (kProbeNoActivationCopies && kt > 1) ? kOob : ln.voff_a[t];
    dma16(st + (uint32_t)((wave * C::A_LOADS + t) * 1024), voff, rsrc_a, (uint32_t)(kt * (A8 ? BKS : BKS * 2)));
  });
  static_for<0, B_LOADS>([&](auto t_c) {
    constexpr int t = decltype(t_c)::value;
    const uint32_t voff = (kProbeNoWeightCopies && kt > 1) ? kOob : ln.voff_b[t];
    dma16(st + C::A_BYTES + (uint32_t)((wave * B_LOADS + t) * 1024), voff, rsrc_b, (uint32_t)kt * b_kstep);
  });
  if constexpr (A8) {
    // the scales of the 128-element block the stage belongs to, one dword per row
    const u32x4 rsrc_s = uniform_rsrc(ln.rsrc_s);
    const uint32_t s_kstep = __builtin_amdgcn_readfirstlane(ln.s_kstep);
    dma4(st + C::A_BYTES + B_BYTES + (uint32_t)(wave * 256), ln.voff_s, rsrc_s, (uint32_t)(kt >> 1) * s_kstep);
  }
}

// The reduction of one item; its stages 0 and 1 have been requested by the caller.
template <bool NT, int NF>
__device__ __forceinline__ void run_item(unsigned char* lds, uint32_t lds0, const Lane<NT, false>& ln,
                                         const StripScales& scale, int kt_cnt, int wave, int frag0,
                                         f32x16 (&acc)[NF > 0 ? NF : 1][2]) {
  constexpr int NST = Cfg<false>::NST, STAGE_BYTES = Cfg<false>::STAGE_BYTES, A_BYTES = Cfg<false>::A_BYTES;
  constexpr int LOADS_PER_STAGE = Cfg<false>::LOADS_PER_STAGE;
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // Software pipeline of a stage, in program order (pinned with scheduling fences).  The unit of work
  // is a 32 x 32 block of the result (row fragment i, column fragment j): 4 MFMAs, one per K step,
  // into one of two sets of partial sums; meanwhile the other set, the partial sums of the block
  // before (for the first block: of the last block of the previous stage), is scaled into the
  // result, 4 multiply-adds after each MFMA.  A stage has an even number of blocks, so block (i, j)
  // always uses set j.  The weight fragments are widened just before the first blocks need them;
  // the A fragment of a K step is refilled with the next row fragment's as soon as both MFMAs that
  // read it have been issued.
  u32x4 bf[4][2];
  u32x4 fa[4];
  f32x16 accq[2];
  accq[0] = accq[1] = zero;
  float sc_prev = 0.f;  // scale of the pending partial sums (none before the first stage)

  auto stage = [&](int kt, float sc) {
    const unsigned char* sa = lds + (kt % NST) * STAGE_BYTES + frag0 * 4096;
    const unsigned char* sb = lds + (kt % NST) * STAGE_BYTES + A_BYTES;
    // raw weight fragments: NT 16 bytes = K steps 2*kp, 2*kp+1 of column fragment j; NN 8 bytes per
    // (K step, column fragment) through the transposing read
    u32x4 raw_nt[2][2];
    i32x2 raw_nn[4][2];
    auto read_raw = [&](auto part_c) {  // part 0: K steps 0,1; part 1: K steps 2,3
      constexpr int part = decltype(part_c)::value;
      static_for<0, 2>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        if constexpr (NT) {
          raw_nt[part][j] = *reinterpret_cast<const u32x4*>(sb + ln.b_off[part] + j * 2048);
        } else {
          static_for<0, 2>([&](auto q_c) {
            constexpr int ks = 2 * part + decltype(q_c)::value;
            raw_nn[ks][j] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                (__attribute__((address_space(3))) i32x2*)(lds_byte*)(sb + ln.b_off[j] + ks * 4096));
          });
        }
      });
    };
    auto widen = [&](auto ks_c, auto j_c) {
      constexpr int ks = decltype(ks_c)::value, j = decltype(j_c)::value;
      uint32_t w0, w1;
      if constexpr (NT) {
        w0 = raw_nt[ks >> 1][j][2 * (ks & 1)];
        w1 = raw_nt[ks >> 1][j][2 * (ks & 1) + 1];
      } else {
        w0 = (uint32_t)raw_nn[ks][j][0];
        w1 = (uint32_t)raw_nn[ks][j][1];
      }
      bf[ks][j] = u32x4{fp8x2_to_bf16x2(w0, false), fp8x2_to_bf16x2(w0, true),
                        fp8x2_to_bf16x2(w1, false), fp8x2_to_bf16x2(w1, true)};
    };
    read_raw(std::integral_constant<int, 0>{});
    static_for<0, 4>([&](auto ks_c) {
      constexpr int ks = decltype(ks_c)::value;
      fa[ks] = *reinterpret_cast<const u32x4*>(sa + ln.a_off[ks]);
    });
    read_raw(std::integral_constant<int, 1>{});
    GMOE_SCHED_FENCE();
    static_for<0, NF>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      static_for<0, 2>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        // the block whose partial sums are pending in set 1 - j
        constexpr int pi = j == 1 ? i : (i == 0 ? NF - 1 : i - 1), pj = 1 - j;
        const float fs = (i == 0 && j == 0) ? sc_prev : sc;
        static_for<0, 4>([&](auto ks_c) {
          constexpr int ks = decltype(ks_c)::value;
          if constexpr (i == 0) {
            widen(ks_c, j_c);
            GMOE_SCHED_FENCE();
          }
          // the first product of a stage takes C = 0 (an inline constant of the instruction)
          if constexpr (ks == 0)
            accq[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, bf[ks][j]), __builtin_bit_cast(bf16x8, fa[ks]), zero, 0, 0, 0);
          else
            Mma<GMOE_BF16>::run(fa[ks], bf[ks][j], accq[j]);
          GMOE_SCHED_FENCE();
#pragma unroll
          for (int v = 4 * ks; v < 4 * ks + 4; ++v) acc[pi][pj][v] = fmaf(fs, accq[pj][v], acc[pi][pj][v]);
          // both MFMAs that read this K step's A fragment have been issued: refill it with the next
          // row fragment's, 4 MFMAs before that is needed
          if constexpr (j == 1 && i + 1 < NF)
            fa[ks] = *reinterpret_cast<const u32x4*>(sa + ln.a_off[ks] + (i + 1) * 4096);
          GMOE_SCHED_FENCE();
        });
      });
    });
    sc_prev = sc;
  };

  float sc = scale.at(0);
  for (int kt = 0; kt < kt_cnt; ++kt) {
    // stage kt has landed (stage kt+1 may still be in flight); after the barrier every wavefront
    // sees it and has finished with stage kt-1, whose buffer the next copies overwrite.  Copies
    // past the reduction read zeros: the count of outstanding copies stays the same to the end.
    wait_dma_outstanding<LOADS_PER_STAGE>();
    if constexpr (!kProbeNoBarrier) __syncthreads();
    issue_stage<NT, false>(lds0, ln, wave, kt + 2);
    const float sc_next = scale.at(kt + 1);
    if constexpr (!kProbeNoCompute && NF > 0) stage(kt, sc);
    sc = sc_next;
  }
  // the last block's partial sums (zero, with scale zero, when the reduction is empty)
  if constexpr (NF > 0) {
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[NF - 1][1][v] = fmaf(sc_prev, accq[1][v], acc[NF - 1][1][v]);
  }
}

// The same for fp8 activations: a 32 x 32 block of a stage is ONE block-scaled fp8 MFMA
// (v_mfma_scale_f32_32x32x64_f8f6f4: 64 reduction elements, 32 bytes per lane and operand, no
// widening), with the rows' power-of-two scales as the instruction's scale operand (exact: an
// exponent adjustment) and ones for the weights, whose bf16 block scales are applied by the fold as
// before.  Stages 0 .. 2 have been requested by the caller.
template <bool NT, int NF>
__device__ __forceinline__ void run_item(unsigned char* lds, uint32_t lds0, const Lane<NT, true>& ln,
                                         const StripScales& scale, int kt_cnt, int wave, int frag0,
                                         f32x16 (&acc)[NF > 0 ? NF : 1][2]) {
  using C = Cfg<true>;
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  constexpr int kOnes = 0x7f7f7f7f;  // E8M0 1.0 in every byte
  f32x16 accq[2];
  accq[0] = accq[1] = zero;
  float sc_prev = 0.f;

  auto stage = [&](int kt, float sc) {
    const unsigned char* st = lds + (kt % C::NST) * C::STAGE_BYTES;
    const unsigned char* sa = st + frag0 * C::FRAG_BYTES;
    const unsigned char* sb = st + C::A_BYTES;
    const int* ss = reinterpret_cast<const int*>(st + C::A_BYTES + B_BYTES) + frag0 * 32 + (threadIdx.x & 31);
    i32x8 fb[2], fa[2];
    int sa_e8[NF > 0 ? NF : 1];
    auto read_a = [&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      const u32x4 lo = *reinterpret_cast<const u32x4*>(sa + ln.a_off[0] + i * C::FRAG_BYTES);
      const u32x4 hi = *reinterpret_cast<const u32x4*>(sa + ln.a_off[1] + i * C::FRAG_BYTES);
      fa[i & 1] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    };
    static_for<0, 2>([&](auto j_c) {
      constexpr int j = decltype(j_c)::value;
      if constexpr (NT) {
        const u32x4 lo = *reinterpret_cast<const u32x4*>(sb + ln.b_off[0] + j * 2048);
        const u32x4 hi = *reinterpret_cast<const u32x4*>(sb + ln.b_off[1] + j * 2048);
        fb[j] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      } else {
        i32x2 q[4];
        static_for<0, 4>([&](auto q_c) {
          constexpr int qq = decltype(q_c)::value;
          q[qq] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
              (__attribute__((address_space(3))) i32x2*)(lds_byte*)(sb + ln.b_off[j] + qq * 2048));
        });
        fb[j] = i32x8{q[0][0], q[0][1], q[1][0], q[1][1], q[2][0], q[2][1], q[3][0], q[3][1]};
      }
    });
    read_a(std::integral_constant<int, 0>{});
#pragma unroll
    for (int i = 0; i < NF; ++i) sa_e8[i] = ss[i * 32];
    GMOE_SCHED_FENCE();
    static_for<0, NF>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      if constexpr (i + 1 < NF) read_a(std::integral_constant<int, i + 1>{});
      static_for<0, 2>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        constexpr int pi = j == 1 ? i : (i == 0 ? NF - 1 : i - 1), pj = 1 - j;
        const float fs = (i == 0 && j == 0) ? sc_prev : sc;
        // first operand: the weights' columns (scale one); second: the rows with their scale, so
        // that a lane ends up with 4 consecutive columns of one row, as in the bf16 kernels
        accq[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i & 1], zero, 0, 0, 0, kOnes, 0,
                                                                  sa_e8[i]);
        GMOE_SCHED_FENCE();
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[pi][pj][v] = fmaf(fs, accq[pj][v], acc[pi][pj][v]);
        GMOE_SCHED_FENCE();
      });
    });
    sc_prev = sc;
  };

  float sc = scale.at(0);
  for (int kt = 0; kt < kt_cnt; ++kt) {
    // stage kt has landed (stages kt+1, kt+2 may still be in flight); after the barrier every
    // wavefront has finished with stage kt-1, whose buffer the next copies overwrite
    wait_dma_outstanding<(C::AHEAD - 1) * C::LOADS_PER_STAGE>();
    if constexpr (!kProbeNoBarrier) __syncthreads();
    issue_stage<NT, true>(lds0, ln, wave, kt + C::AHEAD);
    const float sc_next = scale.at(kt + 1);
    if constexpr (!kProbeNoCompute && NF > 0) stage(kt, sc);
    sc = sc_next;
  }
  if constexpr (NF > 0) {
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[NF - 1][1][v] = fmaf(sc_prev, accq[1][v], acc[NF - 1][1][v]);
  }
}

template <bool NT, bool A8>
__global__ __launch_bounds__(THREADS, 1) void gmm_fp8_skinny_kernel(GmmParams p) {
  using C = Cfg<A8>;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  __shared__ int item_cum[kMaxGroupsLds + 1];          // exclusive prefix of items over `order`
  __shared__ unsigned short order[kMaxGroupsLds];      // experts by ascending rows per chunk
  __shared__ unsigned short rows_key[kMaxGroupsLds];
  __shared__ int wave_tot[THREADS / 64];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rh = wave >> 2, cs = wave & 3;  // row half, column strip
  const uint32_t lds0 = lds_offset_of(lds);
  const int E = p.E;
  const int64_t K = p.K, M = p.M;
  const int nct = (int)((M + BN - 1) / BN);

  {
    // Items per expert (row chunks x column strips).  The experts are taken in the order of their
    // rows per chunk, fewest first (an item's time grows with its row fragments), so that the
    // workgroups that get one item more than the others, the first ones, get the cheapest items.
    constexpr int kPer = kMaxGroupsLds / THREADS;
    constexpr int kSortMax = 256;  // beyond that many experts the order stays as it is
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int e = tid * kPer + j;
      if (e < E) {
        const long long n = group_begin(p, e + 1) - group_begin(p, e);
        const int nch = chunks_of(n);
        rows_key[e] = (unsigned short)(n > 0 ? chunk_rows(n, nch) : 0);
        item_cum[e] = nch * nct;  // for now: the expert's item count
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int e = tid * kPer + j;
      if (e < E) {
        int rank = e;
        if (E <= kSortMax) {
          const unsigned short key = rows_key[e];
          rank = 0;
          for (int o = 0; o < E; ++o) rank += (rows_key[o] < key || (rows_key[o] == key && o < e)) ? 1 : 0;
        }
        order[rank] = (unsigned short)e;
      }
    }
    __syncthreads();
    int cnt[kPer], local = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int i = tid * kPer + j;
      cnt[j] = i < E ? item_cum[order[i]] : 0;
      local += cnt[j];
    }
    int incl = local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(incl, d);
      if (lane >= d) incl += o;
    }
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();  // every count has been read: item_cum turns into the prefix
    int run = incl - local;
    for (int w = 0; w < wave; ++w) run += wave_tot[w];
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int i = tid * kPer + j;
      if (i <= E) item_cum[i] = run;
      run += cnt[j];
    }
    if (tid == THREADS - 1) item_cum[E] = run;
  }
  __syncthreads();
  const long long total = item_cum[E];

  // Lane geometry that does not depend on the item.
  Lane<NT, A8> ln;
  if constexpr (A8) {
    // fp8 activations [row][64 bytes]: 16-byte unit u of row r at unit u ^ ((r >> 2) & 3); a lane
    // supplies the 32 reduction elements 32*h .. 32*h + 31 of its row (units 2*h, 2*h + 1) to the
    // MFMA, the weights' lanes the same elements of their column
    const int r = lane & 31, h = lane >> 5;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      ln.a_off[q] = (uint32_t)(r * 64 + (((2 * h + q) ^ ((r >> 2) & 3)) << 4));
      ln.a_off[2 + q] = 0;
    }
    if (NT) {
#pragma unroll
      for (int q = 0; q < 2; ++q)
        ln.b_off[q] = (uint32_t)((64 * cs + r) * 64 + (((2 * h + q) ^ ((r >> 2) & 3)) << 4));
    } else {
      // four transposing reads of 8 k rows each: k rows 32*h + 8*q + t, t = 0 .. 7
      const int i16 = lane & 15, g16 = (lane >> 4) & 1;
#pragma unroll
      for (int j = 0; j < 2; ++j)
        ln.b_off[j] = (uint32_t)((32 * h + (i16 >> 1)) * 256 + (((2 * cs + j) ^ (i16 >> 1)) << 5) +
                                 16 * g16 + 8 * (i16 & 1));
    }
  } else {
    const int r = lane & 31, h = lane >> 5;
    const int x = (r >> 1) & 7;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      // 16-byte chunk (8 reduction elements) of the row this lane supplies to the MFMA of K step ks:
      // the natural order for NN; for NT the weights arrive 16 bytes (two K steps) per lane, so the
      // lane halves take the chunks 4*(ks/2) + 2*h + ks%2 (any order works as long as both operands
      // agree)
      const int c = NT ? 4 * (ks >> 1) + 2 * h + (ks & 1) : 2 * ks + h;
      ln.a_off[ks] = (uint32_t)((r >> 1) * 256 + (r & 1) * 128 + ((c ^ x) << 4));
    }
    if (NT) {
      // weights [col][64 bytes]: unit u (16 bytes) of column c at unit u ^ ((c >> 2) & 3)
      const int cl = lane & 31;
#pragma unroll
      for (int kp = 0; kp < 2; ++kp)
        ln.b_off[kp] = (uint32_t)((64 * cs + cl) * 64 + (((2 * kp + h) ^ ((cl >> 2) & 3)) << 4));
    } else {
      // weights [k row][256 bytes]: 32-byte segment sg of row k at segment sg ^ (k & 7); lanes 2t,
      // 2t+1 of a group of 16 address the two halves of k row t of an 8 x 16 block
      const int i16 = lane & 15, g16 = (lane >> 4) & 1;
#pragma unroll
      for (int j = 0; j < 2; ++j)
        ln.b_off[j] = (uint32_t)((8 * h + (i16 >> 1)) * 256 + (((2 * cs + j) ^ (i16 >> 1)) << 5) +
                                 16 * g16 + 8 * (i16 & 1));
    }
  }

  const int G = gridDim.x, per_xcd = G / 8;
  const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
  const int kt_cnt = (int)(K / BKS);

  // What the epilogue of an item needs, and what a wavefront's share of it is.
  struct Item {
    int rows;        // rows of the chunk
    int frag0, nfw;  // this wavefront's first row fragment and how many it has
    unsigned char* c_base;
    int64_t col0;
  };
  StripScales scale;
  // Items are dealt in runs: workgroup w of G (numbered XCD by XCD) would get the q or q + 1 consecutive
  // items from run_begin(w) on, one more for the first total % G workgroups, which are the cheapest
  // items.  An XCD takes the runs of its workgroups together and deals them round-robin: at any time
  // its workgroups work on consecutive items, the column strips of one or two experts, so its L2
  // holds those experts' activations for all of them and neighbouring weight columns are streamed
  // together.
  const long long q_items = total / G, r_items = total % G;
  auto run_begin = [&](long long w) {
    return w < r_items ? w * (q_items + 1) : r_items * (q_items + 1) + (w - r_items) * q_items;
  };
  const long long first = run_begin((long long)xcd * per_xcd) + slot;
  const long long last = run_begin((long long)(xcd + 1) * per_xcd);
  int pos = 0;
  // Item `v` of this workgroup's run: fills the copy addresses and requests the block scales.
  auto setup = [&](long long v, Item& it) -> bool {
    if (v >= last) return false;
    while (item_cum[pos + 1] <= v) ++pos;
    pos = __builtin_amdgcn_readfirstlane(pos);
    const int e = __builtin_amdgcn_readfirstlane((int)order[pos]);
    const long long row_e = group_begin(p, e);
    const long long n_e = group_begin(p, e + 1) - row_e;
    const int nch = chunks_of(n_e);
    const int q = (int)(v - item_cum[pos]);
    const int ct = q / nch, ch = q % nch;
    const int per = chunk_rows(n_e, nch);
    const long long r0 = (long long)ch * per;
    const int rows = (int)(n_e - r0 < per ? n_e - r0 : per);  // >= 1: chunks are never empty
    // the chunk's nf row fragments are split between the two wavefronts of a column strip: the
    // first takes the first ceil(nf / 2), the second the rest (none when nf = 1: it then only copies)
    const int nf = (rows + 31) / 32;
    it.rows = rows;
    it.frag0 = __builtin_amdgcn_readfirstlane(rh * ((nf + 1) / 2));
    it.nfw = __builtin_amdgcn_readfirstlane(rh ? nf / 2 : (nf + 1) / 2);
    const long long row0 = row_e + r0;
    const int64_t col0 = (int64_t)ct * BN;
    it.col0 = col0;
    it.c_base = p.c + row0 * M * 2;

    // activations: LDS [row pair SR][16 slots of 16 bytes]; slot s of pair SR holds chunk
    // (s & 7) ^ (SR & 7) of row 2*SR + (s >> 3).  Copy t of wavefront w fills the 1 KiB block
    // 3*w + t: row pairs 4*(3*w + t) .. + 3.
    if constexpr (A8) {
      // fp8 activations: copy t of wavefront w fills block 2*w + t: rows 16*(2*w + t) .. + 15, lane L
      // the unit (L % 4) ^ ((row >> 2) & 3) of row 16*(2*w + t) + L / 4
      ln.rsrc_a = make_raw_rsrc(p.a + row0 * K, (int64_t)rows * K);
#pragma unroll
      for (int t = 0; t < C::A_LOADS; ++t) {
        const int row = 16 * (wave * C::A_LOADS + t) + (lane >> 2), u = (lane & 3) ^ ((row >> 2) & 3);
        ln.voff_a[t] = (uint32_t)((int64_t)row * K + u * 16);
      }
      // the rows' scales: table [128-element block][N] of dwords; lane L of wavefront w copies row 64*w + L
      const int kbs_a = (int)((K + 127) / 128);
      const int srow = 64 * wave + lane;
      ln.rsrc_s = make_raw_rsrc(p.a_scale + row0 * 4, ((int64_t)(kbs_a - 1) * p.N + rows) * 4);
      ln.voff_s = srow < rows ? (uint32_t)(srow * 4) : kOob;
      ln.s_kstep = (uint32_t)(p.N * 4);
    } else {
      ln.rsrc_a = make_raw_rsrc(p.a + row0 * K * 2, (int64_t)rows * K * 2);
#pragma unroll
      for (int t = 0; t < C::A_LOADS; ++t) {
        const int SR = 4 * (wave * C::A_LOADS + t) + (lane >> 4), s = lane & 15;
        const int row = 2 * SR + (s >> 3), c = (s & 7) ^ (SR & 7);
        ln.voff_a[t] = (uint32_t)((int64_t)row * K * 2 + c * 16);
      }
    }
    if (NT) {
      // weights [M,K]: copy t of wavefront w fills block 2*w + t: columns 16*(2*w + t) .. + 15,
      // lane L the 16-byte unit (L % 4) ^ ((col >> 2) & 3) of column 16*(2*w + t) + L / 4
      const int64_t cols = M - col0 < BN ? M - col0 : BN;
      ln.rsrc_b = make_raw_rsrc(p.b + ((int64_t)e * M + col0) * K, cols * K);
#pragma unroll
      for (int t = 0; t < B_LOADS; ++t) {
        const int col = 16 * (wave * B_LOADS + t) + (lane >> 2), u = (lane & 3) ^ ((col >> 2) & 3);
        ln.voff_b[t] = (uint32_t)((int64_t)col * K + u * 16);
      }
      ln.b_kstep = BKS;
    } else {
      // weights [K,M]: block 2*w + t holds k rows 4*(2*w + t) .. + 3, lane L the 16-byte unit U of
      // its row with U = (((L%16) >> 1) ^ (krow & 7)) << 1 | (L & 1)
      ln.rsrc_b = make_raw_rsrc(p.b + (int64_t)e * K * M + col0, K * M - col0);
#pragma unroll
      for (int t = 0; t < B_LOADS; ++t) {
        const int krow = 4 * (wave * B_LOADS + t) + (lane >> 4);
        const int U = ((((lane & 15) >> 1) ^ (krow & 7)) << 1) | (lane & 1);
        ln.voff_b[t] = (uint32_t)((int64_t)krow * M + U * 16);
      }
      ln.b_kstep = (uint32_t)(BKS * M);
    }
    // this wavefront's 64 columns lie inside one 128-column scale block; one load per register
    const int kbs = (int)((K + 127) / 128), mbs = (int)((M + 127) / 128);
    const int mb = (int)((col0 + 64 * cs) / 128);
    const int mbu = mb < mbs ? mb : mbs - 1;
    const uint16_t* sbase = reinterpret_cast<const uint16_t*>(p.b_scale) + (int64_t)e * kbs * mbs;
#pragma unroll
    for (int q2 = 0; q2 < kScaleRegs; ++q2) {
      const int kb = 64 * q2 + lane;
      const int kbc = kb < kbs ? kb : kbs - 1;
      scale.r[q2] = bf16_bits_to_f32(NT ? sbase[(int64_t)mbu * kbs + kbc] : sbase[(int64_t)kbc * mbs + mbu]);
    }
    return true;
  };

  // Items follow each other without draining the copy pipeline: once an item's reduction is done,
  // the next item's addresses are set up and its block scales requested, the finished result is
  // stored straight from the accumulators (8 bytes per lane, a row's two lane halves side by side:
  // the result is a small fraction of the item's bytes, and without LDS staging the stages are free
  // at once), and after one barrier (every wavefront is done reading the last stage) the next
  // item's first two stages are requested.
  Item cur;
  if (!setup(first, cur)) return;
  static_for<0, C::AHEAD>([&](auto s_c) { issue_stage<NT, A8>(lds0, ln, wave, decltype(s_c)::value); });
  for (long long base = first;;) {
    Item nxt;
    bool more = false;
    auto item = [&](auto nf_c) {
      constexpr int NF = decltype(nf_c)::value;
      f32x16 acc[NF > 0 ? NF : 1][2];
#pragma unroll
      for (int i = 0; i < NF; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int vv = 0; vv < 16; ++vv) acc[i][j][vv] = 0.f;
      run_item<NT, NF>(lds, lds0, ln, scale, kt_cnt, wave, cur.frag0, acc);  // overload on the lane type
      base += per_xcd;
      more = setup(base, nxt);
      // lane holds row (lane % 32), columns 8*(v/4) + 4*(lane/32) + v%4 of each 32 x 32 block
#pragma unroll
      for (int i = 0; i < NF; ++i) {
        const int row = (cur.frag0 + i) * 32 + (lane & 31);
        if (row >= cur.rows) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int64_t n = cur.col0 + cs * 64 + j * 32 + 8 * vq + 4 * (lane >> 5);
            if (n < M)
              *reinterpret_cast<u32x2*>(cur.c_base + ((int64_t)row * M + n) * 2) =
                  pack4<GMOE_BF16>(acc[i][j][4 * vq], acc[i][j][4 * vq + 1], acc[i][j][4 * vq + 2],
                                   acc[i][j][4 * vq + 3]);
          }
      }
    };
    // the two row halves may take different paths; both pass the same barriers
    switch (cur.nfw) {
      case 0: item(std::integral_constant<int, 0>{}); break;
      case 1: item(std::integral_constant<int, 1>{}); break;
      case 2: item(std::integral_constant<int, 2>{}); break;
      default: item(std::integral_constant<int, 3>{}); break;
    }
    __syncthreads();
    if (!more) break;
    cur = nxt;
    static_for<0, C::AHEAD>([&](auto s_c) { issue_stage<NT, A8>(lds0, ln, wave, decltype(s_c)::value); });
  }
  // the copies requested past the last reduction (zeros) land before the workgroup ends
  wait_dma_outstanding<0>();
}

template <bool NT, bool A8>
static int launch(const GmmParams& p, hipStream_t st) {
  constexpr size_t smem = (size_t)Cfg<A8>::NST * Cfg<A8>::STAGE_BYTES;
  auto kern = gmm_fp8_skinny_kernel<NT, A8>;
  static std::atomic<uint64_t> done_mask{0};
  if (!gmoe_once_per_device(done_mask, [&] {
        return hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess;
      }))
    return GMOE_ERR_LAUNCH;
  int grid = (gmoe_cu_count() / 8) * 8;
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(THREADS), smem, st, p);
  return gmoe_launch_status();
}

}  // namespace fp8s

// Few rows per expert (on average at most 256: the weights of an expert are then read once or
// twice), a reduction that is whole stages, and strides that fit the 32-bit copy offsets.
bool gmm_fp8_skinny_applies(const GmmParams& p, bool any_row_count) {
  const int64_t experts = p.E > 0 ? p.E : 1;
  return (any_row_count || p.N <= 256 * experts) && p.K % fp8s::BKS == 0 && p.M % 16 == 0 &&
         p.K <= fp8s::kScaleRegs * 64 * 128 && (int64_t)fp8s::MAX_ROWS * p.K * 2 < (1ll << 31) &&
         ((p.K + 127) / 128) * p.N * 4 < (1ll << 31);
}

int launch_gmm_fp8_skinny(const GmmParams& p, bool trans_b, hipStream_t st) {
  if (p.a_scale != nullptr) return trans_b ? fp8s::launch<true, true>(p, st) : fp8s::launch<false, true>(p, st);
  return trans_b ? fp8s::launch<true, false>(p, st) : fp8s::launch<false, false>(p, st);
}

}  // namespace gmoe
