// Grouped GEMM for gfx950 (CDNA4): one persistent kernel over a device-side expert-offset table.
// Replaces `grouped_gemm.ops.gmm` (call sites moe/mlp.py:106-112) and its backward.
//
//   NN  c[rows_e]  = a[rows_e] @ b[e]        a [N,K]  b [E,K,M]  c [N,M]    (forward)
//   NT  c[rows_e]  = a[rows_e] @ b[e]^T      a [N,K]  b [E,M,K]  c [N,M]    (dX)
//   TN  c[e]       = a[rows_e]^T @ b[rows_e] a [N,K]  b [N,M]    c [E,K,M]  (dW)
//
// Structure
//   * 256 threads = 4 wavefronts in a 2x2 grid; the block owns a BM x BN tile of C (256x256, or
//     128x128 for small groups), each wavefront a (BM/2) x (BN/2) sub-tile made of 32x32 MFMA
//     accumulators (fp32, in AGPRs).
//   * Operand tiles go global -> registers -> LDS in 16-byte pieces, two LDS stages of 64 (16-bit)
//     or 32 (fp32) reduction elements.  Global memory is read with buffer loads whose resource
//     covers exactly the expert's rows, so ragged group edges and the reduction tail read as zero
//     without branches.  How an operand sits in LDS depends on its memory layout (the loaders):
//       - reduction index contiguous: rows [outer][k] of 128 bytes padded to 144, so that the
//         16-byte fragment reads of consecutive rows hit disjoint banks (DirectLoader);
//       - reduction index in the slow dimension, 16-bit: kept as in memory, [k][outer], with an XOR
//         segment swizzle, fragments read with the transposing LDS load ds_read_b64_tr_b16
//         (RowMajorLoader for 256-wide, RowMajorSmallLoader for 128-wide tiles);
//       - reduction index in the slow dimension, fp32: 4x4 blocks transposed in registers on the way
//         to LDS (TransposeLoader);
//       - fp8 weights with block scales: widened to bf16 on the way to LDS, the block scale applied
//         in fp32 to the partial sums of each 128-element block (Fp8DirectLoader, Fp8TransposeLoader).
//   * The K loop is software pipelined by hand: a K tile is 4 steps of (BM/64)*(BN/64) MFMAs;
//     while step s runs, the fragments of step s+1 are read from LDS into the other fragment
//     buffer, tile kt+1 (held in registers since the previous iteration) is written to the other
//     LDS stage and tile kt+2 is requested from memory (small tiles hold two register sets and
//     request tile kt+3).  One barrier per K tile, placed before the last step so that the first
//     fragments of the next tile are read under that step's MFMAs.  Every index is a compile-time
//     constant (static_for); the order is pinned with scheduling barriers, the compiler only adds
//     the waitcnts.
//   * The MFMA is issued with the operands swapped (B fragment as SrcA) so that a lane ends up with
//     4 consecutive columns of one row of C; 16-bit results are staged through LDS and written as
//     16-byte row-contiguous pieces, optionally through a fused gated-activation epilogue.
//   * Tiles are numbered expert-major, inside an expert in strips of 8 column tiles, and handed to
//     workgroups so that the 32 workgroups that share an XCD (workgroup id mod 8) work on one
//     4x8 patch of tiles at a time: the A and B panels they stream are shared in that XCD's L2.
#include "gmm_common.h"

#include "gmm_probe.h"

namespace gmoe {

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, int64_t bytes) {
  const uint32_t n = bytes <= 0 ? 0u : (bytes > 0x7fffffffll ? 0x7fffffffu : (uint32_t)bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_ld16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
}

// ---- operand loaders ----------------------------------------------------------------------------
// A tile is R "outer" indices x BK reduction elements (128 bytes per outer index).  Each loader
// moves the tile in NPIECE register pieces: load_piece(i) requests piece i of K tile `kt` from
// memory, store_piece(i) writes it to an LDS stage.

// Reduction index contiguous in memory: element (o, k) at src + o*ld + k.  Thread t covers the
// 16-byte chunk t%8 of rows t/8 + 32*i.
template <int R, int ES, int DEPTH = 1>
struct DirectLoader {
  static constexpr int EPC = 16 / ES;
  static constexpr int BK = 128 / ES;
  static constexpr int NPIECE = R / 32;
  u32x4 r[DEPTH][NPIECE];
  uint32_t voff[NPIECE];
  __amdgpu_buffer_rsrc_t rsrc;
  int64_t k_lim;
  int kchunk;   // first reduction element of this thread's chunk inside a K tile
  int lds_off;  // byte offset of piece 0 inside a stage

  // src: the operand of this expert; the tile starts at outer index o0; rows >= o_lim are zero.
  __device__ __forceinline__ void init(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k_limit, int tid) {
    const int c = tid & 7, r0 = tid >> 3;
    int64_t rows = o_lim - o0;
    rows = rows < 0 ? 0 : (rows > R ? R : rows);
    rsrc = make_rsrc(src + o0 * ld * ES, rows * ld * ES);
    k_lim = k_limit;
    kchunk = c * EPC;
#pragma unroll
    for (int i = 0; i < NPIECE; ++i) voff[i] = (uint32_t)(((int64_t)(r0 + 32 * i) * ld + c * EPC) * ES);
    lds_off = r0 * kRowPad + c * 16;
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void load_piece(int kt) {
    const bool kok = (int64_t)kt * BK + kchunk < k_lim;
    r[SET][i] = buf_ld16(rsrc, kok ? voff[i] : kOob, (uint32_t)(kt * BK * ES));
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void store_piece(unsigned char* stage) const {
    *reinterpret_cast<u32x4*>(stage + lds_off + i * 32 * kRowPad) = r[SET][i];
  }
  // fragment side: 16 bytes (8 reduction elements of the lane's row) per K step, one LDS read
  static constexpr int STAGE_BYTES = R * kRowPad;
  static constexpr int READS = 1;
  static constexpr bool STORE_NEEDS_ALL_PIECES = false;
  int frag_off;
  __device__ __forceinline__ void init_frag(int sub0, int lane) {
    frag_off = (sub0 + (lane & 31)) * kRowPad + (lane >> 5) * 16;
  }
  template <int i, int KS, int h>
  __device__ __forceinline__ void read(const unsigned char* tile, u32x4& f) const {
    f = *reinterpret_cast<const u32x4*>(tile + frag_off + i * 32 * kRowPad + KS * 32);
  }
};

// Reduction index is the slow dimension: element (o, k) at src + k*ld + o.  Thread t owns the
// EPC x EPC block(s) at reduction block t%8, outer block t/8 (+32 per pass); a piece is one row of
// a block on the load side and one transposed row on the store side.
template <int R, int ES, int DEPTH = 1>
struct TransposeLoader {
  static constexpr int EPC = 16 / ES;
  static constexpr int BK = 128 / ES;
  static constexpr int OB = R / EPC;         // outer blocks in the tile
  static constexpr int NP = (OB + 31) / 32;  // passes
  static_assert(OB % 32 == 0 || OB < 32, "outer blocks must tile the 32 thread rows");
  static constexpr int NPIECE = NP * EPC;
  u32x4 r[DEPTH][NP][EPC];
  uint32_t voff[NP];
  uint32_t row_bytes;
  __amdgpu_buffer_rsrc_t rsrc;
  int lds_off;

  __device__ __forceinline__ void init(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k_limit, int tid) {
    (void)o_lim;  // outer indices past the operand only feed rows / columns of C that are not stored
    const int kb = tid & 7, ob0 = tid >> 3;
    rsrc = make_rsrc(src + o0 * ES, k_limit * ld * ES - o0 * ES);
    row_bytes = (uint32_t)(ld * ES);
    // With fewer than 32 outer blocks (16-bit, R = 128) the upper threads repeat the work of the
    // lower ones (same loads, same LDS stores) instead of branching around it.
    const int obw = ob0 % (OB < 32 ? OB : 32);
#pragma unroll
    for (int p = 0; p < NP; ++p)
      voff[p] = (uint32_t)(((int64_t)(kb * EPC) * ld + (int64_t)(obw + 32 * p) * EPC) * ES);
    lds_off = (obw * EPC) * kRowPad + kb * 16;
  }
  template <int q, int SET = 0>
  __device__ __forceinline__ void load_piece(int kt) {
    constexpr int p = q / EPC, i = q % EPC;
    // soffset carries the K tile and the row inside the block: both are wavefront-uniform
    r[SET][p][i] = buf_ld16(rsrc, voff[p], (uint32_t)(kt * BK + i) * row_bytes);
  }
  template <int q, int SET = 0>
  __device__ __forceinline__ void store_piece(unsigned char* stage) const {
    constexpr int p = q / EPC, o = q % EPC;
    u32x4 v;
    if (ES == 2) {
      // v.dword[j] = (r[2j] element o) | (r[2j+1] element o) << 16
      const uint32_t sel = (o & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        v[j] = __builtin_amdgcn_perm(r[SET][p][2 * j + 1][o >> 1], r[SET][p][2 * j][o >> 1], sel);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = r[SET][p][j][o];
    }
    *reinterpret_cast<u32x4*>(stage + lds_off + (p * 32 * EPC + o) * kRowPad) = v;
  }
  // fragment side: 16 bytes (8 reduction elements of the lane's row) per K step, one LDS read
  static constexpr int STAGE_BYTES = R * kRowPad;
  static constexpr int READS = 1;
  static constexpr bool STORE_NEEDS_ALL_PIECES = true;
  int frag_off;
  __device__ __forceinline__ void init_frag(int sub0, int lane) {
    frag_off = (sub0 + (lane & 31)) * kRowPad + (lane >> 5) * 16;
  }
  template <int i, int KS, int h>
  __device__ __forceinline__ void read(const unsigned char* tile, u32x4& f) const {
    f = *reinterpret_cast<const u32x4*>(tile + frag_off + i * 32 * kRowPad + KS * 32);
  }
};

// ---- B operand stored as fp8 (e4m3) with one bf16 scale per 128x128 block -------------------------
// The fp8 values are widened to bf16 (exact) between the global load and the LDS store, so the MFMA
// side sees an ordinary bf16 tile of 64 reduction elements.  Tiles are 128 outer indices wide and
// start on a multiple of 128, and two K tiles make one 128-block: the scale is uniform over a tile,
// and the kernel applies it in fp32 to the partial sums of each block.
// Reduction index contiguous: element (o, k) at src + o*ld + k (bytes).  Thread t covers the
// 16 reduction elements t%4 of rows t/4 + 64*i.
template <int R, int DEPTH = 1>
struct Fp8DirectLoader {
  static constexpr int BK = 64;
  static constexpr int NPIECE = R / 64;
  u32x4 r[DEPTH][NPIECE];
  uint32_t voff[NPIECE];
  __amdgpu_buffer_rsrc_t rsrc;
  Fp8Scale scale;
  int64_t k_lim;
  int kchunk;
  int lds_off;

  __device__ __forceinline__ void init(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k_limit, int tid) {
    const int c = tid & 3, r0 = tid >> 2;
    int64_t rows = o_lim - o0;
    rows = rows < 0 ? 0 : (rows > R ? R : rows);
    rsrc = make_rsrc(src + o0 * ld, rows * ld);
    k_lim = k_limit;
    kchunk = c * 16;
#pragma unroll
    for (int i = 0; i < NPIECE; ++i) voff[i] = (uint32_t)((int64_t)(r0 + 64 * i) * ld + c * 16);
    lds_off = r0 * kRowPad + c * 32;
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void load_piece(int kt) {
    const bool kok = (int64_t)kt * BK + kchunk < k_lim;
    r[SET][i] = buf_ld16(rsrc, kok ? voff[i] : kOob, (uint32_t)(kt * BK));
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void store_piece(unsigned char* stage) const {
    u32x4 lo, hi;
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      lo[2 * d] = fp8x2_to_bf16x2(r[SET][i][d], false);
      lo[2 * d + 1] = fp8x2_to_bf16x2(r[SET][i][d], true);
      hi[2 * d] = fp8x2_to_bf16x2(r[SET][i][2 + d], false);
      hi[2 * d + 1] = fp8x2_to_bf16x2(r[SET][i][2 + d], true);
    }
    unsigned char* dst = stage + lds_off + i * 64 * kRowPad;
    *reinterpret_cast<u32x4*>(dst) = lo;
    *reinterpret_cast<u32x4*>(dst + 16) = hi;
  }
  // fragment side: 16 bytes (8 reduction elements of the lane's row) per K step, one LDS read
  static constexpr int STAGE_BYTES = R * kRowPad;
  static constexpr int READS = 1;
  static constexpr bool STORE_NEEDS_ALL_PIECES = false;
  int frag_off;
  __device__ __forceinline__ void init_frag(int sub0, int lane) {
    frag_off = (sub0 + (lane & 31)) * kRowPad + (lane >> 5) * 16;
  }
  template <int i, int KS, int h>
  __device__ __forceinline__ void read(const unsigned char* tile, u32x4& f) const {
    f = *reinterpret_cast<const u32x4*>(tile + frag_off + i * 32 * kRowPad + KS * 32);
  }
};

// Reduction index is the slow dimension: element (o, k) at src + k*ld + o.  Thread t owns the
// block of 4 outer indices t%32 x 8 reduction elements t/32: eight 4-byte loads (a wavefront
// reads 128 contiguous bytes of two rows), four 16-byte LDS rows.
template <int R, int DEPTH = 1>
struct Fp8TransposeLoader {
  static_assert(R == 128, "one pass of 32 x 4 outer indices");
  static constexpr int BK = 64;
  static constexpr int NPIECE = 8;  // loads; stores are pieces 0..3
  uint32_t r[DEPTH][8];
  uint32_t voff;
  uint32_t row_bytes;
  __amdgpu_buffer_rsrc_t rsrc;
  Fp8Scale scale;
  int lds_off;

  __device__ __forceinline__ void init(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k_limit, int tid) {
    (void)o_lim;
    const int ob = tid & 31, kb = tid >> 5;
    rsrc = make_rsrc(src + o0, k_limit * ld - o0);
    row_bytes = (uint32_t)ld;
    voff = (uint32_t)((int64_t)(kb * 8) * ld + ob * 4);
    lds_off = (ob * 4) * kRowPad + kb * 16;
  }
  template <int q, int SET = 0>
  __device__ __forceinline__ void load_piece(int kt) {
    r[SET][q] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)voff,
                                                          (int)((uint32_t)(kt * BK + q) * row_bytes), 0);
  }
  template <int q, int SET = 0>
  __device__ __forceinline__ void store_piece(unsigned char* stage) const {
    if constexpr (q < 4) {
      u32x4 v;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // bytes q of two consecutive k rows side by side, then one conversion for the pair
        const uint32_t a = r[SET][2 * d], b = r[SET][2 * d + 1];
        const uint32_t pq = q < 2 ? __builtin_amdgcn_perm(b, a, 0x05010400u)   // a.b0 b.b0 a.b1 b.b1
                                  : __builtin_amdgcn_perm(b, a, 0x07030602u);  // a.b2 b.b2 a.b3 b.b3
        v[d] = fp8x2_to_bf16x2(pq, (q & 1) != 0);
      }
      *reinterpret_cast<u32x4*>(stage + lds_off + q * kRowPad) = v;
    }
  }
  // fragment side: 16 bytes (8 reduction elements of the lane's row) per K step, one LDS read
  static constexpr int STAGE_BYTES = R * kRowPad;
  static constexpr int READS = 1;
  static constexpr bool STORE_NEEDS_ALL_PIECES = true;
  int frag_off;
  __device__ __forceinline__ void init_frag(int sub0, int lane) {
    frag_off = (sub0 + (lane & 31)) * kRowPad + (lane >> 5) * 16;
  }
  template <int i, int KS, int h>
  __device__ __forceinline__ void read(const unsigned char* tile, u32x4& f) const {
    f = *reinterpret_cast<const u32x4*>(tile + frag_off + i * 32 * kRowPad + KS * 32);
  }
};

// Reduction index is the slow dimension (16-bit types, 256 outer indices): element (o, k) at
// src + k*ld + o.  The tile is kept in LDS as it is in memory, [k][outer] with 512-byte rows, in
// two blocks of 32 k rows; MFMA fragments are read with the transposing LDS load
// (ds_read_b64_tr_b16: a group of 16 lanes reads a 4(k) x 16(outer) block and every lane receives
// the 4 k-values of its own outer index), two reads per fragment and K step.  No register
// transposition.  Bank conflicts: the 64-byte segment sg of row k sits at segment position
// sg ^ f(k), f(k) = (k & 3) | ((k >> 1) & 4), so the 8 rows one transposing read touches
// (k0..k0+3 and k0+8..k0+11) land in 8 different segments.
// Thread t copies the 16-byte piece t%32 of rows t/32 + 8*i: a wavefront reads two whole 512-byte
// rows per instruction.
template <int R>
struct RowMajorLoader {
  static_assert(R == 256, "512-byte LDS rows");
  static constexpr int BK = 64;
  static constexpr int NPIECE = 8;
  static constexpr int STAGE_BYTES = BK * R * 2;
  static constexpr int READS = 2;
  static constexpr bool STORE_NEEDS_ALL_PIECES = false;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) unsigned char lds_byte;
  u32x4 r[NPIECE];
  uint32_t voff;
  uint32_t row_bytes;
  __amdgpu_buffer_rsrc_t rsrc;
  int lds_off[2];        // store offset of the pieces with even / odd index
  uint32_t frag_k;       // byte offset of the lane's first k row
  uint32_t frag_seg[4];  // byte offset of the lane's 8 bytes inside a k row, per fragment

  // glu_gap > 0: tile columns 0..127 are outer indices o0..o0+127 (gate), columns 128..255 are
  // o0+glu_gap.. (the matching up-projection columns)
  __device__ __forceinline__ void init(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k_limit, int tid, int64_t glu_gap = 0) {
    (void)o_lim;  // outer indices past the operand only feed rows / columns of C that are not stored
    const int c = tid & 31, t5 = tid >> 5;
    rsrc = make_rsrc(src + o0 * 2, k_limit * ld * 2 - o0 * 2);
    row_bytes = (uint32_t)(ld * 2);
    const int64_t col = (glu_gap > 0 && c >= 16) ? glu_gap + (c - 16) * 8 : c * 8;
    voff = (uint32_t)(((int64_t)t5 * ld + col) * 2);
    // piece i holds k row (i%4)*8 + t5 of block i/4; f of that row = (t5 & 3) | ((i & 1) << 2)
    const int P0 = ((((c >> 2) ^ (t5 & 3)) << 2) | (c & 3));
    lds_off[0] = t5 * 512 + P0 * 16;
    lds_off[1] = t5 * 512 + (P0 ^ 16) * 16;
  }
  // sub0: first outer index of the wavefront's 128 inside the tile; glu: fragments 0,1 are the
  // wavefront's 64 gate columns, 2,3 the up columns under them
  __device__ __forceinline__ void init_frag(int sub0, int lane, bool glu = false) {
    const int s = lane & 15, g = lane >> 5, half = (lane >> 4) & 1;
    frag_k = (uint32_t)((8 * g + (s >> 2)) * 512);
    const int f = (s >> 2) | (g << 2);
    const int seg0 = sub0 / 32;  // 0 or 4
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int seg = glu ? (j < 2 ? seg0 / 2 + j : 4 + seg0 / 2 + (j - 2)) : seg0 + j;
      frag_seg[j] = (uint32_t)(((seg ^ f) * 64) + half * 32 + (s & 3) * 8);
    }
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void load_piece(int kt) {
    r[i] = buf_ld16(rsrc, voff, (uint32_t)(kt * BK + i * 8) * row_bytes);
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void store_piece(unsigned char* stage) const {
    *reinterpret_cast<u32x4*>(stage + (i / 4) * 16384 + (i % 4) * 4096 + lds_off[i & 1]) = r[i];
  }
  // half h (4 of the 8 k values) of fragment j of K step KS (0..3)
  template <int j, int KS, int h>
  __device__ __forceinline__ void read(const unsigned char* tile, u32x4& f) const {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(lds_byte*)(tile + (KS / 2) * 16384 + frag_k +
                                                               frag_seg[j] +
                                                               ((KS % 2) * 16 + h * 4) * 512));
    const u32x2 w = __builtin_bit_cast(u32x2, v);
    f[2 * h] = w[0];
    f[2 * h + 1] = w[1];
  }
};

// The same idea for the 128-wide tiles of the small configuration: [k][outer] rows of 256 bytes,
// the 64-byte segment sg of row k at segment position sg ^ (k & 3).  Half of a transposing read
// (32 lanes) touches 4 consecutive k rows x 2 column halves of one logical segment: after the
// swizzle 8 different 32-byte pieces, all 64 banks once.  Thread t copies the 16-byte piece t%16 of
// rows t/16 + 16*i.
template <int R, int DEPTH>
struct RowMajorSmallLoader {
  static_assert(R == 128, "256-byte LDS rows");
  static constexpr int BK = 64;
  static constexpr int NPIECE = 4;
  static constexpr int STAGE_BYTES = BK * R * 2;
  static constexpr int READS = 2;
  static constexpr bool STORE_NEEDS_ALL_PIECES = false;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) unsigned char lds_byte;
  u32x4 r[DEPTH][NPIECE];
  uint32_t voff;
  uint32_t row_bytes;
  __amdgpu_buffer_rsrc_t rsrc;
  int lds_off;
  uint32_t frag_off[2];  // per fragment (32 outer indices) of the wavefront's 64

  __device__ __forceinline__ void init(const unsigned char* src, int64_t ld, int64_t o0,
                                       int64_t o_lim, int64_t k_limit, int tid) {
    (void)o_lim;  // outer indices past the operand only feed rows / columns of C that are not stored
    const int c = tid & 15, t4 = tid >> 4;
    rsrc = make_rsrc(src + o0 * 2, k_limit * ld * 2 - o0 * 2);
    row_bytes = (uint32_t)(ld * 2);
    voff = (uint32_t)(((int64_t)t4 * ld + c * 8) * 2);
    // piece i holds k row 16*i + t4, whose k & 3 is t4 & 3
    lds_off = t4 * 256 + (((c >> 2) ^ (t4 & 3)) * 64) + (c & 3) * 16;
  }
  __device__ __forceinline__ void init_frag(int sub0, int lane) {
    const int s = lane & 15, g = lane >> 5, half = (lane >> 4) & 1;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      frag_off[j] = (uint32_t)((8 * g + (s >> 2)) * 256 + (((sub0 / 32 + j) ^ (s >> 2)) * 64) +
                               half * 32 + (s & 3) * 8);
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void load_piece(int kt) {
    r[SET][i] = buf_ld16(rsrc, voff, (uint32_t)(kt * BK + i * 16) * row_bytes);
  }
  template <int i, int SET = 0>
  __device__ __forceinline__ void store_piece(unsigned char* stage) const {
    *reinterpret_cast<u32x4*>(stage + i * 16 * 256 + lds_off) = r[SET][i];
  }
  // half h (4 of the 8 k values) of fragment j of K step KS (0..3)
  template <int j, int KS, int h>
  __device__ __forceinline__ void read(const unsigned char* tile, u32x4& f) const {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(lds_byte*)(tile + frag_off[j] +
                                                               (KS * 16 + h * 4) * 256));
    const u32x2 w = __builtin_bit_cast(u32x2, v);
    f[2 * h] = w[0];
    f[2 * h + 1] = w[1];
  }
};

// DEPTH register sets per operand: with 2, a piece is requested two K tiles before it is staged.
template <int R, int ES, bool TRANSPOSE, int DEPTH>
struct Loader : DirectLoader<R, ES, DEPTH> {};
template <int R, int ES, int DEPTH>
struct Loader<R, ES, true, DEPTH> : TransposeLoader<R, ES, DEPTH> {};
template <int R, bool TRANSPOSE, int DEPTH>
struct Fp8Loader : Fp8DirectLoader<R, DEPTH> {};
template <int R, int DEPTH>
struct Fp8Loader<R, true, DEPTH> : Fp8TransposeLoader<R, DEPTH> {};

// ROWS_AUTO_MAIN / ROWS_AUTO_REMAINDER -> ROWS_MAIN / ROWS_REMAINDER when leaving the experts' short
// last row tiles to their own launch saves more time in the launch with 256-row tiles (whole rounds
// of its persistent grid) than the second launch takes, else ROWS_ALL / ROWS_NONE.  Both launches
// evaluate the same counts and the same model, so they agree.  Times in microseconds per 128-byte
// K tile, measured on the Mixtral shape: 1.3 in a 256x256 tile; in a 128x128 tile 2.5 with two
// workgroups per CU walking whole reductions, 1.9 when the reduction is split.
__device__ inline int resolve_row_part(const GmmParams& p, int k_tiles, int* counts) {
  if (p.row_part != ROWS_AUTO_MAIN && p.row_part != ROWS_AUTO_REMAINDER) return p.row_part;
  const int tid = threadIdx.x;
  if (tid < 3) counts[tid] = 0;
  __syncthreads();
  int all = 0, main = 0, rem = 0;
  for (int e = tid; e < p.E; e += kGemmThreads) {
    const long long n = group_begin(p, e + 1) - group_begin(p, e);
    long long b, c;
    all += (int)((n + 255) / 256);
    expert_row_part(n, ROWS_MAIN, b, c);
    main += (int)((c + 255) / 256);
    expert_row_part(n, ROWS_REMAINDER, b, c);
    rem += (int)((c + 127) / 128);
  }
  if (all) atomicAdd(&counts[0], all);
  if (main) atomicAdd(&counts[1], main);
  if (rem) atomicAdd(&counts[2], rem);
  __syncthreads();
  const long long nt256 = (p.M + 255) / 256, nt128 = (p.M + 127) / 128;
  const long long tiles_all = counts[0] * nt256, tiles_main = counts[1] * nt256, tiles_rem = counts[2] * nt128;
  const long long g = p.main_grid > 0 ? p.main_grid : 256;
  const long long rounds_saved = (tiles_all + g - 1) / g - (tiles_main + g - 1) / g;
  long long s = 1;
  if (tiles_rem > 0 && p.ws != nullptr) {
    s = kSplitSlots / tiles_rem;
    if (s > kMaxSplit) s = kMaxSplit;
    if (s > k_tiles) s = k_tiles;
    if (s < 2 || s * tiles_rem * 128 * 128 > p.ws_floats) s = 1;
  }
  const float saved = 1.3f * (float)(rounds_saved * k_tiles);
  const float cost = s > 1 ? 1.9f * (float)(k_tiles / s) + 24.f
                           : 2.5f * (float)(((tiles_rem + kSplitSlots - 1) / kSplitSlots) * k_tiles) + 8.f;
  const bool use = tiles_rem > 0 && saved > cost;
  __syncthreads();  // the caller reuses counts
  if (p.row_part == ROWS_AUTO_MAIN) return use ? ROWS_MAIN : ROWS_ALL;
  return use ? ROWS_REMAINDER : ROWS_NONE;
}

// The row passes of the fused activation backward's epilogue, out of line so that its registers are
// allocated apart from the main loop's: the tile of d(act) is staged in LDS (CTile layout); the fc1
// rows of the next batch of passes are requested before the current batch is computed and stored.
// Every row of the tile exists (the caller takes the guarded loop for ragged tiles), so the loads
// carry no conditions and the waits count exactly the loads they need.
template <int DT, int BM, int BN, bool GELU, int PB>
__attribute__((noinline)) __device__ void glu_bwd_tile_rows(const unsigned char* lds,
                                                            const unsigned char* fc1, unsigned char* dfc1,
                                                            int64_t row_stride, int64_t half, int cc,
                                                            int r0) {
  using CT = CTile<BN>;
  constexpr int NPASS = BM / CT::rows_per_pass, NBATCH = NPASS / PB;
  static_assert(NPASS % PB == 0, "whole batches");
  // out of line the pointers no longer carry their address space: say that they are global, or the
  // accesses become flat ones, whose waits cannot tell loads from LDS reads
  typedef __attribute__((address_space(1))) u32x4 global_u32x4;
  auto ld16_nt = [](const unsigned char* q) {
    return __builtin_nontemporal_load((const global_u32x4*)q);
  };
  auto st16 = [](unsigned char* q, const u32x4& v) { *(global_u32x4*)q = v; };
  u32x4 gq[2][PB], uq[2][PB];
  // fc1 / dfc1 point at this thread's 16 bytes of row r0; a pass advances rows_per_pass rows
  auto request = [&](auto buf_c, int b) __attribute__((always_inline)) {
    constexpr int BUF = decltype(buf_c)::value;
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      const int64_t o = (int64_t)(b * PB + j) * CT::rows_per_pass * row_stride;
      gq[BUF][j] = ld16_nt(fc1 + o);
      uq[BUF][j] = ld16_nt(fc1 + o + half);
    }
  };
  auto finish = [&](auto buf_c, int b) __attribute__((always_inline)) {
    constexpr int BUF = decltype(buf_c)::value;
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      const int row = (b * PB + j) * CT::rows_per_pass + r0;
      const int64_t o = (int64_t)(b * PB + j) * CT::rows_per_pass * row_stride;
      float d[8], g[8], u[8], dg[8], du[8];
      Vec16<DT>::unpack(ctile_read16(lds + row * CT::pitch + cc * 16), d);
      Vec16<DT>::unpack(gq[BUF][j], g);
      Vec16<DT>::unpack(uq[BUF][j], u);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        dg[q] = d[q] * glu_act_grad(g[q], GELU) * u[q];
        du[q] = d[q] * glu_act(g[q], GELU);
      }
      st16(dfc1 + o, Vec16<DT>::pack(dg));
      st16(dfc1 + o + half, Vec16<DT>::pack(du));
    }
  };
  request(std::integral_constant<int, 0>{}, 0);
  GMOE_SCHED_FENCE();
  static_for<0, NBATCH>([&](auto b_c) __attribute__((always_inline)) {
    constexpr int b = decltype(b_c)::value;
    if constexpr (b + 1 < NBATCH) request(std::integral_constant<int, (b + 1) & 1>{}, b + 1);
    GMOE_SCHED_FENCE();
    finish(std::integral_constant<int, b & 1>{}, b);
    GMOE_SCHED_FENCE();
  });
}

// ---- the kernel -----------------------------------------------------------------------------------
// BQ: the B operand is fp8 with block scales (p.b_scale), DT is then the type of A and of the MFMA.
// TR: operands whose reduction index is the slow dimension keep their memory layout in LDS and are
// read with transposing LDS loads (RowMajorLoader) instead of being transposed in registers.
template <int DT, int ODT, int MODE, int BM, int BN, int EPI, bool BQ = false, bool TR = false>
__global__ __launch_bounds__(kGemmThreads, (BM == 128 && BN == 128) ? 2 : 1) void gmm_kernel(GmmParams p) {
  constexpr bool GLU = (EPI == EPI_GLU_FWD_SILU || EPI == EPI_GLU_FWD_GELU);
  static_assert(!GLU || (MODE == MODE_NN && TR && DT == ODT), "fused activation: forward GEMM");
  static_assert(!TR || (Elem<DT>::bytes == 2 && BM == 256 && BN == 256 && !BQ), "TR: 16-bit, 256x256");
  constexpr int ES = Elem<DT>::bytes;
  constexpr int BK = 128 / ES;      // reduction elements per LDS row
  constexpr int WTM = BM / 2 / 32;  // 32x32 accumulators per wavefront, rows
  constexpr int WTN = BN / 2 / 32;  // ... columns
  constexpr int NM = WTM * WTN;     // MFMA groups per K step
  constexpr bool A_T = (MODE == MODE_TN);
  constexpr bool B_T = (MODE != MODE_NT);
  // The small tiles leave registers for a second set of staging pieces: their loads then have two
  // K tiles of MFMAs to land (one K tile is only 4 MFMAs per wavefront and step there).  With fp8
  // weights the second accumulator takes that room and only the weight stream gets the second set.
  constexpr bool SMALL = BM == 128 && BN == 128;
  constexpr int DA = (SMALL && !BQ) ? 2 : 1, DB = SMALL ? 2 : 1;
  // 16-bit operands whose reduction index is the slow dimension: transposing LDS reads (TR for the
  // large tiles, always for the small ones); fp32 transposes 4x4 blocks in registers
  constexpr bool TRS = SMALL && ES == 2 && !BQ;
  typedef std::conditional_t<
      TR && A_T, RowMajorLoader<BM>,
      std::conditional_t<TRS && A_T, RowMajorSmallLoader<BM, DA>, Loader<BM, ES, A_T, DA>>> LoaderA;
  typedef std::conditional_t<
      BQ, Fp8Loader<BN, B_T, DB>,
      std::conditional_t<TR && B_T, RowMajorLoader<BN>,
                         std::conditional_t<TRS && B_T, RowMajorSmallLoader<BN, DB>,
                                            Loader<BN, ES, B_T, DB>>>> LoaderB;
  constexpr int RA = LoaderA::READS, RB = LoaderB::READS;
  constexpr int NF = WTM * RA + WTN * RB;  // LDS fragment reads per K step
  constexpr int A_BYTES = LoaderA::STAGE_BYTES;
  constexpr int B_BYTES = LoaderB::STAGE_BYTES;
  constexpr int STAGE = A_BYTES + B_BYTES;
  static_assert(!BQ || (DT == GMOE_BF16 && MODE != MODE_TN && BN == 128), "fp8 weights: bf16 NN / NT");
  constexpr int NPA = LoaderA::NPIECE, NPB = LoaderB::NPIECE;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  __shared__ int tile_cum[kMaxGroupsLds + 1];  // exclusive prefix of tiles per expert
  GMOE_PROBE_WORKGROUP_BEGIN();

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  const int E = p.E;
  const int64_t K = p.K, M = p.M;
  // C is rows x M per expert: NN/NT rows = tokens of the expert;  TN rows = K
  // with the fused activation a column tile is 128 gate + 128 up columns of the [K, 2F] weight
  const int nt_cnt = GLU ? (int)((p.F + 127) / 128) : (int)((M + BN - 1) / BN);
  const int mt_fixed = (int)((K + BM - 1) / BM);  // TN only

  int part = ROWS_ALL;
  if constexpr (MODE != MODE_TN) {
    part = resolve_row_part(p, (int)((K + BK - 1) / BK), tile_cum);
    if (part == ROWS_NONE) return;  // the launch with 256-row tiles takes every row
  }

  {
    // tiles per expert -> exclusive prefix in one pass: a thread owns kPer consecutive experts, the
    // per-thread sums are scanned with wavefront shuffles and four wavefront totals in LDS
    constexpr int kPer = kMaxGroupsLds / kGemmThreads;
    __shared__ int wave_tot[kGemmThreads / 64];
    int cnt[kPer], local = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int e = tid * kPer + j;
      int c = 0;
      if (e < E) {
        long long n = group_begin(p, e + 1) - group_begin(p, e), skip;
        if (MODE != MODE_TN) expert_row_part(n, part, skip, n);
        const long long mt = MODE == MODE_TN ? mt_fixed : (n + BM - 1) / BM;
        c = (int)(mt * nt_cnt);
      }
      cnt[j] = c;
      local += c;
    }
    int incl = local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(incl, d);
      if (lane >= d) incl += o;
    }
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    int run = incl - local;
    for (int w = 0; w < wave; ++w) run += wave_tot[w];
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int e = tid * kPer + j;
      if (e <= E) tile_cum[e] = run;
      run += cnt[j];
    }
    if (tid == kGemmThreads - 1) tile_cum[E] = run;  // experts past E add nothing: the total
  }
  __syncthreads();
  const long long total_tiles = tile_cum[E];

  // A launch with few tiles and a long reduction (the short last row tiles of the experts) leaves
  // most CUs idle while each workgroup walks the whole K range.  With a workspace it runs twice:
  // SPLIT_PARTIAL cuts the reduction of every tile into S pieces, one workgroup each, which store
  // their fp32 accumulators; SPLIT_REDUCE adds the S partial tiles in order and runs the epilogue.
  // S depends only on launch parameters and the tile count, so both launches agree on it.
  constexpr bool CAN_SPLIT = MODE != MODE_TN && EPI == EPI_NONE && !BQ && SMALL;
  constexpr long long TILE_ELEMS = (long long)BM * BN;
  int S = 1;
  if constexpr (CAN_SPLIT) {
    if (p.phase != SPLIT_OFF && total_tiles > 0) {
      const long long kt_all = (K + BK - 1) / BK;
      long long want = p.split_slots / total_tiles;
      if (want > kMaxSplit) want = kMaxSplit;
      if (want > kt_all) want = kt_all;
      if (want >= 2 && want * total_tiles * TILE_ELEMS <= p.ws_floats) S = (int)want;
    }
    if (p.phase == SPLIT_REDUCE && S == 1) return;  // the first launch did everything
  }
  const bool reduce_phase = CAN_SPLIT && p.phase == SPLIT_REDUCE;
  const long long total_work = (S > 1 && !reduce_phase) ? total_tiles * S : total_tiles;

  // Workgroup w runs on XCD w%8.  Give XCD x the consecutive positions [x*G/8, (x+1)*G/8) of
  // every whole round of G = gridDim.x tiles (G is a multiple of 8).  The tiles of the last, partial
  // round are dealt to the eight XCDs in equal consecutive shares: a launch with fewer tiles than
  // workgroups then runs on every XCD (with two workgroups per CU, one per CU on the whole chip
  // instead of two per CU on half of it).
  const int G = gridDim.x, per_xcd = G / 8;
  const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;

  int e = 0;
  for (long long base = 0; base < total_work; base += G) {
    long long v = base + (long long)xcd * per_xcd + slot;
    if (total_work - base < G) {
      const long long share = (total_work - base + 7) / 8;
      v = base + xcd * share + slot;
      if (slot >= share || v >= total_work) break;
    }
    GMOE_PROBE_TILE_BEGIN();
    const long long s = (S > 1 && !reduce_phase) ? v / S : v;
    const int chunk = (S > 1 && !reduce_phase) ? (int)(v % S) : 0;
    while (tile_cum[e + 1] <= s) ++e;
    long long row0 = group_begin(p, e);
    long long n_e = group_begin(p, e + 1) - row0;
    if (MODE != MODE_TN) {
      long long begin;
      expert_row_part(n_e, part, begin, n_e);
      row0 += begin;
    }
    const int mt_cnt = MODE == MODE_TN ? mt_fixed : (int)((n_e + BM - 1) / BM);
    int mt, nt;
    strip_order(s - tile_cum[e], mt_cnt, nt_cnt, mt, nt);

    f32x16 acc[WTM][WTN];
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WTN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // TN reduces over the expert's rows, and a loader's buffer resource spans at most 2 GiB: an
    // expert with more rows than that is walked in segments (one segment in all but extreme cases),
    // the accumulators carried across.
    const int64_t seg_rows = tn_segment_rows(K, M, ES);
    int64_t seg0 = 0;
    do {
    LoaderA la;
    LoaderB lb;
    la.init_frag(wm * (BM / 2), lane);
    if constexpr (GLU) lb.init_frag(wn * (BN / 2), lane, true);
    else lb.init_frag(wn * (BN / 2), lane);
    int64_t k_lim;
    if constexpr (GLU) {
      k_lim = K;
      la.init(p.a + row0 * K * ES, K, (int64_t)mt * BM, n_e, k_lim, tid);
      lb.init(p.b + (int64_t)e * K * M * ES, M, (int64_t)nt * 128, M, k_lim, tid, p.F);
    } else if constexpr (BQ) {
      // b is [E,K,M] (NN) or [E,M,K] (NT) bytes; its scales [E, ceil(K/128), ceil(M/128)] or
      // [E, ceil(M/128), ceil(K/128)]
      k_lim = K;
      la.init(p.a + row0 * K * ES, K, (int64_t)mt * BM, n_e, k_lim, tid);
      const int kbs = (int)((K + 127) / 128), mbs = (int)((M + 127) / 128);
      const int eu = __builtin_amdgcn_readfirstlane(e), ntu = __builtin_amdgcn_readfirstlane(nt);
      const uint16_t* sbase = reinterpret_cast<const uint16_t*>(p.b_scale) + (int64_t)eu * kbs * mbs;
      lb.scale.last = kbs - 1;
      if (MODE == MODE_NN) {
        lb.init(p.b + (int64_t)e * K * M, M, (int64_t)nt * BN, M, k_lim, tid);
        lb.scale.ptr = sbase + ntu;
        lb.scale.stride = mbs;
      } else {
        lb.init(p.b + (int64_t)e * M * K, K, (int64_t)nt * BN, M, k_lim, tid);
        lb.scale.ptr = sbase + (int64_t)ntu * kbs;
        lb.scale.stride = 1;
      }
    } else if (MODE == MODE_NN || MODE == MODE_NT) {
      // this workgroup's piece [k0, k0 + k_lim) of the reduction: all of it unless split
      int64_t k0 = 0;
      k_lim = K;
      if (S > 1) {
        const int64_t kt_all = (K + BK - 1) / BK;
        const int64_t per = (kt_all + S - 1) / S * BK;
        k0 = reduce_phase ? K : chunk * per;
        if (k0 > K) k0 = K;
        k_lim = reduce_phase ? 0 : (k0 + per < K ? per : K - k0);
      }
      la.init(p.a + (row0 * K + k0) * ES, K, (int64_t)mt * BM, n_e, k_lim, tid);
      if (MODE == MODE_NN)
        lb.init(p.b + ((int64_t)e * K + k0) * M * ES, M, (int64_t)nt * BN, M, k_lim, tid);
      else
        lb.init(p.b + ((int64_t)e * M * K + k0) * ES, K, (int64_t)nt * BN, M, k_lim, tid);
    } else {
      k_lim = n_e - seg0 < seg_rows ? n_e - seg0 : seg_rows;
      la.init(p.a + (row0 + seg0) * K * ES, K, (int64_t)mt * BM, K, k_lim, tid);
      lb.init(p.b + (row0 + seg0) * M * ES, M, (int64_t)nt * BN, M, k_lim, tid);
    }

    // fp8 weights: the MFMAs accumulate the unscaled products of one 128-element scale block here
    f32x16 accq[BQ ? WTM : 1][BQ ? WTN : 1];

    const int kt_cnt = (int)((k_lim + BK - 1) / BK);

    // ---- prologue: tile 0 -> LDS stage 0, tile 1 -> registers, fragments of step 0 ------------
    u32x4 fa[2][WTM], fb[2][WTN];
    if (kt_cnt > 0) {
      static_for<0, NPA>([&](auto i) { la.template load_piece<decltype(i)::value>(0); });
      static_for<0, NPB>([&](auto i) { lb.template load_piece<decltype(i)::value>(0); });
      static_for<0, NPA>([&](auto i) { la.template store_piece<decltype(i)::value>(lds); });
      static_for<0, NPB>([&](auto i) { lb.template store_piece<decltype(i)::value>(lds + A_BYTES); });
      static_for<0, NPA>([&](auto i) { la.template load_piece<decltype(i)::value, DA - 1>(1); });
      static_for<0, NPB>([&](auto i) { lb.template load_piece<decltype(i)::value, DB - 1>(1); });
      if constexpr (DA == 2)
        static_for<0, NPA>([&](auto i) { la.template load_piece<decltype(i)::value, 0>(2); });
      if constexpr (DB == 2)
        static_for<0, NPB>([&](auto i) { lb.template load_piece<decltype(i)::value, 0>(2); });
    }
    __syncthreads();
    // fragment read number r of K step KS of the tile at `stage` into fragment buffer BUF
    auto frag_read = [&](auto r_c, auto ks_c, auto buf_c, const unsigned char* stage) {
      constexpr int r = decltype(r_c)::value, KS = decltype(ks_c)::value, BUF = decltype(buf_c)::value;
      if constexpr (r < WTM * RA) {
        la.template read<r / RA, KS, r % RA>(stage, fa[BUF][r / RA]);
      } else {
        constexpr int rb = r - WTM * RA;
        lb.template read<rb / RB, KS, rb % RB>(stage + A_BYTES, fb[BUF][rb / RB]);
      }
    };
    if (kt_cnt > 0) {
      static_for<0, NF>([&](auto r) {
        frag_read(r, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, lds);
      });
    }

    GMOE_PROBE_MAIN_LOOP_BEGIN();
    // ---- main loop ------------------------------------------------------------------------------
    // Every index below is a compile-time constant (static_for), so fragments and pieces stay in
    // named registers and the loop body is one basic block in exactly this order.
    // one K tile; PAR = kt & 1 at compile time selects the register set of a two-deep operand:
    // set 1-PAR holds tile kt+1 (staged now, then re-requested for tile kt+3), set PAR tile kt+2
    auto k_tile = [&](auto par_c, int kt) {
      constexpr int PAR = decltype(par_c)::value;  // -1: no two-deep operand, parity not needed
      constexpr int SA = DA == 2 ? 1 - PAR : 0, SB = DB == 2 ? 1 - PAR : 0;
      const int par = PAR < 0 ? (kt & 1) : PAR;
      unsigned char* cur = lds + par * STAGE;
      unsigned char* nxt = lds + (1 - par) * STAGE;
      static_for<0, 4>([&](auto ks_c) {
        constexpr int ks = decltype(ks_c)::value;
        // Memory operations of this step, spread between the MFMAs: first the NF fragment reads
        // for the next step (step 3: step 0 of the next tile, from the other stage); then, in steps
        // 0..2, a third of the tile-movement sequence: every register piece of tile kt+1 is
        // written to the other stage and re-requested for tile kt+2 as early as its registers
        // are free, so a request has almost a whole K tile of MFMAs to complete.
        const unsigned char* fsrc = ks < 3 ? cur : nxt;
        constexpr int NMOVE = 2 * (NPA + NPB);
        constexpr int mv_begin = ks < 3 ? (NMOVE * ks + 2) / 3 : NMOVE;
        constexpr int mv_end = ks < 3 ? (NMOVE * (ks + 1) + 2) / 3 : NMOVE;
        constexpr int n_ops = NF + (mv_end - mv_begin);
        if (ks == 3) {
          __syncthreads();
          GMOE_SCHED_FENCE();
        }
        static_for<0, NM>([&](auto m_c) {
          constexpr int m = decltype(m_c)::value;
          if constexpr (BQ) {
            // a scale block starts with every even K tile: its first MFMAs take C = 0
            if constexpr (PAR == 0 && ks == 0) {
              f32x16 zero;
#pragma unroll
              for (int v = 0; v < 16; ++v) zero[v] = 0.f;
              accq[m / WTN][m % WTN] = zero;
            }
            Mma<DT>::run(fa[ks & 1][m / WTN], fb[ks & 1][m % WTN], accq[m / WTN][m % WTN]);
          } else
          {
            // boustrophedon order over the wavefront's fragments: one operand changes per MFMA
            constexpr int mi = m / WTN, mj = (mi & 1) ? WTN - 1 - m % WTN : m % WTN;
            Mma<DT>::run(fa[ks & 1][mi], fb[ks & 1][mj], acc[mi][mj]);
          }
          GMOE_SCHED_FENCE();
          // operations [ceil(m*n/NM), ceil((m+1)*n/NM)) go after MFMA group m
          constexpr int op_begin = (m * n_ops + NM - 1) / NM;
          constexpr int op_end = ((m + 1) * n_ops + NM - 1) / NM;
          static_for<op_begin, op_end>([&](auto op_c) {
            constexpr int op = decltype(op_c)::value;
            if constexpr (op < NF) {
              frag_read(op_c, std::integral_constant<int, (ks + 1) & 3>{},
                        std::integral_constant<int, (ks + 1) & 1>{}, fsrc);
            } else {
              // position g in the sequence [A moves | B moves]; a directly copied operand
              // alternates store i / load i, a transposed one stores all pieces (each needs every
              // loaded row) before it loads again
              constexpr int g = mv_begin + (op - NF);
              constexpr bool is_a = g < 2 * NPA;
              constexpr int j = is_a ? g : g - 2 * NPA;
              constexpr int np = is_a ? NPA : NPB;
              constexpr bool transposed =
                  is_a ? LoaderA::STORE_NEEDS_ALL_PIECES : LoaderB::STORE_NEEDS_ALL_PIECES;
              constexpr bool is_store = transposed ? (j < np) : (j % 2 == 0);
              constexpr int c = transposed ? (j % np) : (j / 2);
              if constexpr (is_a) {
                if constexpr (is_store) { if constexpr (!kProbeNoStaging) la.template store_piece<c, SA>(nxt); }
                else { if constexpr (!kProbeNoLoads) la.template load_piece<c, SA>(kProbeLoadsHitL2 ? 0 : kt + 1 + DA); }
              } else {
                if constexpr (is_store) { if constexpr (!kProbeNoStaging) lb.template store_piece<c, SB>(nxt + A_BYTES); }
                else { if constexpr (!kProbeNoLoads) lb.template load_piece<c, SB>(kProbeLoadsHitL2 ? 0 : kt + 1 + DB); }
              }
            }
          });
          GMOE_SCHED_FENCE();
        });
      });
      if constexpr (BQ) {
        // a 128-element scale block ends: fold its fp32 partial sums into the result
        if ((kt & 1) || kt == kt_cnt - 1) {
          const float sb = lb.scale.at(kt);
#pragma unroll
          for (int i = 0; i < WTM; ++i)
#pragma unroll
            for (int j = 0; j < WTN; ++j)
#pragma unroll
              for (int v = 0; v < 16; ++v) acc[i][j][v] = fmaf(sb, accq[i][j][v], acc[i][j][v]);
        }
      }
    };
    if constexpr (DA == 2 || DB == 2) {
      int kt = 0;
      for (; kt + 1 < kt_cnt; kt += 2) {
        k_tile(std::integral_constant<int, 0>{}, kt);
        k_tile(std::integral_constant<int, 1>{}, kt + 1);
      }
      if (kt < kt_cnt) k_tile(std::integral_constant<int, 0>{}, kt);
    } else {
      for (int kt = 0; kt < kt_cnt; ++kt) k_tile(std::integral_constant<int, -1>{}, kt);
    }
    // the fragment reads issued under the last step target the other stage; the next tile's
    // prologue overwrites stage 0 only after this barrier
    __syncthreads();
    GMOE_PROBE_MAIN_LOOP_END();
    seg0 += seg_rows;
    } while (MODE == MODE_TN && seg0 < n_e);

    if constexpr (CAN_SPLIT) {
      if (S > 1) {
        // partial tiles of tile s: S slots of BM x BN floats, each in accumulator order
        // [fragment][quad][thread] so that a wavefront moves 1 KiB per instruction
        float* slot = p.ws + s * S * TILE_ELEMS;
        if (!reduce_phase) {
          float* mine = slot + (long long)chunk * TILE_ELEMS;
#pragma unroll
          for (int i = 0; i < WTM; ++i)
#pragma unroll
            for (int j = 0; j < WTN; ++j)
#pragma unroll
              for (int vq = 0; vq < 4; ++vq) {
                const f32x4 q = {acc[i][j][4 * vq], acc[i][j][4 * vq + 1], acc[i][j][4 * vq + 2],
                                 acc[i][j][4 * vq + 3]};
                *reinterpret_cast<f32x4*>(mine + ((((i * WTN + j) * 4 + vq) * kGemmThreads) + tid) * 4) = q;
              }
          continue;
        }
        for (int c = 0; c < S; ++c) {
          const float* part = slot + (long long)c * TILE_ELEMS;
#pragma unroll
          for (int i = 0; i < WTM; ++i)
#pragma unroll
            for (int j = 0; j < WTN; ++j)
#pragma unroll
              for (int vq = 0; vq < 4; ++vq) {
                const f32x4 q = *reinterpret_cast<const f32x4*>(
                    part + ((((i * WTN + j) * 4 + vq) * kGemmThreads) + tid) * 4);
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[i][j][4 * vq + t] += q[t];
              }
        }
      }
    }

    // ---- epilogue: lane holds row (lane%32), columns 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 ----
    constexpr int OES = Elem<ODT>::bytes;
    if constexpr (GLU) {
      // fragments 0,1 hold gate columns, 2,3 the up columns under them: fc1 = [gate | up] and
      // act = act_fn(gate) * up, both computed from the values as rounded for fc1.  Staged through
      // LDS (columns [gate 64 | up 64] per wavefront column half), then written in 16-byte
      // row-contiguous pieces.
      constexpr bool gelu = EPI == EPI_GLU_FWD_GELU;
      const int64_t F = p.F;
      unsigned char* fc1 = p.c + row0 * M * 2;
      unsigned char* act = p.c2 + row0 * F * 2;
      using CT = CTile<BN>;
      stage_acc_lds<DT, WTM, WTN, BN>(lds, acc, wm * (BM / 2), wn * (BN / 2), lane);
      __syncthreads();
      const int cc = tid & 15, r0 = tid >> 4;  // 16 chunks of 8 gate columns per row
      const int64_t n = (int64_t)nt * 128 + cc * 8;
      const int lcol = (cc >> 3) * 128 + (cc & 7) * 8;
#pragma unroll 4
      for (int it = 0; it < BM / 16; ++it) {
        const int row = it * 16 + r0;
        const int64_t m = (int64_t)mt * BM + row;
        if (m >= n_e || n >= F) continue;
        const u32x4 gw = ctile_read16(lds + row * CT::pitch + lcol * 2);
        const u32x4 uw = ctile_read16(lds + row * CT::pitch + (lcol + 64) * 2);
        float g[8], u[8], o[8];
        Vec16<DT>::unpack(gw, g);
        Vec16<DT>::unpack(uw, u);
#pragma unroll
        for (int q = 0; q < 8; ++q) o[q] = glu_act(g[q], gelu) * u[q];
        st16(fc1 + (m * M + n) * 2, gw);
        st16(fc1 + (m * M + F + n) * 2, uw);
        st16(act + (m * F + n) * 2, Vec16<DT>::pack(o));
      }
      __syncthreads();  // the next tile's prologue writes stage 0
      continue;
    }
    if constexpr (EPI == EPI_GLU_BWD_SILU || EPI == EPI_GLU_BWD_GELU) {
      // C = d(act) is not stored: with fc1 = [gate | up] read back, the tile of
      // d(fc1) = [d * act'(gate) * up | d * act(gate)] is written instead (d rounded to the
      // storage type first, as a separate activation-backward kernel would see it)
      static_assert(MODE == MODE_NT && DT == ODT, "fused activation backward follows the dX GEMM");
      constexpr bool gelu = EPI == EPI_GLU_BWD_GELU;
      const int64_t F = M;
      const unsigned char* fc1 = p.aux + row0 * 2 * F * OES;
      unsigned char* dfc1 = p.c + row0 * 2 * F * OES;
      if constexpr (DT != GMOE_F32) {
        // d goes through LDS so that fc1 is read and d(fc1) written in 16-byte, row-contiguous
        // pieces (the accumulator layout would touch 32 rows per instruction, 8 bytes each)
        using CT = CTile<BN>;
        stage_acc_lds<DT, WTM, WTN, BN>(lds, acc, wm * (BM / 2), wn * (BN / 2), lane);
        __syncthreads();
        const int cc = tid % CT::chunks, r0 = tid / CT::chunks;
        const int64_t n = (int64_t)nt * BN + cc * 8;
        if ((int64_t)mt * BM + BM <= n_e && (int64_t)nt * BN + BN <= F) {
          // a whole tile: the passes without guards, two at a time, the next two requested ahead
          // (15.9 instead of 30.5 us per tile: a CU with four wavefronts has too few bytes in
          // flight when every batch of loads is waited for before the next is requested)
          const int64_t o0 = (((int64_t)mt * BM + r0) * 2 * F + n) * OES;
          glu_bwd_tile_rows<DT, BM, BN, gelu, 2>(lds, fc1 + o0, dfc1 + o0, 2 * F * OES, F * OES, cc, r0);
          __syncthreads();  // the next tile's prologue writes stage 0
          continue;
        }
#pragma unroll 4
        for (int it = 0; it < BM / CT::rows_per_pass; ++it) {
          const int row = it * CT::rows_per_pass + r0;
          const int64_t m = (int64_t)mt * BM + row;
          if (m >= n_e || n >= F) continue;
          const int64_t og = (m * 2 * F + n) * OES, ou = og + F * OES;
          float d[8], g[8], u[8], dg[8], du[8];
          Vec16<DT>::unpack(ctile_read16(lds + row * CT::pitch + cc * 16), d);
          Vec16<DT>::unpack(ld16_nt(fc1 + og), g);
          Vec16<DT>::unpack(ld16_nt(fc1 + ou), u);
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            dg[q] = d[q] * glu_act_grad(g[q], gelu) * u[q];
            du[q] = d[q] * glu_act(g[q], gelu);
          }
          st16(dfc1 + og, Vec16<DT>::pack(dg));
          st16(dfc1 + ou, Vec16<DT>::pack(du));
        }
        __syncthreads();  // the next tile's prologue writes stage 0
        continue;
      }
      if (SMALL && !gelu && (int64_t)mt * BM + BM <= n_e && (int64_t)nt * BN + BN <= F) {
        // a whole tile, straight from the accumulators: the 8 fc1 loads of the next 32x32 block are
        // requested before the current block is computed and stored (fc1 and d(fc1) may alias as
        // far as the compiler knows, so in the guarded loop below every load waits for the stores
        // before it: 22 us per tile with one 16-byte load in flight per lane).  Not for the large
        // tiles and the GELU form, which have no registers to spare for the second set of loads.
        const unsigned char* src = fc1 + (((int64_t)mt * BM + wm * (BM / 2) + (lane & 31)) * 2 * F +
                                          (int64_t)nt * BN + wn * (BN / 2) + 4 * (lane >> 5)) * OES;
        unsigned char* dst = dfc1 + (src - fc1);
        f32x4 gq[2][4], uq[2][4];
        auto request = [&](auto buf_c, auto blk_c) {
          constexpr int BUF = decltype(buf_c)::value, i = decltype(blk_c)::value / WTN, j = decltype(blk_c)::value % WTN;
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int64_t o = ((int64_t)i * 32 * 2 * F + j * 32 + 8 * vq) * OES;
            gq[BUF][vq] = *reinterpret_cast<const f32x4*>(src + o);
            uq[BUF][vq] = *reinterpret_cast<const f32x4*>(src + o + F * OES);
          }
        };
        request(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
        GMOE_SCHED_FENCE();
        static_for<0, NM>([&](auto blk_c) {
          constexpr int blk = decltype(blk_c)::value, i = blk / WTN, j = blk % WTN, BUF = blk & 1;
          if constexpr (blk + 1 < NM)
            request(std::integral_constant<int, (blk + 1) & 1>{}, std::integral_constant<int, blk + 1>{});
          GMOE_SCHED_FENCE();
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int64_t o = ((int64_t)i * 32 * 2 * F + j * 32 + 8 * vq) * OES;
            f32x4 dg, du;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float d = acc[i][j][4 * vq + q];
              dg[q] = d * glu_act_grad(gq[BUF][vq][q], gelu) * uq[BUF][vq][q];
              du[q] = d * glu_act(gq[BUF][vq][q], gelu);
            }
            *reinterpret_cast<f32x4*>(dst + o) = dg;
            *reinterpret_cast<f32x4*>(dst + o + F * OES) = du;
          }
          GMOE_SCHED_FENCE();
        });
        continue;
      }
#pragma unroll
      for (int i = 0; i < WTM; ++i) {
        const int64_t m = (int64_t)mt * BM + wm * (BM / 2) + i * 32 + (lane & 31);
        if (m >= n_e) continue;
#pragma unroll
        for (int j = 0; j < WTN; ++j) {
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int64_t n = (int64_t)nt * BN + wn * (BN / 2) + j * 32 + 8 * vq + 4 * (lane >> 5);
            if (n >= F) continue;
            const int64_t og = (m * 2 * F + n) * OES, ou = (m * 2 * F + F + n) * OES;
            const f32x4 gv = *reinterpret_cast<const f32x4*>(fc1 + og);
            const f32x4 uv = *reinterpret_cast<const f32x4*>(fc1 + ou);
            f32x4 dg, du;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float d = acc[i][j][4 * vq + q];
              dg[q] = d * glu_act_grad(gv[q], gelu) * uv[q];
              du[q] = d * glu_act(gv[q], gelu);
            }
            *reinterpret_cast<f32x4*>(dfc1 + og) = dg;
            *reinterpret_cast<f32x4*>(dfc1 + ou) = du;
          }
        }
      }
      continue;
    }
    unsigned char* c_base;
    int64_t c_rows;
    if (MODE == MODE_TN) {
      c_base = p.c + (int64_t)e * K * M * OES;
      c_rows = K;
    } else {
      c_base = p.c + row0 * M * OES;
      c_rows = n_e;
    }
    if constexpr (ODT != GMOE_F32) {
      using CT = CTile<BN>;
      stage_acc_lds<ODT, WTM, WTN, BN>(lds, acc, wm * (BM / 2), wn * (BN / 2), lane);
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
      __syncthreads();  // the next tile's prologue writes stage 0
      continue;
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
          if (ODT == GMOE_F32)
            *reinterpret_cast<f32x4*>(dst) = f32x4{v0, v1, v2, v3};
          else
            *reinterpret_cast<u32x2*>(dst) = pack4<ODT>(v0, v1, v2, v3);
        }
      }
    }
  }
  GMOE_PROBE_WORKGROUP_END();
}

// Persistent grid: blocks_per_cu workgroups per CU, a multiple of 8 (one share per XCD).
static int gmm_grid(int blocks_per_cu) {
  const int grid = (gmoe_cu_count() / 8) * 8 * blocks_per_cu;
  return grid < 8 ? 8 : grid;
}

template <int DT, int ODT, int MODE, int BM, int BN, int EPI, bool BQ = false, bool TR = false>
static int launch_gmm_cfg(const GmmParams& p, hipStream_t st, int blocks_per_cu = 1) {
  // two stages of both operand tiles; the epilogue reuses them as one tile of 16-bit results
  constexpr bool small_tr = BM == 128 && BN == 128 && Elem<DT>::bytes == 2 && !BQ;
  constexpr size_t a_bytes = MODE != MODE_TN ? BM * kRowPad : ((TR || small_tr) ? 64 * BM * 2 : BM * kRowPad);
  constexpr size_t b_bytes = MODE == MODE_NT ? BN * kRowPad : ((TR || small_tr) ? 64 * BN * 2 : BN * kRowPad);
  constexpr size_t ctile = Elem<ODT>::bytes == 2 ? (size_t)BM * CTile<BN>::pitch : 0;
  constexpr size_t smem = 2 * (a_bytes + b_bytes) > ctile ? 2 * (a_bytes + b_bytes) : ctile;
  auto kern = gmm_kernel<DT, ODT, MODE, BM, BN, EPI, BQ, TR>;
  if (smem > 48 * 1024) {
    // once per kernel and device (the attribute belongs to the device's copy of the code object)
    static std::atomic<uint64_t> done_mask{0};
    if (!gmoe_once_per_device(done_mask, [&] {
          return hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess;
        }))
      return GMOE_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(kern, dim3(gmm_grid(blocks_per_cu)), dim3(kGemmThreads), smem, st, p);
  return gmoe_launch_status();
}

// Large tiles once an expert's share of rows (NN/NT) or the output itself (TN) can fill them and
// there are enough of them for every CU; smaller problems spread over more, smaller tiles.
static inline bool gmm_large_tiles(const GmmParams& p, int mode) {
  const int64_t experts = p.E > 0 ? p.E : 1;
  const int64_t rows_per_expert = mode == MODE_TN ? p.K : p.N / experts;
  if (rows_per_expert < 512 || p.M < 256) return false;
  const int64_t col_tiles = (p.M + 255) / 256;
  const int64_t tiles = mode == MODE_TN ? experts * ((p.K + 255) / 256) * col_tiles
                                        : ((p.N + 255) / 256) * col_tiles;
  // TN: the 128x128 kernel runs at about 0.4 of the large one's rate per FLOP, so the large tiles win
  // as soon as the small ones need a second round of their 512 slots (C3's shared experts, 176 large
  // tiles: 0.29 -> 0.22 ms)
  return tiles >= (mode == MODE_TN ? 129 : 256);
}

// The separate launch for short last row tiles pays off once an expert has many full row tiles:
// at 4096 rows per expert (Mixtral shape) it saves 4-7 % of a GEMM, at 1024 rows per expert (64 or 32
// experts) the main kernel with its partial tiles is 5-10 % faster than the two launches.
constexpr int64_t kRemainderMinRows = 2048;
static inline bool gmm_use_remainder(const GmmParams& p) {
  return p.N / (p.E > 0 ? p.E : 1) >= kRemainderMinRows;
}

// A 128x128-tile NN / NT launch whose tiles (an upper bound from the host-side sizes) fill at most
// half of those slots while every tile walks at least 16 K tiles: worth a split into two phases.
static inline bool gmm_few_tiles_long_k(const GmmParams& p) {
  const int64_t row_tiles = (p.N + 127) / 128 + p.E;  // every expert may end in a partial tile
  const int64_t tiles = row_tiles * ((p.M + 127) / 128);
  return tiles * 2 <= kSplitSlots && p.K >= 1024;
}

// The launch with 128-row tiles for the rows a ROWS_MAIN launch leaves out.
template <int DT, int ODT, int MODE>
static int launch_gmm_remainder(const GmmParams& p, hipStream_t st) {
  GmmParams r = p;
  r.row_part = ROWS_AUTO_REMAINDER;
  if (p.ws == nullptr || p.ws_floats < 2 * 128 * 128)
    return launch_gmm_cfg<DT, ODT, MODE, 128, 128, EPI_NONE>(r, st, 2);
  // few tiles, each with the whole reduction: split it over the idle CUs, then add the pieces
  const int64_t slots = p.ws_floats / (128 * 128);
  r.split_slots = (int)(slots < kSplitSlots ? slots : kSplitSlots);
  r.phase = SPLIT_PARTIAL;
  const int rc = launch_gmm_cfg<DT, ODT, MODE, 128, 128, EPI_NONE>(r, st, 2);
  if (rc != GMOE_OK) return rc;
  r.phase = SPLIT_REDUCE;
  return launch_gmm_cfg<DT, ODT, MODE, 128, 128, EPI_NONE>(r, st, 2);
}

// One kernel per (type, mode, size).  Groups large enough for 256x256 tiles (TFLOP/s measured on the
// Mixtral shape):
//   NT        both operands k-contiguous: register-staged, 128-byte row pieces, plain LDS reads;
//             an expert's short last row tile goes to a second launch with 128-row tiles, which
//             with a workspace splits its reduction over the idle CUs (-7 % on the dX GEMM of fc1
//             with ragged groups); plain NN does the same when it has the workspace (-4 % on fc2);
//   NN 16-bit the same for a, the weight tile kept [k][m] in LDS and read with transposing loads
//             (6 % faster than LDS-DMA copies, whose 64-byte pieces of a load the address path
//             twice); optionally with the gated activation in the epilogue;
//   TN 16-bit both operands [k][outer]: LDS-DMA copies of 512-byte rows, 4 stages (1.5 % faster than
//             the register-staged form);
//   fp32      register-staged, 4x4 blocks transposed in registers where needed.
// Small groups: 128x128 tiles, two workgroups per CU.
template <int DT, int ODT, int MODE, int EPI>
static int launch_gmm_mode(const GmmParams& p, int dtype, int out_dtype, hipStream_t st) {
  constexpr bool half = Elem<DT>::bytes == 2;
  constexpr bool glu_fwd = EPI == EPI_GLU_FWD_SILU || EPI == EPI_GLU_FWD_GELU;
  if (gmm_large_tiles(p, MODE)) {
    if constexpr (MODE == MODE_TN && half) {
      (void)dtype;
      return launch_gmm_dtl_tn(p, dtype, out_dtype, st);
    } else if constexpr (MODE == MODE_NN && half && EPI == EPI_NONE) {
      // the short last row tiles pay off as a launch of their own only when it can be split
      if (p.ws == nullptr || p.ws_floats < 2 * 128 * 128 || !gmm_use_remainder(p))
        return launch_gmm_cfg<DT, ODT, MODE_NN, 256, 256, EPI_NONE, false, true>(p, st);
      GmmParams m = p;
      m.row_part = ROWS_AUTO_MAIN;
      m.main_grid = gmm_grid(1);
      const int rc = launch_gmm_cfg<DT, ODT, MODE_NN, 256, 256, EPI_NONE, false, true>(m, st);
      return rc != GMOE_OK ? rc : launch_gmm_remainder<DT, ODT, MODE_NN>(m, st);
    } else if constexpr (MODE == MODE_NN && half) {
      return launch_gmm_cfg<DT, ODT, MODE_NN, 256, 256, EPI, false, true>(p, st);
    } else if constexpr (MODE == MODE_NT && EPI == EPI_NONE) {
      if (!gmm_use_remainder(p)) return launch_gmm_cfg<DT, ODT, MODE_NT, 256, 256, EPI_NONE>(p, st);
      GmmParams m = p;
      m.row_part = ROWS_AUTO_MAIN;
      m.main_grid = gmm_grid(1);
      const int rc = launch_gmm_cfg<DT, ODT, MODE_NT, 256, 256, EPI_NONE>(m, st);
      return rc != GMOE_OK ? rc : launch_gmm_remainder<DT, ODT, MODE_NT>(m, st);
    } else if constexpr (!glu_fwd) {
      return launch_gmm_cfg<DT, ODT, MODE, 256, 256, EPI>(p, st);
    }
  }
  if constexpr (glu_fwd) {
    return GMOE_ERR_UNSUPPORTED;  // the caller runs the GEMM and the activation kernel instead
  } else {
    if constexpr (MODE != MODE_TN && EPI == EPI_NONE) {
      if (gmm_few_tiles_long_k(p) && p.ws != nullptr && p.ws_floats >= 2 * 128 * 128) {
        // fewer tiles than workgroup slots and a long reduction: split it (see SPLIT_PARTIAL)
        GmmParams r = p;
        const int64_t slots = p.ws_floats / (128 * 128);
        r.split_slots = (int)(slots < kSplitSlots ? slots : kSplitSlots);
        r.phase = SPLIT_PARTIAL;
        const int rc = launch_gmm_cfg<DT, ODT, MODE, 128, 128, EPI_NONE>(r, st, 2);
        if (rc != GMOE_OK) return rc;
        r.phase = SPLIT_REDUCE;
        return launch_gmm_cfg<DT, ODT, MODE, 128, 128, EPI_NONE>(r, st, 2);
      }
    }
    return launch_gmm_cfg<DT, ODT, MODE, 128, 128, EPI>(p, st, 2);
  }
}

template <int DT, int ODT>
static int launch_gmm(const GmmParams& p, int mode, int dtype, int out_dtype, int epi, hipStream_t st) {
  if (epi != EPI_NONE) {
    // fused activation epilogues keep the operand type
    if constexpr (DT == ODT) {
      if (mode == MODE_NN && Elem<DT>::bytes == 2) {
        if (epi == EPI_GLU_FWD_SILU) return launch_gmm_mode<DT, ODT, MODE_NN, EPI_GLU_FWD_SILU>(p, dtype, out_dtype, st);
        if (epi == EPI_GLU_FWD_GELU) return launch_gmm_mode<DT, ODT, MODE_NN, EPI_GLU_FWD_GELU>(p, dtype, out_dtype, st);
      }
      if (mode == MODE_NT) {
        if (epi == EPI_GLU_BWD_SILU) return launch_gmm_mode<DT, ODT, MODE_NT, EPI_GLU_BWD_SILU>(p, dtype, out_dtype, st);
        if (epi == EPI_GLU_BWD_GELU) return launch_gmm_mode<DT, ODT, MODE_NT, EPI_GLU_BWD_GELU>(p, dtype, out_dtype, st);
      }
    }
    return GMOE_ERR_UNSUPPORTED;
  }
  switch (mode) {
    case MODE_NN: return launch_gmm_mode<DT, ODT, MODE_NN, EPI_NONE>(p, dtype, out_dtype, st);
    case MODE_NT: return launch_gmm_mode<DT, ODT, MODE_NT, EPI_NONE>(p, dtype, out_dtype, st);
    default: return launch_gmm_mode<DT, ODT, MODE_TN, EPI_NONE>(p, dtype, out_dtype, st);
  }
}

static int gmm_dispatch(const GmmParams& p, int mode, int dtype, int out_dtype, int epi,
                        hipStream_t st) {
  if (dtype == GMOE_BF16 && out_dtype == GMOE_BF16) return launch_gmm<GMOE_BF16, GMOE_BF16>(p, mode, dtype, out_dtype, epi, st);
  if (dtype == GMOE_BF16 && out_dtype == GMOE_F32) return launch_gmm<GMOE_BF16, GMOE_F32>(p, mode, dtype, out_dtype, epi, st);
  if (dtype == GMOE_F16 && out_dtype == GMOE_F16) return launch_gmm<GMOE_F16, GMOE_F16>(p, mode, dtype, out_dtype, epi, st);
  if (dtype == GMOE_F16 && out_dtype == GMOE_F32) return launch_gmm<GMOE_F16, GMOE_F32>(p, mode, dtype, out_dtype, epi, st);
  if (dtype == GMOE_F32 && out_dtype == GMOE_F32) return launch_gmm<GMOE_F32, GMOE_F32>(p, mode, dtype, out_dtype, epi, st);
  return GMOE_ERR_UNSUPPORTED;
}

// Argument checks shared by the GEMM entry points; fills p.  Returns GMOE_OK to go on.
static int gmm_check(GmmParams& p, const void* a, const void* b, void* c, const int64_t* offsets,
                     int E, int64_t N, int64_t K, int64_t M, int dtype) {
  GMOE_CHECK_ARG(E >= 1 && N >= 0 && K >= 1 && M >= 1 && (offsets || E == 1));
  // with no rows at all the operands may be empty tensors: NN / NT write nothing, TN writes zeros
  GMOE_CHECK_ARG((a != nullptr && b != nullptr && c != nullptr) || N == 0);
  if (E > kMaxGroupsLds) return GMOE_ERR_UNSUPPORTED;
  if ((K % 8) != 0 || (M % 8) != 0) return GMOE_ERR_UNSUPPORTED;
  // buffer offsets are 32-bit: one expert's weight / weight gradient [K,M] and one 256-row tile of a
  // row-partitioned operand must stay below 2 GiB.  The row-partitioned operands as a whole may be
  // larger: their resources are built per tile, or per segment of an expert's rows (TN).
  const int64_t es = dtype == GMOE_F32 ? 4 : 2;
  if (K * M * es >= (1ll << 31) || 256 * (K > M ? K : M) * es >= (1ll << 31)) return GMOE_ERR_UNSUPPORTED;
  if (N >= (1ll << 40)) return GMOE_ERR_UNSUPPORTED;
  if (!gmoe_aligned(a, 16) || !gmoe_aligned(b, 16) || !gmoe_aligned(c, 16)) return GMOE_ERR_INVALID;
  p.a = static_cast<const unsigned char*>(a);
  p.b = static_cast<const unsigned char*>(b);
  p.c = static_cast<unsigned char*>(c);
  p.offsets = reinterpret_cast<const long long*>(offsets);
  p.E = E;
  p.N = N;
  p.K = K;
  p.M = M;
  p.c2 = nullptr;
  p.aux = nullptr;
  p.b_scale = nullptr;
  p.a_scale = nullptr;
  p.row_part = ROWS_ALL;
  p.F = 0;
  p.ws = nullptr;
  p.ws_floats = 0;
  p.split_slots = 0;
  p.phase = SPLIT_OFF;
  p.main_grid = 0;
  return GMOE_OK;
}

int gmm_dense(const void* a, const void* b, void* c, int64_t N, int64_t K, int64_t M, int mode,
              int dtype, int out_dtype, hipStream_t st, float* ws, int64_t ws_floats) {
  GmmParams p;
  const int rc = gmm_check(p, a, b, c, nullptr, 1, N, K, M, dtype);
  if (rc != GMOE_OK) return rc;
  if (mode != MODE_TN && N == 0) return GMOE_OK;
  if (ws != nullptr && ws_floats > 0 && gmoe_aligned(ws, 16)) {
    p.ws = ws;
    p.ws_floats = ws_floats;
  }
  return gmm_dispatch(p, mode, dtype, out_dtype, EPI_NONE, st);
}

int64_t gmm_dense_workspace_floats(int64_t N, int64_t K, int64_t M, int mode) {
  if (mode == MODE_TN || N < 1) return 0;
  GmmParams p;
  p.E = 1;
  p.N = N;
  p.K = K;
  p.M = M;
  const bool split = (gmm_large_tiles(p, mode) && gmm_use_remainder(p)) || gmm_few_tiles_long_k(p);
  return split ? (int64_t)kSplitSlots * 128 * 128 : 0;
}

int gmm_grouped_tn(const void* a, const void* b, void* c, const int64_t* offsets, int groups, int64_t N,
                   int64_t K, int64_t M, int dtype, int out_dtype, hipStream_t st) {
  GmmParams p;
  const int rc = gmm_check(p, a, b, c, offsets, groups, N, K, M, dtype);
  if (rc != GMOE_OK) return rc;
  return gmm_dispatch(p, MODE_TN, dtype, out_dtype, EPI_NONE, st);
}

}  // namespace gmoe

using namespace gmoe;

extern "C" int64_t gmoe_gmm_workspace_bytes(int E, int64_t N, int64_t K, int64_t M, int trans_a,
                                            int trans_b, int dtype) {
  if (trans_a || E < 1 || N < 0 || K < 1 || M < 1) return 0;
  GmmParams p;
  p.E = E;
  p.N = N;
  p.K = K;
  p.M = M;
  const int mode = trans_b ? MODE_NT : MODE_NN;
  const bool split = (gmm_large_tiles(p, mode) && gmm_use_remainder(p)) || gmm_few_tiles_long_k(p);
  return split ? (int64_t)kSplitSlots * 128 * 128 * 4 : 0;
}

extern "C" int gmoe_gmm(const void* a, const void* b, void* c, const int64_t* expert_offsets, int E,
                        int64_t N, int64_t K, int64_t M, int trans_a, int trans_b, int dtype,
                        int out_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  GMOE_CHECK_ARG(!(trans_a && trans_b) && expert_offsets != nullptr);
  GmmParams p;
  const int rc = gmm_check(p, a, b, c, expert_offsets, E, N, K, M, dtype);
  if (rc != GMOE_OK) return rc;
  if (!trans_a && N == 0) return GMOE_OK;  // nothing to write
  GMOE_CHECK_ARG(c != nullptr);
  if (workspace != nullptr && workspace_bytes > 0 && gmoe_aligned(workspace, 16)) {
    p.ws = static_cast<float*>(workspace);
    p.ws_floats = workspace_bytes / 4;
  }
  const int mode = trans_a ? MODE_TN : (trans_b ? MODE_NT : MODE_NN);
  return gmm_dispatch(p, mode, dtype, out_dtype, EPI_NONE, static_cast<hipStream_t>(stream));
}

extern "C" int gmoe_gmm_glu(const void* a, const void* w1, void* fc1, void* act_out,
                            const int64_t* expert_offsets, int E, int64_t N, int64_t K, int64_t F,
                            int act, int dtype, void* stream) {
  GMOE_CHECK_ARG(F >= 1 && act_out != nullptr && expert_offsets != nullptr);
  GMOE_CHECK_ARG(act == GMOE_ACT_SILU || act == GMOE_ACT_GELU);
  GmmParams p;
  const int rc = gmm_check(p, a, w1, fc1, expert_offsets, E, N, K, 2 * F, dtype);
  if (rc != GMOE_OK) return rc;
  if (!gmoe_aligned(act_out, 16)) return GMOE_ERR_INVALID;
  if (N == 0) return GMOE_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  p.c2 = static_cast<unsigned char*>(act_out);
  p.F = F;
  if (dtype != GMOE_F32 && gmm_large_tiles(p, MODE_NN) && F % 8 == 0)
    return gmm_dispatch(p, MODE_NN, dtype, dtype, act == GMOE_ACT_SILU ? EPI_GLU_FWD_SILU : EPI_GLU_FWD_GELU, st);
  // small groups / fp32: the GEMM followed by the activation kernel
  const int rc2 = gmm_dispatch(p, MODE_NN, dtype, dtype, EPI_NONE, st);
  if (rc2 != GMOE_OK) return rc2;
  return gmoe_glu_fwd(fc1, dtype, N, F, act, act_out, stream);
}

extern "C" int gmoe_gmm_glu_bwd(const void* grad_out, const void* w2, const void* fc1,
                                void* grad_fc1, const int64_t* expert_offsets, int E, int64_t N,
                                int64_t K, int64_t F, int act, int dtype, void* stream) {
  GMOE_CHECK_ARG(fc1 != nullptr && expert_offsets != nullptr);
  GMOE_CHECK_ARG(act == GMOE_ACT_SILU || act == GMOE_ACT_GELU);
  GmmParams p;
  const int rc = gmm_check(p, grad_out, w2, grad_fc1, expert_offsets, E, N, K, F, dtype);
  if (rc != GMOE_OK) return rc;
  if (!gmoe_aligned(fc1, 16)) return GMOE_ERR_INVALID;
  if (N == 0) return GMOE_OK;
  p.aux = static_cast<const unsigned char*>(fc1);
  p.F = F;
  return gmm_dispatch(p, MODE_NT, dtype, dtype, act == GMOE_ACT_SILU ? EPI_GLU_BWD_SILU : EPI_GLU_BWD_GELU,
                      static_cast<hipStream_t>(stream));
}

extern "C" int gmoe_gmm_fp8w(const void* a, const void* b_q, const void* b_scale, void* c,
                             const int64_t* expert_offsets, int E, int64_t N, int64_t K, int64_t M,
                             int trans_b, void* stream) {
  GMOE_CHECK_ARG(b_scale != nullptr && expert_offsets != nullptr);
  GmmParams p;
  const int rc = gmm_check(p, a, b_q, c, expert_offsets, E, N, K, M, GMOE_BF16);
  if (rc != GMOE_OK) return rc;
  if ((K % 16) != 0 || (M % 16) != 0) return GMOE_ERR_UNSUPPORTED;  // 16-byte pieces of fp8
  if (N == 0) return GMOE_OK;
  p.b_scale = static_cast<const unsigned char*>(b_scale);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // few rows per expert: the weight-streaming kernel, which reads an expert's weights once
  if (gmm_fp8_skinny_applies(p)) return launch_gmm_fp8_skinny(p, trans_b != 0, st);
  // 128x128 tiles: two workgroups fit a CU (LDS and registers), which hides the latency of the
  // weight stream when an expert has only a row tile or two
  if (trans_b)
    return launch_gmm_cfg<GMOE_BF16, GMOE_BF16, MODE_NT, 128, 128, EPI_NONE, true>(p, st, 2);
  return launch_gmm_cfg<GMOE_BF16, GMOE_BF16, MODE_NN, 128, 128, EPI_NONE, true>(p, st, 2);
}

extern "C" int gmoe_gmm_fp8a(const void* a_q, const int32_t* a_scale, const void* b_q,
                             const void* b_scale, void* c, const int64_t* expert_offsets, int E,
                             int64_t N, int64_t K, int64_t M, int trans_b, void* stream) {
  GMOE_CHECK_ARG(a_scale != nullptr && b_scale != nullptr && expert_offsets != nullptr);
  GmmParams p;
  const int rc = gmm_check(p, a_q, b_q, c, expert_offsets, E, N, K, M, GMOE_BF16);
  if (rc != GMOE_OK) return rc;
  if ((K % 16) != 0 || (M % 16) != 0) return GMOE_ERR_UNSUPPORTED;
  if (N == 0) return GMOE_OK;
  p.b_scale = static_cast<const unsigned char*>(b_scale);
  p.a_scale = reinterpret_cast<const unsigned char*>(a_scale);
  // one kernel form, built for few rows per expert; more rows are cut into chunks of up to 192,
  // each of which streams the expert's weights again
  if (!gmm_fp8_skinny_applies(p, true)) return GMOE_ERR_UNSUPPORTED;
  return launch_gmm_fp8_skinny(p, trans_b != 0, static_cast<hipStream_t>(stream));
}
