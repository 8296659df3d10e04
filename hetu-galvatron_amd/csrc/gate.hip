// The router's gate projection for gfx950: logits = x @ W^T with x [T,H], W [E,H] (Router.gating,
// moe/router.py:49-68: F.linear(input, weight)) and its two gradients.  With E of 8 or 16 the
// products are a tall-skinny GEMM (forward, weight gradient) and a rank-E update (input gradient):
// all three are bound by one pass over a [T,H] tensor in HBM and have the kernels below.  Larger
// expert counts (64, 256) are ordinary dense products and run on the grouped-GEMM kernels as one
// group; an fp32 gradient of the logits against 16-bit operands is split into two 16-bit terms
// (value = hi + lo to 2^-17), so the products stay exact and the sums fp32 as with fp32 operands.
//
//  * forward: matrix cores.  A workgroup owns 32 token rows; lane (r, g) of a wavefront supplies 16
//    bytes of row r, the MFMA pairs them with the same 16 bytes of the weight row of expert
//    lane % 32 (zero beyond E; the weight stays in L1/L2).  The four wavefronts of a workgroup split
//    the reduction over H and meet in LDS.  The order of the reduction elements inside an MFMA
//    is free as long as both operands agree, so no transposition is needed; x is read in whole
//    cache lines and turned into the lane-per-row operand layout through LDS (loading it in that
//    layout directly uses 32 bytes of a line per instruction and cost 15-20 % more time).
//  * input gradient dx = dlogits @ W: vector ALUs; a lane owns the same column vectors of every
//    row with its slice of W in registers (E FMAs per element), coalesced 16-byte stores.  The
//    columns are cut into slabs of 256 * NV vectors (blockIdx.y) so the registers do not grow with H.
//  * weight gradient dW = dlogits^T @ x: the same ownership with the accumulators in registers; one
//    fp32 partial [E,H] per workgroup, summed in a fixed order by sum_partial_rows.
#include <type_traits>

#include "gmm_common.h"

namespace gmoe {

constexpr int kGateThreads = 256;
constexpr int kGateWaves = kGateThreads / GMOE_WAVE;
constexpr int kGateMaxE = 16;      // vector-ALU backward kernels keep E x columns in registers
constexpr int kGateFwdMaxE = 64;   // the forward kernel pairs an x fragment with 1 or 2 blocks of 32 experts
constexpr int kGateDwRows = 8;     // rows per step of the dW kernel
constexpr int kGateDwWorkgroups = 512;  // dW kernel: partial weight gradients x column slabs, two per CU

// ---- forward ------------------------------------------------------------------------------------
// A workgroup owns 32 token rows, its four wavefronts a quarter of H each.  A wavefront walks its
// quarter in stages of 256 bytes per row: eight coalesced loads (a load covers 4 rows x 256 bytes,
// whole cache lines), kept two stages ahead in registers, go to the wavefront's own 8 KiB of LDS and
// come back as MFMA operands, lane (r, g) reading 16 bytes of row r.  Piece p of row r sits in slot
// p ^ (r & 15) of the row, so the 16 lanes one LDS pass serves hit 16 different bank groups on both
// sides.  Only this wavefront touches the region and its LDS operations execute in order, so no
// barrier is needed inside the loop.  The weight pieces come straight from L1/L2.
constexpr int kGateStagePieces = 16;  // 16-byte pieces per row and stage
constexpr int kGateStageLoads = 32 * kGateStagePieces / GMOE_WAVE;  // loads per lane and stage

// NE: blocks of 32 experts (1 or 2): every x fragment meets NE weight fragments.
template <int DT, int ODT, int NE>
__global__ __launch_bounds__(kGateThreads) void gate_fwd_kernel(
    const unsigned char* __restrict__ x, const unsigned char* __restrict__ w, int64_t T, int H, int E,
    unsigned char* __restrict__ logits) {
  constexpr int EPV = Vec16<DT>::n;  // elements per 16-byte piece
  constexpr int SP = kGateStagePieces, NL = kGateStageLoads, NU = SP / 2;
  __shared__ u32x4 stage[kGateWaves][32 * SP];
  __shared__ float red[kGateWaves][16 * NE][GMOE_WAVE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int64_t row_bytes = (int64_t)H * Elem<DT>::bytes;
  // this wavefront's share of the reduction, in pieces: whole stages per wavefront, so that every
  // stage of an aligned row starts on a cache line
  const int pieces = H / EPV;
  const int per_wave = ((pieces + kGateWaves - 1) / kGateWaves + SP - 1) / SP * SP;
  const int p_begin = wave * per_wave < pieces ? wave * per_wave : pieces;
  const int p_end = p_begin + per_wave < pieces ? p_begin + per_wave : pieces;
  const unsigned char* wrow[NE];
  bool has_w[NE];
#pragma unroll
  for (int nb = 0; nb < NE; ++nb) {
    has_w[nb] = 32 * nb + r < E;
    wrow[nb] = w + (int64_t)(has_w[nb] ? 32 * nb + r : 0) * row_bytes;
  }
  u32x4* mine = stage[wave];
  // loader side: load i of a stage covers rows 4 i + lane / 16, piece lane % 16 of the stage
  const int lrow = lane >> 4, lpiece = lane & 15;

  const int64_t blocks = (T + 31) / 32;
  for (int64_t blk = blockIdx.x; blk < blocks; blk += gridDim.x) {
    const int64_t row = blk * 32 + r;
    const bool has_x = row < T;
    f32x16 acc[NE];
#pragma unroll
    for (int nb = 0; nb < NE; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nb][i] = 0.f;
    u32x4 xs[2][NL];
    auto request = [&](auto buf_c, int p0) {
      constexpr int BUF = decltype(buf_c)::value;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int64_t lr = blk * 32 + 4 * i + lrow;
        const int p = p0 + lpiece;
        xs[BUF][i] = u32x4{0u, 0u, 0u, 0u};
        if (lr < T && p < p_end) xs[BUF][i] = ld16_nt(x + lr * row_bytes + (int64_t)p * 16);
      }
    };
    auto consume = [&](auto buf_c, int p0) {
      constexpr int BUF = decltype(buf_c)::value;
      u32x4 wv[NE][NU], xv[NU];
#pragma unroll
      for (int nb = 0; nb < NE; ++nb)
#pragma unroll
        for (int u = 0; u < NU; ++u) {
          const int p = p0 + 2 * u + g;
          wv[nb][u] = u32x4{0u, 0u, 0u, 0u};
          if (has_w[nb] && p < p_end) wv[nb][u] = ld16(wrow[nb] + (int64_t)p * 16);
        }
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int sr = 4 * i + lrow;
        mine[sr * SP + (lpiece ^ (sr & 15))] = xs[BUF][i];
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int u = 0; u < NU; ++u) xv[u] = mine[r * SP + ((2 * u + g) ^ (r & 15))];
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int u = 0; u < NU; ++u)
#pragma unroll
        for (int nb = 0; nb < NE; ++nb) Mma<DT>::run(xv[u], wv[nb][u], acc[nb]);
    };
    request(std::integral_constant<int, 0>{}, p_begin);
    for (int p0 = p_begin; p0 < p_end; p0 += 2 * SP) {
      request(std::integral_constant<int, 1>{}, p0 + SP);
      consume(std::integral_constant<int, 0>{}, p0);
      if (p0 + SP < p_end) {
        request(std::integral_constant<int, 0>{}, p0 + 2 * SP);
        consume(std::integral_constant<int, 1>{}, p0 + SP);
      }
    }
    // lane (r, g) now holds, for token row blk*32 + r, experts 32 nb + 8 i + 4 g + v in acc[nb][4 i + v]
#pragma unroll
    for (int nb = 0; nb < NE; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) red[wave][16 * nb + i][lane] = acc[nb][i];
    __syncthreads();
    if (wave == 0 && has_x) {
#pragma unroll
      for (int nb = 0; nb < NE; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e0 = 32 * nb + 8 * i + 4 * g;
          if (e0 >= E) continue;
          float s[4];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            float t = red[0][16 * nb + 4 * i + v][lane];
#pragma unroll
            for (int q = 1; q < kGateWaves; ++q) t += red[q][16 * nb + 4 * i + v][lane];
            s[v] = t;
          }
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (e0 + v < E) Elem<ODT>::store(logits, row * E + e0 + v, s[v]);
        }
    }
    __syncthreads();
  }
}

// One row of dlogits as fp32, zero beyond E.  The address is the same in every lane; 16-bit rows of
// an even E are read as dwords so that the loads can be scalar ones.
template <int LDT, int EMAX>
__device__ __forceinline__ void load_dl_row(const unsigned char* __restrict__ dlogits, int64_t row,
                                            int E, bool valid, float (&out)[EMAX]) {
  if (LDT != GMOE_F32 && (E & 1) == 0) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(dlogits) + row * (E / 2);
#pragma unroll
    for (int h = 0; h < EMAX / 2; ++h) {
      const uint32_t v = (valid && 2 * h < E) ? p[h] : 0u;
      if (LDT == GMOE_BF16) {
        out[2 * h] = __uint_as_float(v << 16);
        out[2 * h + 1] = __uint_as_float(v & 0xffff0000u);
      } else {
        out[2 * h] = f16_bits_to_f32(v & 0xffffu);
        out[2 * h + 1] = f16_bits_to_f32(v >> 16);
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < EMAX; ++e)
      out[e] = (valid && e < E) ? Elem<LDT>::load(dlogits, row * E + e) : 0.f;
  }
}

// R consecutive rows of dlogits as fp32.  Rows are contiguous, so a full group of a full-width
// table (E == EMAX, all R rows inside T) is one run of R * EMAX elements at a fixed stride: its loads
// carry no conditions and merge into a few wide scalar loads.  Other groups go row by row.
template <int LDT, int EMAX, int R>
__device__ __forceinline__ void load_dl_block(const unsigned char* __restrict__ dlogits, int64_t row0,
                                              int64_t T, int E, float (&out)[R][EMAX]) {
  if (E == EMAX && row0 + R <= T) {
    if (LDT == GMOE_F32) {
      const float* p = reinterpret_cast<const float*>(dlogits) + row0 * EMAX;
#pragma unroll
      for (int i = 0; i < R * EMAX; ++i) out[i / EMAX][i % EMAX] = p[i];
    } else {
      const uint32_t* p = reinterpret_cast<const uint32_t*>(dlogits) + row0 * (EMAX / 2);
#pragma unroll
      for (int h = 0; h < R * EMAX / 2; ++h) {
        const uint32_t v = p[h];
        float lo, hi;
        if (LDT == GMOE_BF16) {
          lo = __uint_as_float(v << 16);
          hi = __uint_as_float(v & 0xffff0000u);
        } else {
          lo = f16_bits_to_f32(v & 0xffffu);
          hi = f16_bits_to_f32(v >> 16);
        }
        out[(2 * h) / EMAX][(2 * h) % EMAX] = lo;
        out[(2 * h + 1) / EMAX][(2 * h + 1) % EMAX] = hi;
      }
    }
    return;
  }
#pragma unroll
  for (int rr = 0; rr < R; ++rr) load_dl_row<LDT, EMAX>(dlogits, row0 + rr, E, row0 + rr < T, out[rr]);
}

// R consecutive 16-bit dlogits rows as dwords (two experts each), zero beyond E and beyond T; the
// same fast and slow paths as load_dl_block.
template <int EMAX, int R>
__device__ __forceinline__ void load_dl_dwords(const unsigned char* __restrict__ dlogits, int64_t row0,
                                               int64_t T, int E, uint32_t (&out)[R][EMAX / 2]) {
  if (E == EMAX && row0 + R <= T) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(dlogits) + row0 * (EMAX / 2);
#pragma unroll
    for (int i = 0; i < R * EMAX / 2; ++i) out[i / (EMAX / 2)][i % (EMAX / 2)] = p[i];
    return;
  }
#pragma unroll
  for (int rr = 0; rr < R; ++rr) {
    const int64_t row = row0 + rr;
    const bool valid = row < T;
    if ((E & 1) == 0) {
      const uint32_t* p = reinterpret_cast<const uint32_t*>(dlogits) + row * (E / 2);
#pragma unroll
      for (int h = 0; h < EMAX / 2; ++h) out[rr][h] = (valid && 2 * h < E) ? p[h] : 0u;
    } else {
      const uint16_t* p = reinterpret_cast<const uint16_t*>(dlogits) + row * E;
#pragma unroll
      for (int h = 0; h < EMAX / 2; ++h) {
        const uint32_t lo = (valid && 2 * h < E) ? p[2 * h] : 0u;
        const uint32_t hi = (valid && 2 * h + 1 < E) ? p[2 * h + 1] : 0u;
        out[rr][h] = lo | (hi << 16);
      }
    }
  }
}
// acc + a.lo * b.lo + a.hi * b.hi on two packed 16-bit pairs (products exact in fp32)
template <int DT>
__device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float acc) {
  if (DT == GMOE_BF16)
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc, false);
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), acc, false);
}

// ---- input gradient -----------------------------------------------------------------------------
// dx[t, cols] = sum_e dlogits[t,e] * W[e, cols]
template <int DT, int LDT, int NV, int EMAX>
__global__ __launch_bounds__(kGateThreads) void gate_bwd_input_kernel(
    const unsigned char* __restrict__ dlogits, const unsigned char* __restrict__ w, int64_t T, int H,
    int E, unsigned char* __restrict__ dx) {
  constexpr int EPV = Vec16<DT>::n;
  constexpr int R = 4;
  const int tid = blockIdx.y * (kGateThreads * NV) + threadIdx.x;  // first column vector of this lane
  const int nvec = H / EPV;
  const int64_t row_bytes = (int64_t)H * Elem<DT>::bytes;
  float wf[EMAX][NV][EPV];
#pragma unroll
  for (int e = 0; e < EMAX; ++e)
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int c = tid + kGateThreads * j;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (e < E && c < nvec) v = ld16(w + e * row_bytes + (int64_t)c * 16);
      Vec16<DT>::unpack(v, wf[e][j]);
    }
  const int64_t groups = (T + R - 1) / R;
  for (int64_t gidx = blockIdx.x; gidx < groups; gidx += gridDim.x) {
    float dl[R][EMAX];
    load_dl_block<LDT, EMAX, R>(dlogits, gidx * R, T, E, dl);
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
      const int64_t row = gidx * R + rr;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = tid + kGateThreads * j;
        if (row >= T || c >= nvec) continue;
        float o[EPV];
#pragma unroll
        for (int q = 0; q < EPV; ++q) o[q] = 0.f;
#pragma unroll
        for (int e = 0; e < EMAX; ++e)
#pragma unroll
          for (int q = 0; q < EPV; ++q) o[q] = fmaf(dl[rr][e], wf[e][j][q], o[q]);
        st16(dx + row * row_bytes + (int64_t)c * 16, Vec16<DT>::pack(o));
      }
    }
  }
}

// ---- weight gradient ----------------------------------------------------------------------------
// partial[blockIdx.x][e][cols] = sum over this workgroup's rows of dlogits[t,e] * x[t, cols]
template <int DT, int LDT, int NV, int EMAX>
__global__ __launch_bounds__(kGateThreads) void gate_bwd_weight_kernel(
    const unsigned char* __restrict__ dlogits, const unsigned char* __restrict__ x, int64_t T, int H,
    int E, float* __restrict__ partial) {
  constexpr int EPV = Vec16<DT>::n;
  constexpr int R = EMAX <= 8 ? kGateDwRows : kGateDwRows / 2;
  const int tid = blockIdx.y * (kGateThreads * NV) + threadIdx.x;
  const int nvec = H / EPV;
  const int64_t row_bytes = (int64_t)H * Elem<DT>::bytes;
  float acc[EMAX][NV][EPV];
#pragma unroll
  for (int e = 0; e < EMAX; ++e)
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int q = 0; q < EPV; ++q) acc[e][j][q] = 0.f;

  // Row groups are double-buffered: the x rows of the next group are requested before the current
  // group's E x 8 multiply-adds per element run, so the arithmetic (a third of the kernel's time
  // at 8 experts) hides under the loads instead of alternating with them.
  const int64_t groups = (T + R - 1) / R;
  u32x4 xv[2][R][NV];
  auto request = [&](auto buf_c, int64_t gidx) {
    constexpr int BUF = decltype(buf_c)::value;
#pragma unroll
    for (int rr = 0; rr < R; ++rr)
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int64_t row = gidx * R + rr;
        const int c = tid + kGateThreads * j;
        xv[BUF][rr][j] = u32x4{0u, 0u, 0u, 0u};
        if (gidx < groups && row < T && c < nvec)
          xv[BUF][rr][j] = ld16_nt(x + row * row_bytes + (int64_t)c * 16);
      }
  };
  // 16-bit x and dlogits of one type: rows go in pairs through the two-element dot product, one
  // instruction per expert and column for two rows (the kernel is bound by vector-ALU issue: 64
  // dot products and 8 byte permutes per row pair and 8 columns instead of 128 multiply-adds and
  // 16 conversions).  The pairs (row t, row t+1) of a column are cut out of the two rows' dwords.
  constexpr bool DOT2 = DT != GMOE_F32 && LDT == DT;
  auto consume = [&](auto buf_c, int64_t gidx) {
    constexpr int BUF = decltype(buf_c)::value;
    if constexpr (DOT2) {
      uint32_t raw[R][EMAX / 2];
      load_dl_dwords<EMAX, R>(dlogits, gidx * R, T, E, raw);
#pragma unroll
      for (int rr = 0; rr < R; rr += 2) {
        uint32_t pe[EMAX];  // (dlogits[t][e], dlogits[t+1][e])
#pragma unroll
        for (int h = 0; h < EMAX / 2; ++h) {
          pe[2 * h] = (raw[rr][h] & 0xffffu) | (raw[rr + 1][h] << 16);
          pe[2 * h + 1] = (raw[rr][h] >> 16) | (raw[rr + 1][h] & 0xffff0000u);
        }
#pragma unroll
        for (int j = 0; j < NV; ++j)
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const uint32_t a = xv[BUF][rr][j][d], b = xv[BUF][rr + 1][j][d];
            const uint32_t lo = __builtin_amdgcn_perm(b, a, 0x05040100u);  // (a.lo, b.lo)
            const uint32_t hi = __builtin_amdgcn_perm(b, a, 0x07060302u);  // (a.hi, b.hi)
#pragma unroll
            for (int e = 0; e < EMAX; ++e) {
              acc[e][j][2 * d] = dot2_acc<DT>(pe[e], lo, acc[e][j][2 * d]);
              acc[e][j][2 * d + 1] = dot2_acc<DT>(pe[e], hi, acc[e][j][2 * d + 1]);
            }
          }
      }
      return;
    }
    float dl[R][EMAX];
    load_dl_block<LDT, EMAX, R>(dlogits, gidx * R, T, E, dl);
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        float xf[EPV];
        Vec16<DT>::unpack(xv[BUF][rr][j], xf);
#pragma unroll
        for (int e = 0; e < EMAX; ++e)
#pragma unroll
          for (int q = 0; q < EPV; ++q) acc[e][j][q] = fmaf(dl[rr][e], xf[q], acc[e][j][q]);
      }
    }
  };
  const int64_t gstep = gridDim.x;
  request(std::integral_constant<int, 0>{}, (int64_t)blockIdx.x);
  for (int64_t gidx = blockIdx.x; gidx < groups; gidx += 2 * gstep) {
    request(std::integral_constant<int, 1>{}, gidx + gstep);
    consume(std::integral_constant<int, 0>{}, gidx);
    if (gidx + gstep < groups) {
      request(std::integral_constant<int, 0>{}, gidx + 2 * gstep);
      consume(std::integral_constant<int, 1>{}, gidx + gstep);
    }
  }
  float* mine = partial + (int64_t)blockIdx.x * E * H;
#pragma unroll
  for (int e = 0; e < EMAX; ++e) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int c = tid + kGateThreads * j;
      if (e >= E || c >= nvec) continue;
#pragma unroll
      for (int q = 0; q < EPV; q += 4) {
        const f32x4 v = {acc[e][j][q], acc[e][j][q + 1], acc[e][j][q + 2], acc[e][j][q + 3]};
        *reinterpret_cast<f32x4*>(mine + (int64_t)e * H + (int64_t)c * EPV + q) = v;
      }
    }
  }
}

// ---- large expert counts: helpers around the dense products ---------------------------------------
// out [T, 2E] in DT: out[t, e] = round(dl[t,e]), out[t, E + e] = round(dl[t,e] - out[t,e])
template <int DT>
__global__ __launch_bounds__(256) void gate_split_kernel(const float* __restrict__ dl, int64_t n,
                                                          int E, void* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int64_t t = i / E;
  const int e = (int)(i - t * E);
  const float v = dl[i];
  const float hi = Elem<DT>::round(v);
  Elem<DT>::store(out, t * 2 * E + e, hi);
  Elem<DT>::store(out, t * 2 * E + E + e, v - hi);
}
// dup [2E, H] = [W; W] in 16-byte pieces
__global__ __launch_bounds__(256) void gate_dup_kernel(const u32x4* __restrict__ w, int64_t pieces,
                                                        u32x4* __restrict__ dup) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= pieces) return;
  const u32x4 v = w[i];
  dup[i] = v;
  dup[pieces + i] = v;
}
static void gate_split(const void* dl, int64_t T, int E, int dtype, void* out, hipStream_t st) {
  const int64_t n = T * E;
  if (n == 0) return;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (dtype == GMOE_BF16)
    hipLaunchKernelGGL((gate_split_kernel<GMOE_BF16>), grid, dim3(256), 0, st, static_cast<const float*>(dl), n, E, out);
  else
    hipLaunchKernelGGL((gate_split_kernel<GMOE_F16>), grid, dim3(256), 0, st, static_cast<const float*>(dl), n, E, out);
}
static inline int64_t round_up_256(int64_t v) { return (v + 255) / 256 * 256; }

// ---- host side ----------------------------------------------------------------------------------
// Column vectors per lane of the backward kernels: E * NV * 8 values of W (or of dW) in registers.
static int gate_nv(int) { return 1; }
static unsigned gate_slabs(int64_t H, int E, int dtype) {
  const int64_t nvec = H / (dtype == GMOE_F32 ? 4 : 8);
  const int64_t per = (int64_t)kGateThreads * gate_nv(E);
  return (unsigned)((nvec + per - 1) / per);
}

static int gate_status(int64_t T, int64_t H, int E, int dtype, int ldtype, bool backward) {
  if (dtype != GMOE_F32 && dtype != GMOE_BF16 && dtype != GMOE_F16) return GMOE_ERR_UNSUPPORTED;
  if (ldtype != dtype && ldtype != GMOE_F32) return GMOE_ERR_UNSUPPORTED;
  if (T < 0 || H < 1 || E < 1) return GMOE_ERR_INVALID;
  if (H % (dtype == GMOE_F32 ? 4 : 8) != 0) return GMOE_ERR_INVALID;
  // beyond the dedicated kernels the products run on the grouped-GEMM kernels: 16-byte rows
  if (E > (backward ? kGateMaxE : kGateFwdMaxE) && (E % 8 != 0 || H % 8 != 0)) return GMOE_ERR_UNSUPPORTED;
  if (H > (1 << 20) || E > 4096) return GMOE_ERR_UNSUPPORTED;
  return GMOE_OK;
}

// Partial weight gradients (= workgroups along T) of the dW kernel: with the column slabs they make
// about two workgroups per CU; more of them only add partial sums to write and read back.
static int gate_parts(int64_t T, int64_t H, int E, int dtype) {
  const int64_t groups = (T + kGateDwRows - 1) / kGateDwRows;
  int64_t parts = kGateDwWorkgroups / (int64_t)gate_slabs(H, E, dtype);
  if (parts < 32) parts = 32;
  return (int)(groups < parts ? groups : parts);
}

// Calls f(DT, LDT) with the storage type and the logits type as integral constants.
template <typename F>
static void gate_by_types(int dtype, int ldtype, F&& f) {
  auto inner = [&](auto dt) {
    constexpr int DT = decltype(dt)::value;
    if (ldtype == GMOE_F32) f(dt, std::integral_constant<int, GMOE_F32>{});
    else f(dt, std::integral_constant<int, DT>{});
  };
  if (dtype == GMOE_F32) inner(std::integral_constant<int, GMOE_F32>{});
  else if (dtype == GMOE_BF16) inner(std::integral_constant<int, GMOE_BF16>{});
  else inner(std::integral_constant<int, GMOE_F16>{});
}

template <typename F>
static void gate_by_e(int E, F&& f) {
  if (E <= 8) f(std::integral_constant<int, 1>{}, std::integral_constant<int, 8>{});
  else f(std::integral_constant<int, 1>{}, std::integral_constant<int, 16>{});
}

}  // namespace gmoe

extern "C" int64_t gmoe_gate_fwd_workspace_bytes(int64_t T, int64_t H, int E, int dtype) {
  using namespace gmoe;
  if (gate_status(T, H, E, dtype, dtype, false) != GMOE_OK) return -1;
  if (E <= kGateFwdMaxE) return 0;
  return gmm_dense_workspace_floats(T, H, E, MODE_NT) * 4;
}

extern "C" int gmoe_gate_fwd(const void* x, const void* weight, int64_t T, int64_t H, int E, int dtype,
                             void* logits, int logits_dtype, void* workspace, int64_t workspace_bytes,
                             void* stream) {
  using namespace gmoe;
  const int stt = gate_status(T, H, E, dtype, logits_dtype, false);
  if (stt != GMOE_OK) return stt;
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(x && weight && logits);
  GMOE_CHECK_ARG(gmoe_aligned(x, 16) && gmoe_aligned(weight, 16));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (E > kGateFwdMaxE) {
    // [T,E] is a few tiles wide and H deep: with the workspace the reduction spreads over the CUs
    GMOE_CHECK_ARG(workspace_bytes >= 0 && (workspace == nullptr || gmoe_aligned(workspace, 16)));
    return gmm_dense(x, weight, logits, T, H, E, MODE_NT, dtype, logits_dtype, st,
                     static_cast<float*>(workspace), workspace ? workspace_bytes / 4 : 0);
  }
  const int64_t blocks = (T + 31) / 32;
  const unsigned grid = (unsigned)(blocks < 2048 ? blocks : 2048);
  gate_by_types(dtype, logits_dtype, [&](auto dt, auto ldt) {
    constexpr int DT = decltype(dt)::value, LDT = decltype(ldt)::value;
    auto launch = [&](auto ne) {
      hipLaunchKernelGGL((gate_fwd_kernel<DT, LDT, decltype(ne)::value>), dim3(grid), dim3(kGateThreads),
                         0, st, static_cast<const unsigned char*>(x),
                         static_cast<const unsigned char*>(weight), T, (int)H, E,
                         static_cast<unsigned char*>(logits));
    };
    if (E <= 32) launch(std::integral_constant<int, 1>{});
    else launch(std::integral_constant<int, 2>{});
  });
  return gmoe_launch_status();
}

extern "C" int64_t gmoe_gate_bwd_input_workspace_bytes(int64_t T, int64_t H, int E, int dtype,
                                                       int logits_dtype) {
  using namespace gmoe;
  if (gate_status(T, H, E, dtype, logits_dtype, true) != GMOE_OK) return -1;
  if (E <= kGateMaxE || logits_dtype == dtype) return 0;
  return round_up_256(T * 2 * E * 2) + round_up_256((int64_t)2 * E * H * 2);
}

extern "C" int gmoe_gate_bwd_input(const void* dlogits, int logits_dtype, const void* weight, int64_t T,
                                   int64_t H, int E, int dtype, void* dx, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
  using namespace gmoe;
  const int stt = gate_status(T, H, E, dtype, logits_dtype, true);
  if (stt != GMOE_OK) return stt;
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(dlogits && weight && dx);
  GMOE_CHECK_ARG(gmoe_aligned(dlogits, 4));  // its rows are read as dwords
  GMOE_CHECK_ARG(gmoe_aligned(weight, 16) && gmoe_aligned(dx, 16));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (E > kGateMaxE) {
    GMOE_CHECK_ARG(gmoe_aligned(dlogits, 16));
    if (logits_dtype == dtype)
      return gmm_dense(dlogits, weight, dx, T, E, H, MODE_NN, dtype, dtype, st);
    // fp32 gradient, 16-bit weight: dx = [hi | lo] @ [W; W]
    const int64_t need = gmoe_gate_bwd_input_workspace_bytes(T, H, E, dtype, logits_dtype);
    GMOE_CHECK_ARG(workspace != nullptr && gmoe_aligned(workspace, 16) && workspace_bytes >= need);
    unsigned char* split = static_cast<unsigned char*>(workspace);
    unsigned char* dup = split + round_up_256(T * 2 * E * 2);
    gate_split(dlogits, T, E, dtype, split, st);
    const int64_t pieces = (int64_t)E * H * 2 / 16;
    hipLaunchKernelGGL(gate_dup_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st,
                       static_cast<const u32x4*>(weight), pieces, reinterpret_cast<u32x4*>(dup));
    return gmm_dense(split, dup, dx, T, 2 * E, H, MODE_NN, dtype, dtype, st);
  }
  const int64_t groups = (T + 3) / 4;
  const unsigned grid = (unsigned)(groups < 2048 ? groups : 2048);
  gate_by_types(dtype, logits_dtype, [&](auto dt, auto ldt) {
    constexpr int DT = decltype(dt)::value, LDT = decltype(ldt)::value;
    gate_by_e(E, [&](auto n, auto em) {
      hipLaunchKernelGGL((gate_bwd_input_kernel<DT, LDT, decltype(n)::value, decltype(em)::value>),
                         dim3(grid, gate_slabs(H, E, dtype)), dim3(kGateThreads), 0, st,
                         static_cast<const unsigned char*>(dlogits),
                         static_cast<const unsigned char*>(weight), T, (int)H, E,
                         static_cast<unsigned char*>(dx));
    });
  });
  return gmoe_launch_status();
}

// Large expert counts: dW = dlogits^T @ x has few output tiles ([E,H]) and a reduction over all T
// rows.  The rows are cut into `parts` ranges that run as the groups of one grouped TN product, each
// writing an fp32 partial [cols,H]; sum_partial_rows adds them in order.  cols = E, or 2E when an
// fp32 gradient enters as two 16-bit terms.
struct GateDwPlan {
  int cols;            // columns of the 16-bit gradient operand
  int parts;           // row ranges = groups of the TN product
  int64_t part_rows;   // rows per range (a multiple of 64)
  int64_t sum_rows;    // workspace rows ([E*H] fp32 each) of the partial sums
  int64_t table_rows;  // ... of the offset table
  int64_t split_rows;  // ... of the split gradient [T,2E]
};
static GateDwPlan gate_dw_plan(int64_t T, int64_t H, int E, bool split) {
  GateDwPlan g;
  g.cols = split ? 2 * E : E;
  const bool large = g.cols >= 512 && H >= 256;  // the tile size the TN product will choose
  const int64_t tile = large ? 256 : 128;
  const int64_t tiles = ((g.cols + tile - 1) / tile) * ((H + tile - 1) / tile);
  int64_t parts = ((large ? 256 : 512) + tiles - 1) / tiles;
  const int64_t most = T / 256 > 1 ? T / 256 : 1;  // at least 256 rows per range
  if (parts > most) parts = most;
  if (parts > 64) parts = 64;
  g.part_rows = ((T + parts - 1) / parts + 63) / 64 * 64;
  if (g.part_rows < 64) g.part_rows = 64;
  g.parts = (int)((T + g.part_rows - 1) / g.part_rows);
  if (g.parts < 1) g.parts = 1;
  const int64_t row = (int64_t)E * H * 4;
  g.sum_rows = (int64_t)g.parts * (g.cols / E);
  g.table_rows = ((int64_t)(g.parts + 1) * 8 + row - 1) / row;
  g.split_rows = split ? (T * 2 * E * 2 + row - 1) / row : 0;
  return g;
}
__global__ void gate_part_offsets_kernel(long long* off, int parts, long long part_rows, long long T) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i > parts) return;
  const long long v = (long long)i * part_rows;
  off[i] = v < T ? v : T;
}

extern "C" int64_t gmoe_gate_bwd_workspace_rows(int64_t T, int64_t H, int E, int dtype) {
  using namespace gmoe;
  if (gate_status(T, H, E, dtype, dtype, true) != GMOE_OK) return -1;
  if (E > kGateMaxE) {
    // sized for an fp32 gradient against 16-bit operands (the caller's logits type is not known
    // here): partial sums of both terms, the offset table, the gradient split into the two terms
    const GateDwPlan g = gate_dw_plan(T, H, E, dtype != GMOE_F32);
    return g.sum_rows + g.table_rows + g.split_rows;
  }
  return gate_parts(T, H, E, dtype);
}

extern "C" int gmoe_gate_bwd_weight(const void* dlogits, int logits_dtype, const void* x, int64_t T,
                                    int64_t H, int E, int dtype, void* dweight, float* workspace,
                                    int64_t workspace_rows, void* stream) {
  using namespace gmoe;
  const int stt = gate_status(T, H, E, dtype, logits_dtype, true);
  if (stt != GMOE_OK) return stt;
  GMOE_CHECK_ARG(dweight != nullptr);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (E > kGateMaxE) {
    GMOE_CHECK_ARG(T == 0 || (dlogits && x && gmoe_aligned(dlogits, 16) && gmoe_aligned(x, 16)));
    GMOE_CHECK_ARG(gmoe_aligned(dweight, 16));
    if (T == 0) return gmm_dense(dlogits, x, dweight, T, E, H, MODE_TN, dtype, dtype, st);  // zeros
    const bool split = logits_dtype != dtype;
    const GateDwPlan g = gate_dw_plan(T, H, E, split);
    GMOE_CHECK_ARG(workspace != nullptr && gmoe_aligned(workspace, 16));
    GMOE_CHECK_ARG(workspace_rows >= g.sum_rows + g.table_rows + g.split_rows);
    const int64_t row = (int64_t)E * H;  // floats
    float* sums = workspace;                                              // [parts][cols,H] fp32
    long long* table = reinterpret_cast<long long*>(workspace + g.sum_rows * row);
    unsigned char* terms = reinterpret_cast<unsigned char*>(workspace + (g.sum_rows + g.table_rows) * row);
    hipLaunchKernelGGL(gate_part_offsets_kernel, dim3(1), dim3(128), 0, st, table, g.parts,
                       (long long)g.part_rows, (long long)T);
    const void* grad = dlogits;
    if (split) {
      gate_split(dlogits, T, E, dtype, terms, st);
      grad = terms;
    }
    const int rc = gmm_grouped_tn(grad, x, sums, reinterpret_cast<const int64_t*>(table), g.parts, T,
                                  g.cols, H, dtype, GMOE_F32, st);
    if (rc != GMOE_OK) return rc;
    sum_partial_rows(sums, (int)g.sum_rows, row, dweight, dtype, st);
    return gmoe_launch_status();
  }
  const int parts = T > 0 ? gate_parts(T, H, E, dtype) : 0;
  if (T > 0) {
    GMOE_CHECK_ARG(dlogits && x && workspace);
    GMOE_CHECK_ARG(gmoe_aligned(dlogits, 4));  // its rows are read as dwords
    GMOE_CHECK_ARG(gmoe_aligned(x, 16) && gmoe_aligned(workspace, 16));
    GMOE_CHECK_ARG(workspace_rows >= parts);
    gate_by_types(dtype, logits_dtype, [&](auto dt, auto ldt) {
      constexpr int DT = decltype(dt)::value, LDT = decltype(ldt)::value;
      gate_by_e(E, [&](auto n, auto em) {
        hipLaunchKernelGGL((gate_bwd_weight_kernel<DT, LDT, decltype(n)::value, decltype(em)::value>),
                           dim3((unsigned)parts, gate_slabs(H, E, dtype)), dim3(kGateThreads), 0, st,
                           static_cast<const unsigned char*>(dlogits),
                           static_cast<const unsigned char*>(x), T, (int)H, E, workspace);
      });
    });
  }
  sum_partial_rows(workspace, parts, (int64_t)E * H, dweight, dtype, st);
  return gmoe_launch_status();
}
