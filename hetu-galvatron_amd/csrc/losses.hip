// Router losses and bookkeeping that the reference computes with small torch graphs, as device-side
// work on the router's own outputs (no host synchronisation, fixed summation orders):
//   * the sequence-level load-balancing loss (`sequence_load_balancing_loss_func`,
//     moe/moe_utils.py:62-112; its gradient is a mode of route_topk_bwd_kernel in route.hip);
//   * the sinkhorn normalisation of the routing costs (`sinkhorn`, moe/moe_utils.py:130-144);
//   * the loss values from the router kernel's statistics, their logging tracker
//     (`save_to_aux_losses_tracker`, moe/moe_utils.py:547-574), the token-count accumulation of the
//     expert-bias scheme (moe/router.py:415-419) and the bias update itself
//     (`get_updated_expert_bias`, moe/moe_utils.py:645-662).
#include "route_common.h"

namespace gmoe {

// Sum over the lanes of a wavefront that hold the same position of their token's lane group
// (lanes l with equal l % G), same order in every lane.
template <int G>
__device__ __forceinline__ float across_groups_sum(float v) {
#pragma unroll
  for (int m = G; m < GMOE_WAVE; m <<= 1) v += __shfl_xor(v, m);
  return v;
}

// The normalised routing scores of one token (`compute_routing_scores_for_aux_loss`,
// moe/router.py:173-191): fp32 softmax over all experts, or sigmoid divided by its sum (k > 1).
// score_fn GMOE_SCORE_IDENTITY: the input already holds the scores.
template <int G>
__device__ __forceinline__ void routing_scores(const float (&logit)[kVpt], const bool (&evalid)[kVpt],
                                               int score_fn, int k, float (&score)[kVpt]) {
  if (score_fn == GMOE_SCORE_IDENTITY) {
#pragma unroll
    for (int v = 0; v < kVpt; ++v) score[v] = evalid[v] ? logit[v] : 0.f;
  } else if (score_fn == GMOE_SCORE_SOFTMAX) {
    float m = -INFINITY;
#pragma unroll
    for (int v = 0; v < kVpt; ++v) m = fmaxf(m, logit[v]);
    const float rmax = group_max_f32<G>(m);
    float sm = 0.f;
#pragma unroll
    for (int v = 0; v < kVpt; ++v) sm += evalid[v] ? expf(logit[v] - rmax) : 0.f;
    const float rsum = group_sum_f32<G>(sm);
#pragma unroll
    for (int v = 0; v < kVpt; ++v) score[v] = evalid[v] ? expf(logit[v] - rmax) / rsum : 0.f;
  } else {
    float sm = 0.f;
#pragma unroll
    for (int v = 0; v < kVpt; ++v) {
      score[v] = evalid[v] ? sigmoidf(logit[v]) : 0.f;
      sm += score[v];
    }
    const float den = k > 1 ? group_sum_f32<G>(sm) + 1e-20f : 1.f;
#pragma unroll
    for (int v = 0; v < kVpt; ++v) score[v] = score[v] / den;
  }
}

// ---- sequence-level load-balancing loss ------------------------------------------------------------
// One workgroup per sequence b: token (s, b) is row s * B + b.  counts[b,e] = number of tokens of the
// sequence routed to e, scores[b,e] = sum_s score(s,b,e).
constexpr int kSeqThreads = 256;

template <int DT, int G>
__global__ __launch_bounds__(kSeqThreads) void seq_aux_stats_kernel(
    const void* logits, const uint8_t* map, int64_t S, int B, int E, int k, int score_fn,
    float* seq_counts, float* seq_scores) {
  typedef Elem<DT> El;
  constexpr int TPW = GMOE_WAVE / G;
  constexpr int NW = kSeqThreads / GMOE_WAVE;
  __shared__ float red[NW][2][G * kVpt];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int s = lane & (G - 1), e0 = s * kVpt;
  const int b = blockIdx.x;
  float accP[kVpt], accC[kVpt];
  bool evalid[kVpt];
#pragma unroll
  for (int v = 0; v < kVpt; ++v) {
    accP[v] = accC[v] = 0.f;
    evalid[v] = (e0 + v) < E;
  }
  for (int64_t q0 = 0; q0 < S; q0 += NW * TPW) {
    const int64_t q = q0 + wave * TPW + lane / G;
    const bool tvalid = q < S;
    const int64_t row = ((tvalid ? q : 0) * B + b) * (int64_t)E;
    float logit[kVpt], score[kVpt];
#pragma unroll
    for (int v = 0; v < kVpt; ++v) logit[v] = evalid[v] ? El::load(logits, row + e0 + v) : -INFINITY;
    routing_scores<G>(logit, evalid, score_fn, k, score);
    if (tvalid) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        accP[v] += score[v];
        accC[v] += (evalid[v] && map[row + e0 + v] != 0) ? 1.f : 0.f;
      }
    }
  }
#pragma unroll
  for (int v = 0; v < kVpt; ++v) {
    const float p = across_groups_sum<G>(accP[v]);
    const float c = across_groups_sum<G>(accC[v]);
    if (lane < G) {
      red[wave][0][e0 + v] = p;
      red[wave][1][e0 + v] = c;
    }
  }
  __syncthreads();
  for (int e = tid; e < E; e += kSeqThreads) {
    float p = 0.f, c = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      p += red[w][0][e];
      c += red[w][1][e];
    }
    seq_scores[(int64_t)b * E + e] = p;
    seq_counts[(int64_t)b * E + e] = c;
  }
}

// loss = scale * sum_b sum_e counts[b,e] * scores[b,e], summed per sequence by one wavefront each in
// lane-strided order, the sequences added in ascending order.
__global__ __launch_bounds__(64) void seq_aux_finish_kernel(const float* seq_counts,
                                                            const float* seq_scores, int B, int E,
                                                            float scale, float* loss) {
  const int lane = threadIdx.x;
  float total = 0.f;
  for (int b = 0; b < B; ++b) {
    float a = 0.f;
    for (int e = lane; e < E; e += 64) a += seq_counts[(int64_t)b * E + e] * seq_scores[(int64_t)b * E + e];
    total += wave_sum_f32(a);
  }
  if (lane == 0) loss[0] = total * scale;
}

// ---- sinkhorn ----------------------------------------------------------------------------------------
// One workgroup iterates d0 <- (1/T) / (cost d1 + eps), d1 <- (1/E) / (cost^T d0 + eps) until the mean
// change of d1 is at most tol.  cost = exp(logits) in fp32 sits in the output buffer (it stays in
// L2); every pass over it computes a token's d0 from the previous d1 and adds the token's
// contribution to the column sums of the new d1, so an iteration reads the matrix once.  The last
// pass forms d1 * cost * d0 in place.  Column sums are reduced in a fixed order.
constexpr int kSinkThreads = 1024;

template <int DT, int G>
__global__ __launch_bounds__(kSinkThreads) void sinkhorn_kernel(const void* logits, int64_t T, int E,
                                                                float tol, int max_iters, float* out,
                                                                int* iters_out) {
  typedef Elem<DT> El;
  constexpr int TPW = GMOE_WAVE / G;
  constexpr int NW = kSinkThreads / GMOE_WAVE;
  constexpr int TPB = TPW * NW;
  __shared__ float d1[G * kVpt], d1_prev[G * kVpt];
  __shared__ float red[NW][G * kVpt];
  __shared__ float errw[8];
  __shared__ float err_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int s = lane & (G - 1), e0 = s * kVpt;
  const float eps = 0.00000001f;
  const float inv_t = 1.f / (float)T, inv_e = 1.f / (float)E;
  bool evalid[kVpt];
#pragma unroll
  for (int v = 0; v < kVpt; ++v) evalid[v] = (e0 + v) < E;

  for (int e = tid; e < G * kVpt; e += kSinkThreads) d1[e] = e < E ? 1.f : 0.f;
  // cost = exp(logits)
  for (int64_t t0 = 0; t0 < T; t0 += TPB) {
    const int64_t t = t0 + wave * TPW + lane / G;
    if (t < T) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v)
        if (evalid[v]) out[t * E + e0 + v] = expf(El::load(logits, t * E + e0 + v));
    }
  }
  __syncthreads();  // a thread reads back only what it wrote itself; d1 is what needs the barrier

  int it = 0;
  float err = 1e9f;
  while (err > tol && it < max_iters) {
    float dv[kVpt], col[kVpt];
#pragma unroll
    for (int v = 0; v < kVpt; ++v) {
      dv[v] = d1[e0 + v];
      col[v] = 0.f;
    }
    for (int64_t t0 = 0; t0 < T; t0 += TPB) {
      const int64_t t = t0 + wave * TPW + lane / G;
      const bool tvalid = t < T;
      float c[kVpt], r = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        c[v] = (tvalid && evalid[v]) ? out[t * E + e0 + v] : 0.f;
        r += dv[v] * c[v];
      }
      r = group_sum_f32<G>(r);
      const float d0 = inv_t * 1.f / (r + eps);
      if (tvalid) {
#pragma unroll
        for (int v = 0; v < kVpt; ++v) col[v] += d0 * c[v];
      }
    }
#pragma unroll
    for (int v = 0; v < kVpt; ++v) {
      const float a = across_groups_sum<G>(col[v]);
      if (lane < G) red[wave][e0 + v] = a;
    }
    __syncthreads();
    float diff = 0.f;
    if (tid < G * kVpt) {
      const int e = tid;
      float a = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) a += red[w][e];
      const float old = d1[e];
      const float nw = e < E ? inv_e * 1.f / (a + eps) : 0.f;
      d1_prev[e] = old;
      d1[e] = nw;
      diff = e < E ? fabsf(old - nw) : 0.f;
    }
    // G * kVpt <= 512: the first eight wavefronts hold the differences
    if (wave < 8) {
      const float wsum = wave_sum_f32(diff);
      if (lane == 0) errw[wave] = wsum;
    }
    __syncthreads();
    if (tid == 0) {
      float a = 0.f;
      for (int w = 0; w < 8; ++w) a += errw[w];
      err_s = a * inv_e;
    }
    __syncthreads();
    err = err_s;
    ++it;
    __syncthreads();  // err_s, errw and red are rewritten in the next iteration
  }

  // d1 * cost * d0 with d0 of the last iteration (computed from d1_prev)
  float dp[kVpt], dn[kVpt];
#pragma unroll
  for (int v = 0; v < kVpt; ++v) {
    dp[v] = it > 0 ? d1_prev[e0 + v] : 0.f;
    dn[v] = d1[e0 + v];
  }
  for (int64_t t0 = 0; t0 < T; t0 += TPB) {
    const int64_t t = t0 + wave * TPW + lane / G;
    const bool tvalid = t < T;
    float c[kVpt], r = 0.f;
#pragma unroll
    for (int v = 0; v < kVpt; ++v) {
      c[v] = (tvalid && evalid[v]) ? out[t * E + e0 + v] : 0.f;
      r += dp[v] * c[v];
    }
    r = group_sum_f32<G>(r);
    const float d0 = it > 0 ? inv_t * 1.f / (r + eps) : 1.f;
    if (tvalid) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v)
        if (evalid[v]) out[t * E + e0 + v] = dn[v] * c[v] * d0;
    }
  }
  if (iters_out && tid == 0) iters_out[0] = it;
}

// ---- loss values, tracker, token-count accumulation ---------------------------------------------
// aux = aux_factor * sum_e stats[e] * tokens_per_expert[e]   (moe/moe_utils.py:55-58)
// z   = z_factor * stats[E]                                   (moe/moe_utils.py:126)
__global__ __launch_bounds__(64) void router_bookkeeping_kernel(
    const float* stats, const long long* counts, int E, float aux_factor, float z_factor,
    float* aux_loss, float* z_loss, float* aux_slot, float aux_slot_scale, float* z_slot,
    float z_slot_scale, float* local_tokens) {
  const int lane = threadIdx.x;
  if (stats != nullptr && (aux_loss != nullptr || aux_slot != nullptr)) {
    float a = 0.f;
    for (int e = lane; e < E; e += 64) a += stats[e] * (float)counts[e];
    a = wave_sum_f32(a) * aux_factor;
    if (lane == 0) {
      if (aux_loss) aux_loss[0] = a;
      if (aux_slot) aux_slot[0] += a * aux_slot_scale;
    }
  }
  if (stats != nullptr && lane == 0 && (z_loss != nullptr || z_slot != nullptr)) {
    const float z = stats[E] * z_factor;
    if (z_loss) z_loss[0] = z;
    if (z_slot) z_slot[0] += z * z_slot_scale;
  }
  if (local_tokens != nullptr && counts != nullptr)
    for (int e = lane; e < E; e += 64) local_tokens[e] += (float)counts[e];
}

// out[r,e] = bias[r,e] + sign(mean_e(tokens[r,:]) - tokens[r,e]) * rate, one wavefront per row
__global__ __launch_bounds__(64) void expert_bias_update_kernel(const float* tokens,
                                                                const float* bias, int E, float rate,
                                                                float* out) {
  const int lane = threadIdx.x;
  const int64_t r = blockIdx.x;
  float a = 0.f;
  for (int e = lane; e < E; e += 64) a += tokens[r * E + e];
  const float mean = wave_sum_f32(a) / (float)E;
  for (int e = lane; e < E; e += 64) {
    const float off = mean - tokens[r * E + e];
    const float sgn = off > 0.f ? 1.f : (off < 0.f ? -1.f : off);  // sign(0) = 0, NaN stays NaN
    out[r * E + e] = bias[r * E + e] + sgn * rate;
  }
}

// ---- column statistics of a [T,E] score or logit matrix ---------------------------------------------
// What the free functions `switch_load_balancing_loss_func` (moe/moe_utils.py:14-59) and `z_loss_func`
// (:115-127) reduce over the tokens: partial[e] = sum_t score(x)[t,e] and partial[E] = sum_t
// logsumexp(x[t,:])^2 per workgroup, in the router kernel's lane layout; route_stats_reduce_kernel
// adds the workgroups' partials in a fixed order.
template <int DT, int G>
__global__ __launch_bounds__(kRouteThreads) void score_stats_kernel(const void* x, int64_t T, int E,
                                                                    int k, int score_fn, float* ws) {
  typedef Elem<DT> El;
  constexpr int TPW = GMOE_WAVE / G;
  constexpr int NW = kRouteThreads / GMOE_WAVE;
  constexpr int TPB = TPW * NW;
  __shared__ float red[NW][G * kVpt + 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int s = lane & (G - 1), e0 = s * kVpt;
  float accP[kVpt], accZ = 0.f;
  bool evalid[kVpt];
#pragma unroll
  for (int v = 0; v < kVpt; ++v) {
    accP[v] = 0.f;
    evalid[v] = (e0 + v) < E;
  }
  const int64_t num_tiles = (T + TPB - 1) / TPB;
  for (int64_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const int64_t t = tile * TPB + wave * TPW + lane / G;
    const bool tvalid = t < T;
    const int64_t row = (tvalid ? t : 0) * (int64_t)E;
    float logit[kVpt], score[kVpt];
#pragma unroll
    for (int v = 0; v < kVpt; ++v) logit[v] = evalid[v] ? El::load(x, row + e0 + v) : -INFINITY;
    routing_scores<G>(logit, evalid, score_fn, k, score);
    if (score_fn != GMOE_SCORE_IDENTITY) {
      float m = -INFINITY;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) m = fmaxf(m, logit[v]);
      const float rmax = group_max_f32<G>(m);
      float sm = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) sm += evalid[v] ? expf(logit[v] - rmax) : 0.f;
      const float lse = rmax + logf(group_sum_f32<G>(sm));
      if (tvalid && s == 0) accZ += lse * lse;
    }
    if (tvalid) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v) accP[v] += score[v];
    }
  }
#pragma unroll
  for (int v = 0; v < kVpt; ++v) {
    const float p = across_groups_sum<G>(accP[v]);
    if (lane < G) red[wave][e0 + v] = p;
  }
  accZ = across_groups_sum<G>(accZ);
  if (lane == 0) red[wave][G * kVpt] = accZ;
  __syncthreads();
  float* out = ws + (int64_t)blockIdx.x * (E + 1);
  for (int e = tid; e <= E; e += kRouteThreads) {
    const int idx = e < E ? e : G * kVpt;
    float a = red[0][idx];
#pragma unroll
    for (int w = 1; w < NW; ++w) a += red[w][idx];
    out[e] = a;
  }
}

template <int DT>
static int launch_score_stats(int G, int grid, const void* x, int64_t T, int E, int k, int score_fn,
                              float* ws, hipStream_t st) {
#define GMOE_CASE(g)                                                                                \
  case g:                                                                                           \
    hipLaunchKernelGGL((score_stats_kernel<DT, g>), dim3(grid), dim3(kRouteThreads), 0, st, x, T, E, \
                       k, score_fn, ws);                                                            \
    break;
  switch (G) {
    GMOE_CASE(1) GMOE_CASE(2) GMOE_CASE(4) GMOE_CASE(8) GMOE_CASE(16) GMOE_CASE(32) GMOE_CASE(64)
    default: return GMOE_ERR_UNSUPPORTED;
  }
#undef GMOE_CASE
  return GMOE_OK;
}

template <int DT>
static int launch_seq_stats(int G, const void* logits, const uint8_t* map, int64_t S, int B, int E,
                            int k, int score_fn, float* counts, float* scores, hipStream_t st) {
#define GMOE_CASE(g)                                                                              \
  case g:                                                                                         \
    hipLaunchKernelGGL((seq_aux_stats_kernel<DT, g>), dim3(B), dim3(kSeqThreads), 0, st, logits, \
                       map, S, B, E, k, score_fn, counts, scores);                                 \
    break;
  switch (G) {
    GMOE_CASE(1) GMOE_CASE(2) GMOE_CASE(4) GMOE_CASE(8) GMOE_CASE(16) GMOE_CASE(32) GMOE_CASE(64)
    default: return GMOE_ERR_UNSUPPORTED;
  }
#undef GMOE_CASE
  return GMOE_OK;
}

template <int DT>
static int launch_sinkhorn(int G, const void* logits, int64_t T, int E, float tol, int max_iters,
                           float* out, int* iters, hipStream_t st) {
#define GMOE_CASE(g)                                                                               \
  case g:                                                                                          \
    hipLaunchKernelGGL((sinkhorn_kernel<DT, g>), dim3(1), dim3(kSinkThreads), 0, st, logits, T, E, \
                       tol, max_iters, out, iters);                                                \
    break;
  switch (G) {
    GMOE_CASE(1) GMOE_CASE(2) GMOE_CASE(4) GMOE_CASE(8) GMOE_CASE(16) GMOE_CASE(32) GMOE_CASE(64)
    default: return GMOE_ERR_UNSUPPORTED;
  }
#undef GMOE_CASE
  return GMOE_OK;
}

}  // namespace gmoe

using namespace gmoe;

extern "C" int gmoe_seq_aux_loss(const void* logits, int dtype, const uint8_t* routing_map,
                                 int64_t seq_length, int batch_size, int E, int k, int score_fn,
                                 float coeff, float* seq_counts, float* seq_scores, float* loss,
                                 void* stream) {
  GMOE_CHECK_ARG(seq_length >= 1 && batch_size >= 1 && E >= 1 && k >= 1 && k <= E);
  GMOE_CHECK_ARG(score_fn == GMOE_SCORE_SOFTMAX || score_fn == GMOE_SCORE_SIGMOID ||
                 score_fn == GMOE_SCORE_IDENTITY);
  GMOE_CHECK_ARG(logits && routing_map && seq_counts && seq_scores && loss);
  if (E > kVpt * GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int G = route_group_lanes(E, 0);
  const int sig = score_fn;
  int rc;
  switch (dtype) {
    case GMOE_F32: rc = launch_seq_stats<GMOE_F32>(G, logits, routing_map, seq_length, batch_size, E, k, sig, seq_counts, seq_scores, st); break;
    case GMOE_BF16: rc = launch_seq_stats<GMOE_BF16>(G, logits, routing_map, seq_length, batch_size, E, k, sig, seq_counts, seq_scores, st); break;
    case GMOE_F16: rc = launch_seq_stats<GMOE_F16>(G, logits, routing_map, seq_length, batch_size, E, k, sig, seq_counts, seq_scores, st); break;
    default: return GMOE_ERR_UNSUPPORTED;
  }
  if (rc != GMOE_OK) return rc;
  // cost_coeff = counts * E / (S k), mean over s of the scores, sum over e, mean over b, times coeff
  const float scale = coeff * (float)E /
                      ((float)batch_size * (float)seq_length * (float)seq_length * (float)k);
  hipLaunchKernelGGL(seq_aux_finish_kernel, dim3(1), dim3(64), 0, st, seq_counts, seq_scores,
                     batch_size, E, scale, loss);
  return gmoe_launch_status();
}

extern "C" int gmoe_score_stats(const void* x, int dtype, int64_t T, int E, int k, int score_fn,
                                float* stats, void* stats_ws, void* stream) {
  GMOE_CHECK_ARG(T >= 0 && E >= 1 && k >= 1 && k <= E && stats != nullptr && stats_ws != nullptr);
  GMOE_CHECK_ARG(score_fn == GMOE_SCORE_SOFTMAX || score_fn == GMOE_SCORE_SIGMOID ||
                 score_fn == GMOE_SCORE_IDENTITY);
  GMOE_CHECK_ARG(T == 0 || x != nullptr);
  if (E > kVpt * GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int G = route_group_lanes(E, 0);
  const int grid = route_grid(T, G);
  if (T > 0) {
    int rc;
    float* ws = static_cast<float*>(stats_ws);
    switch (dtype) {
      case GMOE_F32: rc = launch_score_stats<GMOE_F32>(G, grid, x, T, E, k, score_fn, ws, st); break;
      case GMOE_BF16: rc = launch_score_stats<GMOE_BF16>(G, grid, x, T, E, k, score_fn, ws, st); break;
      case GMOE_F16: rc = launch_score_stats<GMOE_F16>(G, grid, x, T, E, k, score_fn, ws, st); break;
      default: return GMOE_ERR_UNSUPPORTED;
    }
    if (rc != GMOE_OK) return rc;
  }
  hipLaunchKernelGGL(route_stats_reduce_kernel, dim3(E + 1), dim3(GMOE_WAVE), 0, st,
                     static_cast<const float*>(stats_ws), T > 0 ? grid : 0, E, stats);
  return gmoe_launch_status();
}

extern "C" int gmoe_sinkhorn(const void* logits, int dtype, int64_t T, int E, float tol,
                             int max_iters, float* norm_out, int* iters_out, void* stream) {
  GMOE_CHECK_ARG(T >= 0 && E >= 1 && max_iters >= 1 && tol >= 0.f);
  if (E > kVpt * GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(logits && norm_out);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int G = route_group_lanes(E, 0);
  int rc;
  switch (dtype) {
    case GMOE_F32: rc = launch_sinkhorn<GMOE_F32>(G, logits, T, E, tol, max_iters, norm_out, iters_out, st); break;
    case GMOE_BF16: rc = launch_sinkhorn<GMOE_BF16>(G, logits, T, E, tol, max_iters, norm_out, iters_out, st); break;
    case GMOE_F16: rc = launch_sinkhorn<GMOE_F16>(G, logits, T, E, tol, max_iters, norm_out, iters_out, st); break;
    default: return GMOE_ERR_UNSUPPORTED;
  }
  if (rc != GMOE_OK) return rc;
  return gmoe_launch_status();
}

extern "C" int gmoe_router_bookkeeping(const float* stats, const int64_t* tokens_per_expert, int E,
                                       float aux_factor, float z_factor, float* aux_loss,
                                       float* z_loss, float* aux_tracker_slot,
                                       float aux_tracker_scale, float* z_tracker_slot,
                                       float z_tracker_scale, float* local_tokens_per_expert,
                                       void* stream) {
  GMOE_CHECK_ARG(E >= 1);
  const bool wants_aux = aux_loss != nullptr || aux_tracker_slot != nullptr;
  const bool wants_z = z_loss != nullptr || z_tracker_slot != nullptr;
  GMOE_CHECK_ARG(!(wants_aux || wants_z) || stats != nullptr);
  GMOE_CHECK_ARG(!(wants_aux || local_tokens_per_expert != nullptr) || tokens_per_expert != nullptr);
  hipLaunchKernelGGL(router_bookkeeping_kernel, dim3(1), dim3(64), 0,
                     static_cast<hipStream_t>(stream), stats,
                     reinterpret_cast<const long long*>(tokens_per_expert), E, aux_factor, z_factor,
                     aux_loss, z_loss, aux_tracker_slot, aux_tracker_scale, z_tracker_slot,
                     z_tracker_scale, local_tokens_per_expert);
  return gmoe_launch_status();
}

extern "C" int gmoe_expert_bias_update(const float* tokens_per_expert, const float* expert_bias,
                                       int64_t rows, int E, float update_rate, float* updated_bias,
                                       void* stream) {
  GMOE_CHECK_ARG(rows >= 0 && E >= 1 && rows < (1ll << 31));
  if (rows == 0) return GMOE_OK;
  GMOE_CHECK_ARG(tokens_per_expert && expert_bias && updated_bias);
  hipLaunchKernelGGL(expert_bias_update_kernel, dim3((unsigned)rows), dim3(64), 0,
                     static_cast<hipStream_t>(stream), tokens_per_expert, expert_bias, E,
                     update_rate, updated_bias);
  return gmoe_launch_status();
}
