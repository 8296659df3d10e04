// Top-k router for gfx950: score function, top-k selection with a fixed tie rule, gate values,
// dense probs / routing-map outputs, per-expert token histogram and the statistics the
// load-balancing and z losses need, in one pass over the logits.  Follows
// `topk_softmax_with_capacity` (moe/moe_utils.py:430-518), `group_limited_topk` (:372-427),
// `compute_routing_scores_for_aux_loss` (moe/router.py:173-191), `switch_load_balancing_loss_func`
// (moe/moe_utils.py:14-59) and `z_loss_func` (:115-127).
//
// Work decomposition: a token's E logits are spread over a group of G consecutive lanes, 8 experts
// per lane (E <= 8*G, G a power of two), so a wavefront routes 64/G tokens at once.  A top-k step is
// a per-lane scan of 8 keys followed by a G-lane max all-reduce done with DPP row operations
// (ds_bpermute only for the 32- and 64-lane steps).  Keys are 64-bit: the order-preserving image of
// the fp32 score in the high word, ~expert in the low word, so that equal scores resolve to the
// lowest expert index and the winner's identity and value come out of the same reduction.
#include "route_common.h"

namespace gmoe {

struct RouteParams {
  const void* logits;
  int64_t T;
  int E;
  int k;
  int mode;  // 0 softmax after top-k, 1 softmax before top-k, 2 sigmoid
  float scaling;
  const float* expert_bias;
  const float* sel_override;  // [T,E] fp32, optional: what top-k ranks instead of the scores
  int num_groups;
  int group_topk;
  void* probs;
  uint8_t* map;
  int32_t* topk_idx;
  unsigned long long* counts;
  float* stats_ws;  // [gridDim.x][E+1]
};

template <int DT, int G>
__global__ __launch_bounds__(kRouteThreads) void route_topk_kernel(RouteParams p) {
  typedef Elem<DT> El;
  constexpr int TPW = GMOE_WAVE / G;                   // tokens per wavefront
  constexpr int TPB = TPW * (kRouteThreads / GMOE_WAVE);  // tokens per block iteration
  extern __shared__ unsigned char smem_raw[];
  int* hist = reinterpret_cast<int*>(smem_raw);  // [E]
  float* red = reinterpret_cast<float*>(smem_raw + ((p.E * 4 + 15) / 16) * 16);  // [4][G*kVpt + 1]

  const int tid = threadIdx.x;
  const int lane = tid & (GMOE_WAVE - 1);
  const int wave = tid >> 6;
  const int s = lane & (G - 1);  // position in the token's lane group
  const int e0 = s * kVpt;
  const int E = p.E;
  const bool want_stats = p.stats_ws != nullptr;

  for (int i = tid; i < E; i += kRouteThreads) hist[i] = 0;
  __syncthreads();

  float accP[kVpt];
#pragma unroll
  for (int v = 0; v < kVpt; ++v) accP[v] = 0.f;
  float accZ = 0.f;

  const int gsz = p.group_topk > 0 ? E / p.num_groups : 0;  // experts per routing group

  const int64_t num_tiles = (p.T + TPB - 1) / TPB;
  for (int64_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const int64_t t = tile * TPB + wave * TPW + lane / G;
    const bool tvalid = t < p.T;
    const int64_t row = (tvalid ? t : 0) * (int64_t)E;

    float logit[kVpt];
    bool evalid[kVpt];
#pragma unroll
    for (int v = 0; v < kVpt; ++v) {
      evalid[v] = (e0 + v) < E;
      logit[v] = evalid[v] ? El::load(p.logits, row + e0 + v) : -INFINITY;
    }

    // ---- full-row statistics (softmax over all experts) when some consumer needs them --------
    float rmax = 0.f, rsum = 1.f;
    const bool need_full = (p.mode == 1) || want_stats;
    if (need_full) {
      float m = -INFINITY;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) m = fmaxf(m, logit[v]);
      rmax = group_max_f32<G>(m);
      float sm = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) sm += evalid[v] ? expf(logit[v] - rmax) : 0.f;
      rsum = group_sum_f32<G>(sm);
    }

    // ---- scores used for selection and the (unnormalised) gate scores ------------------------
    float sel[kVpt];    // what top-k ranks
    float gate[kVpt];   // what the gate is computed from
#pragma unroll
    for (int v = 0; v < kVpt; ++v) {
      if (p.mode == 0) {
        sel[v] = gate[v] = logit[v];
      } else if (p.mode == 1) {
        sel[v] = gate[v] = El::round(expf(logit[v] - rmax) / rsum);
      } else {
        gate[v] = El::round(sigmoidf(logit[v]));
        sel[v] = p.expert_bias ? gate[v] + (evalid[v] ? p.expert_bias[e0 + v] : 0.f) : gate[v];
      }
    }

    if (p.sel_override) {
      // selection by an externally computed matrix (sinkhorn-normalised costs, moe/router.py:140-171);
      // the gates still come from the scores above
#pragma unroll
      for (int v = 0; v < kVpt; ++v) sel[v] = evalid[v] ? p.sel_override[row + e0 + v] : -INFINITY;
    }

    if (want_stats) {
      const float lse = rmax + logf(rsum);
      if (tvalid && s == 0) accZ += lse * lse;
      if (p.mode != 2) {
        if (tvalid) {
#pragma unroll
          for (int v = 0; v < kVpt; ++v)
            if (evalid[v]) accP[v] += expf(logit[v] - rmax) / rsum;
        }
      } else {
        float sm = 0.f;
#pragma unroll
        for (int v = 0; v < kVpt; ++v) sm += evalid[v] ? sigmoidf(logit[v]) : 0.f;
        const float ssum = group_sum_f32<G>(sm);
        const float den = p.k > 1 ? ssum + 1e-20f : 1.f;
        if (tvalid) {
#pragma unroll
          for (int v = 0; v < kVpt; ++v)
            if (evalid[v]) accP[v] += sigmoidf(logit[v]) / den;
        }
      }
    }

    uint32_t key[kVpt];
#pragma unroll
    for (int v = 0; v < kVpt; ++v) key[v] = evalid[v] ? score_key(sel[v]) : 0u;

    // ---- group-limited routing: keep the best `group_topk` routing groups ---------------------
    if (p.group_topk > 0) {
      const int m_per_group = p.k / p.group_topk;
      float my_group_score = 0.f;  // lane s holds the score of routing group s
      for (int g = 0; g < p.num_groups; ++g) {
        uint32_t taken = 0;
        float gs = 0.f;
        for (int j = 0; j < m_per_group; ++j) {
          uint64_t best = 0;
#pragma unroll
          for (int v = 0; v < kVpt; ++v) {
            const int e = e0 + v;
            const bool in = evalid[v] && (e / gsz == g) && !((taken >> v) & 1u);
            const uint64_t c = in ? ((uint64_t)key[v] << 32) | (0xffffffffu - (uint32_t)e) : 0ull;
            best = c > best ? c : best;
          }
          best = group_max_u64<G>(best);
          const int we = (int)(0xffffffffu - (uint32_t)best);
          gs += key_score((uint32_t)(best >> 32));
          if (we >= e0 && we < e0 + kVpt) taken |= 1u << (we - e0);
        }
        gs = El::round(gs);
        if (s == g) my_group_score = gs;
      }
      uint64_t chosen = 0;  // bitmask of surviving routing groups
      bool mine_taken = false;
      for (int j = 0; j < p.group_topk; ++j) {
        const bool in = (s < p.num_groups) && !mine_taken;
        uint64_t c = in ? ((uint64_t)score_key(my_group_score) << 32) | (0xffffffffu - (uint32_t)s)
                        : 0ull;
        c = group_max_u64<G>(c);
        const int wg = (int)(0xffffffffu - (uint32_t)c);
        chosen |= 1ull << wg;
        if (wg == s) mine_taken = true;
      }
      const uint32_t ninf_key = score_key(-INFINITY);
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        if (evalid[v] && !((chosen >> ((e0 + v) / gsz)) & 1ull)) key[v] = ninf_key;
      }
    }

    // ---- top-k -----------------------------------------------------------------------------
    uint32_t taken = 0;      // bit v: expert e0+v selected
    float first = 0.f;       // best selected score
    float denom = 0.f;       // softmax / sigmoid normaliser over the selected
    float selgate[kVpt];     // gate score of the selected experts of this lane
#pragma unroll
    for (int v = 0; v < kVpt; ++v) selgate[v] = 0.f;
    for (int j = 0; j < p.k; ++j) {
      uint64_t best = 0;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        const bool in = evalid[v] && !((taken >> v) & 1u);
        const uint64_t c = in ? ((uint64_t)key[v] << 32) | (0xffffffffu - (uint32_t)(e0 + v)) : 0ull;
        best = c > best ? c : best;
      }
      best = group_max_u64<G>(best);
      const int we = (int)(0xffffffffu - (uint32_t)best);
      float wscore;  // gate score of the winner, known to every lane of the group
      if ((p.mode == 2 && p.expert_bias) || p.sel_override) {
        // the ranked value is not the gate score (bias added, or another matrix ranked): fetch the
        // winner's gate score from the lane that owns it
        float mine = 0.f;
#pragma unroll
        for (int v = 0; v < kVpt; ++v) mine = (we == e0 + v) ? gate[v] : mine;
        wscore = group_sum_f32<G>((we >= e0 && we < e0 + kVpt) ? mine : 0.f);
      } else if (p.group_topk > 0) {
        // keys of masked experts were overwritten; fetch the true score from its owner
        float mine = 0.f;
#pragma unroll
        for (int v = 0; v < kVpt; ++v) mine = (we == e0 + v) ? gate[v] : mine;
        const bool masked = (uint32_t)(best >> 32) == score_key(-INFINITY);
        wscore = group_sum_f32<G>((we >= e0 && we < e0 + kVpt) ? mine : 0.f);
        if (masked && p.mode != 2) wscore = -INFINITY;
      } else {
        wscore = key_score((uint32_t)(best >> 32));
      }
      if (j == 0) first = wscore;
      if (p.mode == 0)
        denom += expf(wscore - first);
      else if (p.mode == 2)
        denom += wscore;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        if (we == e0 + v) {
          taken |= 1u << v;
          selgate[v] = wscore;
        }
      }
      if (p.topk_idx && tvalid && s == 0) p.topk_idx[t * p.k + j] = we;
    }
    if (p.mode == 2) denom = El::round(El::round(denom) + 1e-20f);

    // ---- outputs -----------------------------------------------------------------------------
    if (tvalid) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        if (!evalid[v]) continue;
        const bool on = (taken >> v) & 1u;
        float pr = 0.f;
        if (on) {
          if (p.mode == 0)
            pr = El::round(expf(selgate[v] - first) / denom);
          else if (p.mode == 1)
            pr = selgate[v];
          else
            pr = p.k > 1 ? El::round(selgate[v] / denom) : selgate[v];
          if (p.scaling > 0.f) pr = El::round(pr * p.scaling);
          atomicAdd(&hist[e0 + v], 1);
        }
        El::store(p.probs, row + e0 + v, pr);
        p.map[row + e0 + v] = on ? 1 : 0;
      }
    }
  }

  __syncthreads();
  for (int i = tid; i < E; i += kRouteThreads) {
    const int c = hist[i];
    if (c) atomicAdd(&p.counts[i], (unsigned long long)c);
  }

  if (want_stats) {
    // Fixed-order block reduction.  The lanes of a wavefront with the same position s in their lane
    // group hold the same experts: they meet in a butterfly over the lane bits above the group,
    // then thread e adds the four wavefront sums of expert e.  (One thread per expert walking all
    // 256 partials in LDS took 15 us of this kernel's 20 at 8 experts.)
#pragma unroll
    for (int d = G; d < GMOE_WAVE; d <<= 1) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v) accP[v] += __shfl_xor(accP[v], d);
      accZ += __shfl_xor(accZ, d);
    }
    constexpr int kWaveStride = G * kVpt + 1;  // [experts of the lane group | z]
    if (lane < G) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v) red[wave * kWaveStride + s * kVpt + v] = accP[v];
      if (s == 0) red[wave * kWaveStride + G * kVpt] = accZ;
    }
    __syncthreads();
    float* ws = p.stats_ws + (int64_t)blockIdx.x * (E + 1);
    for (int e = tid; e <= E; e += kRouteThreads) {
      const int idx = e < E ? e : G * kVpt;
      float a = red[idx];
#pragma unroll
      for (int w = 1; w < kRouteThreads / GMOE_WAVE; ++w) a += red[w * kWaveStride + idx];
      ws[e] = a;
    }
  }
}

__global__ void fill_u64_kernel(unsigned long long* p, int n, unsigned long long v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// ---- backward --------------------------------------------------------------------------------
struct RouteBwdParams {
  const void* logits;
  int64_t T;
  int E;
  int k;
  int mode;
  float scaling;
  const uint8_t* map;
  const void* dprobs;
  const long long* counts;
  const float* seq_counts;  // [batch, E] fp32, optional: per-sequence factors instead of counts
  int batch;                // token t belongs to sequence t % batch
  float aux_scale;
  float z_scale;
  const float* loss_scale;
  void* dlogits;
};

template <int DT, int G>
__global__ __launch_bounds__(kRouteThreads) void route_topk_bwd_kernel(RouteBwdParams p) {
  typedef Elem<DT> El;
  constexpr int TPW = GMOE_WAVE / G;
  constexpr int TPB = TPW * (kRouteThreads / GMOE_WAVE);
  const int tid = threadIdx.x;
  const int lane = tid & (GMOE_WAVE - 1);
  const int wave = tid >> 6;
  const int s = lane & (G - 1);
  const int e0 = s * kVpt;
  const int E = p.E;
  const float sc = p.scaling > 0.f ? p.scaling : 1.f;
  const float lscale = p.loss_scale ? p.loss_scale[0] : 1.f;
  const float aux_scale = p.aux_scale * lscale;
  const float z_scale = p.z_scale * lscale;

  float fcount[kVpt];
#pragma unroll
  for (int v = 0; v < kVpt; ++v)
    fcount[v] = (p.counts && (e0 + v) < E) ? (float)p.counts[e0 + v] : 0.f;

  const int64_t num_tiles = (p.T + TPB - 1) / TPB;
  for (int64_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const int64_t t = tile * TPB + wave * TPW + lane / G;
    const bool tvalid = t < p.T;
    const int64_t row = (tvalid ? t : 0) * (int64_t)E;

    float logit[kVpt], g[kVpt], dl[kVpt];
    bool evalid[kVpt], on[kVpt];
#pragma unroll
    for (int v = 0; v < kVpt; ++v) {
      evalid[v] = (e0 + v) < E;
      logit[v] = evalid[v] ? El::load(p.logits, row + e0 + v) : -INFINITY;
      on[v] = evalid[v] && p.map != nullptr && p.map[row + e0 + v] != 0;
      g[v] = on[v] ? sc * El::load(p.dprobs, row + e0 + v) : 0.f;
      dl[v] = 0.f;
    }
    if (p.seq_counts) {
      const int64_t b = (tvalid ? t : 0) % p.batch;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) fcount[v] = evalid[v] ? p.seq_counts[b * E + e0 + v] : 0.f;
    }

    // full softmax (needed by pre-softmax gates, softmax aux loss and z loss)
    float m = -INFINITY;
#pragma unroll
    for (int v = 0; v < kVpt; ++v) m = fmaxf(m, logit[v]);
    const float rmax = group_max_f32<G>(m);
    float sm = 0.f;
#pragma unroll
    for (int v = 0; v < kVpt; ++v) sm += evalid[v] ? expf(logit[v] - rmax) : 0.f;
    const float rsum = group_sum_f32<G>(sm);
    float sfull[kVpt];
#pragma unroll
    for (int v = 0; v < kVpt; ++v) sfull[v] = evalid[v] ? expf(logit[v] - rmax) / rsum : 0.f;

    if (p.mode == 0) {
      float ms = -INFINITY;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) ms = on[v] ? fmaxf(ms, logit[v]) : ms;
      const float smax = group_max_f32<G>(ms);
      float ss = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) ss += on[v] ? expf(logit[v] - smax) : 0.f;
      const float ssum = group_sum_f32<G>(ss);
      float pr[kVpt], d = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        pr[v] = on[v] ? expf(logit[v] - smax) / ssum : 0.f;
        d += pr[v] * g[v];
      }
      const float dot = group_sum_f32<G>(d);
#pragma unroll
      for (int v = 0; v < kVpt; ++v) dl[v] = pr[v] * (g[v] - dot);
    } else if (p.mode == 1) {
      float d = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) d += sfull[v] * g[v];
      const float dot = group_sum_f32<G>(d);
#pragma unroll
      for (int v = 0; v < kVpt; ++v) dl[v] = sfull[v] * (g[v] - dot);
    } else if (p.mode == 2) {
      float sg[kVpt], ss = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) {
        sg[v] = evalid[v] ? sigmoidf(logit[v]) : 0.f;
        ss += on[v] ? sg[v] : 0.f;
      }
      if (p.k > 1) {
        const float D = group_sum_f32<G>(ss) + 1e-20f;
        float d = 0.f;
#pragma unroll
        for (int v = 0; v < kVpt; ++v) d += on[v] ? (sg[v] / D) * g[v] : 0.f;
        const float dot = group_sum_f32<G>(d);
#pragma unroll
        for (int v = 0; v < kVpt; ++v)
          dl[v] = on[v] ? (g[v] - dot) / D * sg[v] * (1.f - sg[v]) : 0.f;
      } else {
#pragma unroll
        for (int v = 0; v < kVpt; ++v) dl[v] = on[v] ? g[v] * sg[v] * (1.f - sg[v]) : 0.f;
      }
      if (aux_scale != 0.f) {
        float sa = 0.f;
#pragma unroll
        for (int v = 0; v < kVpt; ++v) sa += sg[v];
        if (p.k > 1) {
          const float S = group_sum_f32<G>(sa) + 1e-20f;
          float d = 0.f;
#pragma unroll
          for (int v = 0; v < kVpt; ++v) d += (sg[v] / S) * fcount[v];
          const float dot = group_sum_f32<G>(d);
#pragma unroll
          for (int v = 0; v < kVpt; ++v)
            dl[v] += evalid[v] ? aux_scale * (fcount[v] - dot) / S * sg[v] * (1.f - sg[v]) : 0.f;
        } else {
#pragma unroll
          for (int v = 0; v < kVpt; ++v)
            dl[v] += evalid[v] ? aux_scale * fcount[v] * sg[v] * (1.f - sg[v]) : 0.f;
        }
      }
    }

    if (p.mode == 3) {
      // the input already holds the scores: the loss is linear in them
#pragma unroll
      for (int v = 0; v < kVpt; ++v) dl[v] = aux_scale * fcount[v];
    } else if (p.mode != 2 && aux_scale != 0.f) {
      float d = 0.f;
#pragma unroll
      for (int v = 0; v < kVpt; ++v) d += sfull[v] * fcount[v];
      const float dot = group_sum_f32<G>(d);
#pragma unroll
      for (int v = 0; v < kVpt; ++v) dl[v] += aux_scale * sfull[v] * (fcount[v] - dot);
    }
    if (z_scale != 0.f) {
      const float lse = rmax + logf(rsum);
#pragma unroll
      for (int v = 0; v < kVpt; ++v) dl[v] += z_scale * 2.f * lse * sfull[v];
    }

    if (tvalid) {
#pragma unroll
      for (int v = 0; v < kVpt; ++v)
        if (evalid[v]) El::store(p.dlogits, row + e0 + v, dl[v]);
    }
  }
}

template <int DT>
static int launch_route(const RouteParams& p, int G, int grid, size_t smem, hipStream_t st) {
#define GMOE_ROUTE_CASE(g)                                                           \
  case g:                                                                            \
    hipLaunchKernelGGL((route_topk_kernel<DT, g>), dim3(grid), dim3(kRouteThreads), smem, st, p); \
    break;
  switch (G) {
    GMOE_ROUTE_CASE(1)
    GMOE_ROUTE_CASE(2)
    GMOE_ROUTE_CASE(4)
    GMOE_ROUTE_CASE(8)
    GMOE_ROUTE_CASE(16)
    GMOE_ROUTE_CASE(32)
    GMOE_ROUTE_CASE(64)
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
#undef GMOE_ROUTE_CASE
  return GMOE_OK;
}

template <int DT>
static int launch_route_bwd(const RouteBwdParams& p, int G, int grid, hipStream_t st) {
#define GMOE_ROUTE_CASE(g)                                                              \
  case g:                                                                               \
    hipLaunchKernelGGL((route_topk_bwd_kernel<DT, g>), dim3(grid), dim3(kRouteThreads), 0, st, p); \
    break;
  switch (G) {
    GMOE_ROUTE_CASE(1)
    GMOE_ROUTE_CASE(2)
    GMOE_ROUTE_CASE(4)
    GMOE_ROUTE_CASE(8)
    GMOE_ROUTE_CASE(16)
    GMOE_ROUTE_CASE(32)
    GMOE_ROUTE_CASE(64)
    default:
      return GMOE_ERR_UNSUPPORTED;
  }
#undef GMOE_ROUTE_CASE
  return GMOE_OK;
}

}  // namespace gmoe

using namespace gmoe;

extern "C" int64_t gmoe_route_workspace_bytes(int64_t T, int E) {
  (void)T;
  return (int64_t)kRouteMaxBlocks * (E + 1) * (int64_t)sizeof(float);
}

extern "C" int gmoe_route_topk(const void* logits, int dtype, int64_t T, int E, int k, int score_fn,
                               int pre_softmax, float scaling, const float* expert_bias,
                               const float* selection_scores, int num_groups, int group_topk,
                               void* probs, uint8_t* routing_map,
                               int32_t* topk_idx, int64_t* tokens_per_expert, float* stats,
                               void* stats_ws, void* stream) {
  GMOE_CHECK_ARG(T >= 0 && E >= 1 && k >= 1 && k <= E);
  GMOE_CHECK_ARG(tokens_per_expert != nullptr);
  GMOE_CHECK_ARG(T == 0 || (logits && probs && routing_map));
  GMOE_CHECK_ARG(score_fn == GMOE_SCORE_SOFTMAX || score_fn == GMOE_SCORE_SIGMOID);
  GMOE_CHECK_ARG(stats == nullptr || stats_ws != nullptr);
  if (E > kVpt * GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  if (group_topk > 0) {
    GMOE_CHECK_ARG(num_groups > 0 && E % num_groups == 0 && group_topk <= num_groups);
    GMOE_CHECK_ARG(k % group_topk == 0 && k / group_topk <= E / num_groups);
    if (num_groups > GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  } else {
    num_groups = 0;
    group_topk = 0;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(fill_u64_kernel, dim3((E + 255) / 256), dim3(256), 0, st,
                     reinterpret_cast<unsigned long long*>(tokens_per_expert), E, 0ull);
  const int G = route_group_lanes(E, num_groups);
  const int grid = route_grid(T, G);
  if (T > 0) {
    RouteParams p;
    p.logits = logits;
    p.T = T;
    p.E = E;
    p.k = k;
    p.mode = score_fn == GMOE_SCORE_SIGMOID ? 2 : (pre_softmax ? 1 : 0);
    p.scaling = scaling;
    p.expert_bias = score_fn == GMOE_SCORE_SIGMOID ? expert_bias : nullptr;
    p.sel_override = selection_scores;
    p.num_groups = num_groups;
    p.group_topk = group_topk;
    p.probs = probs;
    p.map = routing_map;
    p.topk_idx = topk_idx;
    p.counts = reinterpret_cast<unsigned long long*>(tokens_per_expert);
    p.stats_ws = stats ? static_cast<float*>(stats_ws) : nullptr;
    const size_t smem = ((E * 4 + 15) / 16) * 16 + (size_t)kRouteThreads * (kVpt + 1) * 4;
    int rc;
    switch (dtype) {
      case GMOE_F32: rc = launch_route<GMOE_F32>(p, G, grid, smem, st); break;
      case GMOE_BF16: rc = launch_route<GMOE_BF16>(p, G, grid, smem, st); break;
      case GMOE_F16: rc = launch_route<GMOE_F16>(p, G, grid, smem, st); break;
      default: return GMOE_ERR_UNSUPPORTED;
    }
    if (rc != GMOE_OK) return rc;
  }
  if (stats) {
    hipLaunchKernelGGL(route_stats_reduce_kernel, dim3(E + 1), dim3(GMOE_WAVE), 0, st,
                       static_cast<const float*>(stats_ws), T > 0 ? grid : 0, E, stats);
  }
  return gmoe_launch_status();
}

static int route_bwd_launch(RouteBwdParams& p, int dtype, hipStream_t st) {
  const int G = route_group_lanes(p.E, 0);
  const int grid = route_grid(p.T, G);
  int rc;
  switch (dtype) {
    case GMOE_F32: rc = launch_route_bwd<GMOE_F32>(p, G, grid, st); break;
    case GMOE_BF16: rc = launch_route_bwd<GMOE_BF16>(p, G, grid, st); break;
    case GMOE_F16: rc = launch_route_bwd<GMOE_F16>(p, G, grid, st); break;
    default: return GMOE_ERR_UNSUPPORTED;
  }
  if (rc != GMOE_OK) return rc;
  return gmoe_launch_status();
}

extern "C" int gmoe_route_topk_bwd(const void* logits, int dtype, int64_t T, int E, int k,
                                   int score_fn, int pre_softmax, float scaling,
                                   const uint8_t* routing_map, const void* dprobs,
                                   const int64_t* tokens_per_expert, float aux_scale, float z_scale,
                                   const float* loss_scale, void* dlogits, void* stream) {
  GMOE_CHECK_ARG(T >= 0 && E >= 1 && k >= 1 && k <= E);
  GMOE_CHECK_ARG(T == 0 || (logits && routing_map && dprobs && dlogits));
  GMOE_CHECK_ARG(aux_scale == 0.f || tokens_per_expert != nullptr);
  if (E > kVpt * GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  if (T == 0) return GMOE_OK;
  RouteBwdParams p;
  p.logits = logits;
  p.T = T;
  p.E = E;
  p.k = k;
  p.mode = score_fn == GMOE_SCORE_SIGMOID ? 2 : (pre_softmax ? 1 : 0);
  p.scaling = scaling;
  p.map = routing_map;
  p.dprobs = dprobs;
  p.counts = reinterpret_cast<const long long*>(tokens_per_expert);
  p.seq_counts = nullptr;
  p.batch = 1;
  p.aux_scale = aux_scale;
  p.z_scale = z_scale;
  p.loss_scale = loss_scale;
  p.dlogits = dlogits;
  return route_bwd_launch(p, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int gmoe_seq_aux_loss_bwd(const void* logits, int dtype, int64_t seq_length,
                                     int batch_size, int E, int k, int score_fn,
                                     const float* seq_counts, float scale, const float* grad_loss,
                                     void* dlogits, void* stream) {
  GMOE_CHECK_ARG(seq_length >= 0 && batch_size >= 1 && E >= 1 && k >= 1 && k <= E);
  GMOE_CHECK_ARG(score_fn == GMOE_SCORE_SOFTMAX || score_fn == GMOE_SCORE_SIGMOID ||
                 score_fn == GMOE_SCORE_IDENTITY);
  if (E > kVpt * GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  const int64_t T = seq_length * batch_size;
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(logits && seq_counts && dlogits);
  RouteBwdParams p;
  p.logits = logits;
  p.T = T;
  p.E = E;
  p.k = k;
  p.mode = score_fn == GMOE_SCORE_SIGMOID ? 2 : (score_fn == GMOE_SCORE_IDENTITY ? 3 : 0);
  p.scaling = 0.f;
  p.map = nullptr;  // no gate gradient: only the loss term
  p.dprobs = nullptr;
  p.counts = nullptr;
  p.seq_counts = seq_counts;
  p.batch = batch_size;
  p.aux_scale = scale;
  p.z_scale = 0.f;
  p.loss_scale = grad_loss;
  p.dlogits = dlogits;
  return route_bwd_launch(p, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int gmoe_score_stats_bwd(const void* x, int dtype, int64_t T, int E, int k, int score_fn,
                                    const float* weights, float aux_scale, float z_scale,
                                    const float* grad_loss, void* dx, void* stream) {
  GMOE_CHECK_ARG(T >= 0 && E >= 1 && k >= 1 && k <= E);
  GMOE_CHECK_ARG(score_fn == GMOE_SCORE_SOFTMAX || score_fn == GMOE_SCORE_SIGMOID ||
                 score_fn == GMOE_SCORE_IDENTITY);
  GMOE_CHECK_ARG(aux_scale == 0.f || weights != nullptr);
  GMOE_CHECK_ARG(score_fn != GMOE_SCORE_IDENTITY || z_scale == 0.f);
  if (E > kVpt * GMOE_WAVE) return GMOE_ERR_UNSUPPORTED;
  if (T == 0) return GMOE_OK;
  GMOE_CHECK_ARG(x && dx);
  RouteBwdParams p;
  p.logits = x;
  p.T = T;
  p.E = E;
  p.k = k;
  p.mode = score_fn == GMOE_SCORE_SIGMOID ? 2 : (score_fn == GMOE_SCORE_IDENTITY ? 3 : 0);
  p.scaling = 0.f;
  p.map = nullptr;  // no gate gradient: only the loss terms
  p.dprobs = nullptr;
  p.counts = nullptr;
  p.seq_counts = aux_scale != 0.f ? weights : nullptr;
  p.batch = 1;
  p.aux_scale = aux_scale;
  p.z_scale = z_scale;
  p.loss_scale = grad_loss;
  p.dlogits = dx;
  return route_bwd_launch(p, dtype, static_cast<hipStream_t>(stream));
}
