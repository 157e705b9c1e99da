// Router gate after the logits GEMM: softmax, top-k selection and the weights of the chosen
// experts in one launch, the step right before the expert path (its topk_idx feed the dispatch).
//
//   mode 0 (Qwen3MoeGate, Qwen35MoeTopKRouter, DeepSeekV2MoEGate):
//       scores = softmax(logits, fp32); optionally only the topk_group best of num_group
//       contiguous expert groups (by their maximum score) keep their scores, the rest become 0;
//       topk_idx = top-k of scores; w = scores[topk_idx]; optionally w /= sum(w); w *= scale.
//   mode 1 (GptOssTopKRouter): topk_idx = top-k of the logits; w = softmax(logits[topk_idx], fp32).
//
// One wave per token, expert e in lane e % 64.  Selection is k rounds of a wave-wide maximum over
// 64-bit keys (value in an order-preserving integer form, then the smaller index): the result is
// sorted by descending value and ties go to the lower expert index.  All reductions have a fixed
// order, so the result is the same on every run.  With forced_idx (router replay) the selection
// is skipped and the weights are gathered at the given experts.
//
// Backward: the scores are recomputed from the logits (same code, same bits) and
//   mode 0: d_scores = scatter(d_w through the normalisation and the scale) [+ dense d_scores from
//           the load-balance loss], zero where the group limit zeroed the score;
//           d_logits = scores * (d_scores - sum(d_scores * scores)), rounded to the logits' type;
//   mode 1: d_l[topk] = w * (d_w - sum(d_w * w)) rounded to the logits' type [+ the rounded softmax
//           backward of the dense d_scores, added the way autograd adds two gradients].
#include "common.h"

namespace pt {

static constexpr int kRouterMaxK = 32;

struct RouterArgs {
  const char* logits;
  char* d_logits;
  int64_t ld_logits, ld_dlogits;  // bytes
  int64_t T;
  int32_t E, k, mode, norm, num_group, topk_group;
  float scale;
  const int64_t* forced_idx;  // forward: replayed selection (or null); backward: the selection of the forward
  int64_t* topk_idx;
  float* topk_weight;
  float* scores;          // forward: optional [T, E] output
  const float* d_weight;  // backward: [T, k]
  const float* d_scores;  // backward: optional [T, E]
};

__device__ __forceinline__ uint32_t orderable(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u >> 31) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float wave_max_f(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d));
  return v;
}
__device__ __forceinline__ float wave_sum_f(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
  return v;
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)v, d), hi = __shfl_xor((uint32_t)(v >> 32), d);
    const uint64_t o = ((uint64_t)hi << 32) | lo;
    v = o > v ? o : v;
  }
  return v;
}
__device__ __forceinline__ uint64_t make_key(float v, uint32_t index) {
  return ((uint64_t)orderable(v) << 32) | (0xFFFFFFFFu - index);
}

// Per-wave state of one token: the values the selection runs on (scores after the group limit in
// mode 0, logits in mode 1) in registers and in the wave's LDS row, and the unlimited softmax.
template <typename S, int VPT>
struct RouterToken {
  float soft[VPT];  // softmax of the logits (mode 0 always, mode 1 when asked for)
  float val[VPT];   // what the top-k runs on
  bool live[VPT];   // false where the group limit zeroed the score
};

template <typename S, int VPT>
__device__ __forceinline__ void router_token(const RouterArgs& p, int64_t t, int lane, float* s_row, bool want_soft,
                                             RouterToken<S, VPT>& r) {
  float x[VPT];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int e = i * 64 + lane;
    x[i] = e < p.E ? S::load1(p.logits + t * p.ld_logits + (int64_t)e * S::kBytes) : -INFINITY;
    m = fmaxf(m, x[i]);
    r.live[i] = e < p.E;
  }
  if (p.mode == 0 || want_soft) {
    m = wave_max_f(m);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      r.soft[i] = i * 64 + lane < p.E ? expf(x[i] - m) : 0.f;
      part += r.soft[i];
    }
    const float sum = wave_sum_f(part);
#pragma unroll
    for (int i = 0; i < VPT; ++i) r.soft[i] = r.soft[i] / sum;
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i) r.val[i] = p.mode == 0 ? r.soft[i] : x[i];
  if (p.mode == 0 && p.num_group > 1) {
    // group-limited greedy: the best topk_group groups (by their maximum score) stay
    const int gsz = p.E / p.num_group;
#pragma unroll
    for (int i = 0; i < VPT; ++i)
      if (i * 64 + lane < p.E) s_row[i * 64 + lane] = r.val[i];
    __syncthreads();
    uint64_t key = 0;
    if (lane < p.num_group) {
      float gm = s_row[lane * gsz];
      for (int q = 1; q < gsz; ++q) gm = fmaxf(gm, s_row[lane * gsz + q]);
      key = make_key(gm, (uint32_t)lane);
    }
    uint64_t keep = 0;
    for (int j = 0; j < p.topk_group; ++j) {
      const uint64_t best = wave_max_u64(key);
      const uint32_t g = 0xFFFFFFFFu - (uint32_t)best;
      keep |= 1ull << g;
      if ((uint32_t)lane == g) key = 0;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int e = i * 64 + lane;
      if (e < p.E && !((keep >> (e / gsz)) & 1)) {
        r.val[i] = 0.f;
        r.live[i] = false;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i)
    if (i * 64 + lane < p.E) s_row[i * 64 + lane] = r.val[i];
  __syncthreads();
}

template <typename S, int VPT>
__global__ __launch_bounds__(256) void router_topk_fwd_kernel(RouterArgs p) {
  __shared__ float s_val[4][VPT * 64];
  __shared__ int32_t s_sel[4][kRouterMaxK];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t tok = (int64_t)blockIdx.x * 4 + wave;
  const bool valid = tok < p.T;
  const int64_t t = valid ? tok : p.T - 1;  // waves past the end shadow the last token and store nothing
  float* s_row = s_val[wave];
  RouterToken<S, VPT> r;
  router_token<S, VPT>(p, t, lane, s_row, p.scores != nullptr, r);
  if (p.forced_idx) {
    if (lane < p.k) {
      int64_t e = p.forced_idx[t * p.k + lane];
      s_sel[wave][lane] = (int32_t)(e < 0 ? 0 : (e >= p.E ? p.E - 1 : e));
    }
  } else {
    uint64_t key[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) key[i] = i * 64 + lane < p.E ? make_key(r.val[i], (uint32_t)(i * 64 + lane)) : 0;
    for (int j = 0; j < p.k; ++j) {
      uint64_t local = 0;
#pragma unroll
      for (int i = 0; i < VPT; ++i) local = key[i] > local ? key[i] : local;
      const uint64_t best = wave_max_u64(local);
      const uint32_t e = 0xFFFFFFFFu - (uint32_t)best;
#pragma unroll
      for (int i = 0; i < VPT; ++i)
        if ((uint32_t)(i * 64 + lane) == e) key[i] = 0;
      if (lane == 0) s_sel[wave][j] = (int32_t)e;
    }
  }
  __syncthreads();
  float w = 0.f;
  if (p.mode == 0) {
    float total = 0.f;
    for (int j = 0; j < p.k; ++j) total += s_row[s_sel[wave][j]];
    if (lane < p.k) {
      w = s_row[s_sel[wave][lane]];
      if (p.norm) w = w / total;
      w = w * p.scale;
    }
  } else {
    float m = -INFINITY;
    for (int j = 0; j < p.k; ++j) m = fmaxf(m, s_row[s_sel[wave][j]]);
    float total = 0.f;
    for (int j = 0; j < p.k; ++j) total += expf(s_row[s_sel[wave][j]] - m);
    if (lane < p.k) w = expf(s_row[s_sel[wave][lane]] - m) / total;
  }
  if (!valid) return;
  if (lane < p.k) {
    p.topk_idx[t * p.k + lane] = s_sel[wave][lane];
    p.topk_weight[t * p.k + lane] = w;
  }
  if (p.scores) {
#pragma unroll
    for (int i = 0; i < VPT; ++i)
      if (i * 64 + lane < p.E) p.scores[t * p.E + i * 64 + lane] = p.mode == 0 ? r.val[i] : r.soft[i];
  }
}

template <typename S, int VPT>
__global__ __launch_bounds__(256) void router_topk_bwd_kernel(RouterArgs p) {
  __shared__ float s_val[4][VPT * 64];
  __shared__ float s_ds[4][VPT * 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t tok = (int64_t)blockIdx.x * 4 + wave;
  const bool valid = tok < p.T;
  const int64_t t = valid ? tok : p.T - 1;
  float* s_row = s_val[wave];
  float* ds_row = s_ds[wave];
  RouterToken<S, VPT> r;
  router_token<S, VPT>(p, t, lane, s_row, p.d_scores != nullptr, r);
  __shared__ int32_t s_sel[4][kRouterMaxK];
  if (lane < p.k) {
    const int64_t e = p.forced_idx[t * p.k + lane];
    s_sel[wave][lane] = (int32_t)(e < 0 ? 0 : (e >= p.E ? p.E - 1 : e));  // never index outside the row
  }
  const int32_t* sel = s_sel[wave];
  const float* dw = p.d_weight + t * p.k;
#pragma unroll
  for (int i = 0; i < VPT; ++i)
    if (i * 64 + lane < p.E) ds_row[i * 64 + lane] = (p.mode == 0 && p.d_scores) ? p.d_scores[t * p.E + i * 64 + lane] : 0.f;
  __syncthreads();
  if (lane == 0) {
    // one lane walks the k chosen experts in order: a replayed selection may name an expert twice
    if (p.mode == 0) {
      float total = 0.f, dot = 0.f;
      for (int j = 0; j < p.k; ++j) total += s_row[sel[j]];
      if (p.norm)
        for (int j = 0; j < p.k; ++j) dot += (dw[j] * p.scale) * (s_row[sel[j]] / total);
      for (int j = 0; j < p.k; ++j) {
        const float g = dw[j] * p.scale;
        ds_row[sel[j]] += p.norm ? (g - dot) / total : g;
      }
    } else {
      float m = -INFINITY, total = 0.f, dot = 0.f;
      for (int j = 0; j < p.k; ++j) m = fmaxf(m, s_row[sel[j]]);
      for (int j = 0; j < p.k; ++j) total += expf(s_row[sel[j]] - m);
      for (int j = 0; j < p.k; ++j) dot += dw[j] * (expf(s_row[sel[j]] - m) / total);
      for (int j = 0; j < p.k; ++j) {
        const float w = expf(s_row[sel[j]] - m) / total;
        ds_row[sel[j]] += S::round(w * (dw[j] - dot));
      }
    }
  }
  __syncthreads();
  float out[VPT];
  if (p.mode == 0) {
    float ds[VPT], part = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      ds[i] = (i * 64 + lane < p.E && r.live[i]) ? ds_row[i * 64 + lane] : 0.f;
      part += ds[i] * r.soft[i];
    }
    const float dot = wave_sum_f(part);
#pragma unroll
    for (int i = 0; i < VPT; ++i) out[i] = (ds[i] - dot) * r.soft[i];
  } else {
    float part = 0.f;
    if (p.d_scores) {
#pragma unroll
      for (int i = 0; i < VPT; ++i)
        if (i * 64 + lane < p.E) part += p.d_scores[t * p.E + i * 64 + lane] * r.soft[i];
    }
    const float dot = wave_sum_f(part);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int e = i * 64 + lane;
      out[i] = e < p.E ? ds_row[e] : 0.f;
      if (p.d_scores && e < p.E) out[i] = out[i] + S::round((p.d_scores[t * p.E + e] - dot) * r.soft[i]);
    }
  }
  if (!valid) return;
#pragma unroll
  for (int i = 0; i < VPT; ++i)
    if (i * 64 + lane < p.E) S::store1(p.d_logits + t * p.ld_dlogits + (int64_t)(i * 64 + lane) * S::kBytes, out[i]);
}

template <typename S, bool BWD>
static void launch_router_vpt(const RouterArgs& a, hipStream_t stream) {
  const dim3 grid((unsigned)cdiv(a.T, 4)), block(256);
#define PT_ROUTER_LAUNCH(V)                                                                     \
  do {                                                                                          \
    if (BWD) hipLaunchKernelGGL((router_topk_bwd_kernel<S, V>), grid, block, 0, stream, a);     \
    else hipLaunchKernelGGL((router_topk_fwd_kernel<S, V>), grid, block, 0, stream, a);         \
  } while (0)
  if (a.E <= 64) PT_ROUTER_LAUNCH(1);
  else if (a.E <= 128) PT_ROUTER_LAUNCH(2);
  else if (a.E <= 256) PT_ROUTER_LAUNCH(4);
  else PT_ROUTER_LAUNCH(8);
#undef PT_ROUTER_LAUNCH
}

template <bool BWD>
static int launch_router(const RouterArgs& a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case PT_BF16: launch_router_vpt<st_bf16, BWD>(a, stream); break;
    case PT_F16: launch_router_vpt<st_f16, BWD>(a, stream); break;
    case PT_F32: launch_router_vpt<st_f32, BWD>(a, stream); break;
    default: PT_REQUIRE(false, "router_topk: unsupported dtype %d", dtype);
  }
  return check_launch(BWD ? "router_topk_bwd_kernel" : "router_topk_fwd_kernel");
}

static int check_router_sizes(const char* who, int64_t T, int32_t E, int32_t k, int mode, int32_t num_group,
                              int32_t topk_group) {
  PT_REQUIRE(T >= 0 && T < (1ll << 33), "%s: bad token count", who);
  PT_REQUIRE(E >= 1 && E <= 512, "%s: 1 <= experts <= 512, got %d", who, E);
  PT_REQUIRE(k >= 1 && k <= kRouterMaxK && k <= E, "%s: 1 <= k <= min(%d, experts), got %d", who, kRouterMaxK, k);
  PT_REQUIRE(mode == 0 || mode == 1, "%s: mode must be 0 (softmax then top-k) or 1 (top-k then softmax)", who);
  PT_REQUIRE(num_group >= 1 && num_group <= 64 && E % num_group == 0, "%s: num_group must divide the experts and be <= 64", who);
  PT_REQUIRE(topk_group >= 1 && topk_group <= num_group, "%s: 1 <= topk_group <= num_group", who);
  PT_REQUIRE(num_group == 1 || mode == 0, "%s: the group limit belongs to mode 0", who);
  return PT_OK;
}

}  // namespace pt

using namespace pt;

extern "C" int pt_router_topk_fwd(const void* logits, int64_t ld_logits, int dtype, int64_t T, int32_t E, int32_t k,
                                  int mode, int norm_topk_prob, float scale, int32_t num_group, int32_t topk_group,
                                  const int64_t* forced_idx, int64_t* topk_idx, float* topk_weight, float* scores,
                                  pt_stream_t stream) {
  if (int rc = check_router_sizes("router_topk_fwd", T, E, k, mode, num_group, topk_group)) return rc;
  if (T == 0) return PT_OK;
  PT_REQUIRE(logits && topk_idx && topk_weight, "router_topk_fwd: null pointer");
  PT_REQUIRE(ld_logits >= E, "router_topk_fwd: bad leading dimension");
  RouterArgs a = {};
  a.logits = (const char*)logits; a.ld_logits = ld_logits * (dtype == PT_F32 ? 4 : 2);
  a.T = T; a.E = E; a.k = k; a.mode = mode; a.norm = norm_topk_prob; a.num_group = num_group; a.topk_group = topk_group;
  a.scale = scale; a.forced_idx = forced_idx; a.topk_idx = topk_idx; a.topk_weight = topk_weight; a.scores = scores;
  return launch_router<false>(a, dtype, (hipStream_t)stream);
}

extern "C" int pt_router_topk_bwd(const void* logits, int64_t ld_logits, int dtype, int64_t T, int32_t E, int32_t k,
                                  int mode, int norm_topk_prob, float scale, int32_t num_group, int32_t topk_group,
                                  const int64_t* topk_idx, const float* d_weight, const float* d_scores, void* d_logits,
                                  int64_t ld_dlogits, pt_stream_t stream) {
  if (int rc = check_router_sizes("router_topk_bwd", T, E, k, mode, num_group, topk_group)) return rc;
  if (T == 0) return PT_OK;
  PT_REQUIRE(logits && topk_idx && d_weight && d_logits, "router_topk_bwd: null pointer");
  PT_REQUIRE(ld_logits >= E && ld_dlogits >= E, "router_topk_bwd: bad leading dimension");
  const int eb = dtype == PT_F32 ? 4 : 2;
  RouterArgs a = {};
  a.logits = (const char*)logits; a.ld_logits = ld_logits * eb; a.d_logits = (char*)d_logits; a.ld_dlogits = ld_dlogits * eb;
  a.T = T; a.E = E; a.k = k; a.mode = mode; a.norm = norm_topk_prob; a.num_group = num_group; a.topk_group = topk_group;
  a.scale = scale; a.forced_idx = topk_idx; a.d_weight = d_weight; a.d_scores = d_scores;
  return launch_router<true>(a, dtype, (hipStream_t)stream);
}
