// Top-k weighted combine of the expert outputs with the residual stream: the memory-bound step
// right after the expert path (forward_stage5 of the decoder layers, single-rank branch).
//
//   out[t, :] = residual[t, :] + S( sum_j float(moe[t*k + j, :]) * w[t, j] )
//
// with the products rounded to fp32, added in the order j = 0..k-1, the sum rounded once to the
// storage type S and the final addition rounded once more (what the tensor expression
// residual + (moe.view(T, k, H) * w[..., None]).sum(1).to(dtype) computes).  One workgroup per
// token; a thread owns 16-byte chunks of the row, so every access is a full-width vector access.
// Backward: d_moe[t*k + j, :] = S(float(g[t, :]) * w[t, j]), d_w[t, j] = sum_h g[t, h] * moe[t*k + j, h]
// (fp32, reduced over the workgroup in a fixed order: deterministic), d_residual = g.
//
// Expert-parallel branch of the same function: the expert outputs come back in the order of the
// dispatch sort, row r belonging to the flat top-k slot local_idxs[r], and the reference rounds
// every weighted row to S and adds it to a zeroed S accumulator (scatter_add_; on a GPU the order
// of those adds is whatever the atomics make it).  Here the rows of a token are added in
// ascending r, every partial sum rounded to S, which is what a sequential scatter_add_ gives:
//
//   out[t, :] = S( residual[t, :] + (..((0 + S(float(moe[r0,:]) * w0)) + S(float(moe[r1,:]) * w1)) ..) )
//
// through an inverse map slot_row[t*k + j] = r (or -1 for a slot without a row) built by
// pt_moe_combine_ep_index.  The backward is the one above with rows taken through slot_row.
#include "common.h"

// Cache policy (build switch, make EXTRA=-DPT_COMBINE_NT=<bits>): 1 = non-temporal loads of the
// expert rows and of the incoming gradient (each read once), 2 = non-temporal stores of the results.
// The results are the next operator's input and stay ordinary stores; the loads alone take 8-9 %
// off both kernels at 8192 tokens x top-8 x 2048 (forward 65.9 -> 60.9 us, backward 121 -> 110 us).
#ifndef PT_COMBINE_NT
#define PT_COMBINE_NT 1
#endif

namespace pt {

static constexpr int kMaxTopK = 16;

struct CombineArgs {
  const char *moe, *res, *go;
  char *out, *dmoe;
  const float* w;
  const int32_t* slot_row;  // expert-parallel branch: row of moe for every flat (token, choice) slot
  float* dw;
  int64_t rows;  // rows of moe in the expert-parallel branch: slot_row entries outside [0, rows) are ignored
  int64_t ld_moe, ld_res, ld_out, ld_go, ld_dmoe;  // bytes
  int32_t k;
  uint32_t H, chunks;  // chunks of 8 elements per row
  int vec;
};

// Expert-parallel forward: sequential S-rounded accumulation over the token's rows in ascending
// row order.  The first k threads rank the token's rows; everyone then walks the ranked list.
template <typename S>
__global__ __launch_bounds__(256) void moe_combine_ep_fwd_kernel(CombineArgs p) {
#pragma clang fp contract(off)
  __shared__ int32_t s_row[kMaxTopK];
  __shared__ float s_w[kMaxTopK];
  __shared__ int s_n;
  const int64_t t = blockIdx.x;
  if ((int)threadIdx.x < p.k) {
    const int32_t* sr = p.slot_row + t * p.k;
    const int32_t mine = sr[threadIdx.x] < p.rows ? sr[threadIdx.x] : -1;
    int rank = 0, n = 0;
    for (int j = 0; j < p.k; ++j) {
      const int32_t o = sr[j] < p.rows ? sr[j] : -1;
      n += o >= 0;
      rank += o >= 0 && o < mine;
    }
    if (mine >= 0) {
      s_row[rank] = mine;
      s_w[rank] = p.w[t * p.k + threadIdx.x];
    }
    if (threadIdx.x == 0) s_n = n;
  }
  __syncthreads();
  const int n = s_n;
  for (uint32_t c = threadIdx.x; c < p.chunks; c += 256) {
    const uint32_t col = c * 8u;
    const int nval = (p.H - col) < 8u ? (int)(p.H - col) : 8;
    const int64_t cb = (int64_t)col * S::kBytes;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    if (p.vec) {
      // Up to eight rows are requested together (a row past the list reads the first one again and
      // is not used); the accumulation walks them in list order as before.
      for (int j0 = 0; j0 < n; j0 += 8) {
        float m[8][8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          load8_policy<S, (PT_COMBINE_NT & 1) != 0>(p.moe + (int64_t)s_row[j0 + u < n ? j0 + u : j0] * p.ld_moe + cb, m[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const bool ok = j0 + u < n;
          const float wj = s_w[ok ? j0 + u : j0];
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[i] = ok ? S::round(acc[i] + S::round(m[u][i] * wj)) : acc[i];
        }
      }
    } else {
      for (int j = 0; j < n; ++j) {
        const char* mp = p.moe + (int64_t)s_row[j] * p.ld_moe + cb;
        const float wj = s_w[j];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float mi = i < nval ? S::load1(mp + i * S::kBytes) : 0.f;
          acc[i] = S::round(acc[i] + S::round(mi * wj));
        }
      }
    }
    const char* rp = p.res + t * p.ld_res + cb;
    char* op = p.out + t * p.ld_out + cb;
    if (p.vec) {
      float r[8], o[8];
      S::load8(rp, r);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = r[i] + acc[i];
      store8_policy<S, (PT_COMBINE_NT & 2) != 0>(op, o);
    } else {
      for (int i = 0; i < nval; ++i) S::store1(op + i * S::kBytes, S::load1(rp + i * S::kBytes) + acc[i]);
    }
  }
}

__global__ __launch_bounds__(256) void combine_slot_fill_kernel(int32_t* slot_row, int64_t slots) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < slots) slot_row[i] = -1;
}

__global__ __launch_bounds__(256) void combine_slot_index_kernel(const int64_t* local_idxs, int64_t rows, int64_t slots,
                                                                 int32_t* slot_row) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  const int64_t s = local_idxs[r];
  if (s >= 0 && s < slots) slot_row[s] = (int32_t)r;  // an index outside the slots is dropped, never followed
}

template <typename S>
__global__ __launch_bounds__(256) void moe_combine_fwd_kernel(CombineArgs p) {
  // The product is rounded before it is added (the reference materialises the product tensor): a
  // fused multiply-add would differ in the last bit often enough to move the rounding of the sum.
#pragma clang fp contract(off)
  const int64_t t = blockIdx.x;
  const float* w = p.w + t * p.k;
  for (uint32_t c = threadIdx.x; c < p.chunks; c += 256) {
    const uint32_t col = c * 8u;
    const int nval = (p.H - col) < 8u ? (int)(p.H - col) : 8;
    const int64_t cb = (int64_t)col * S::kBytes;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    if (p.vec) {
      // up to eight rows requested together; the sum still runs over j = 0, 1, ... in order
      for (int j0 = 0; j0 < p.k; j0 += 8) {
        float m[8][8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          load8_policy<S, (PT_COMBINE_NT & 1) != 0>(p.moe + (t * p.k + (j0 + u < p.k ? j0 + u : j0)) * p.ld_moe + cb, m[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const bool ok = j0 + u < p.k;
          const float wj = w[ok ? j0 + u : j0];
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[i] = ok ? acc[i] + m[u][i] * wj : acc[i];
        }
      }
    } else {
      for (int j = 0; j < p.k; ++j) {
        const char* mp = p.moe + (t * p.k + j) * p.ld_moe + cb;
        const float wj = w[j];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = acc[i] + (i < nval ? S::load1(mp + i * S::kBytes) : 0.f) * wj;
      }
    }
    char* op = p.out + t * p.ld_out + cb;
    if (p.res == nullptr) {
      // no residual: the rounded sum itself (the weighted sum of the single-device MoE forward)
      if (p.vec) store8_policy<S, (PT_COMBINE_NT & 2) != 0>(op, acc);
      else for (int i = 0; i < nval; ++i) S::store1(op + i * S::kBytes, acc[i]);
      continue;
    }
    const char* rp = p.res + t * p.ld_res + cb;
    // round the sum to the storage type, then add the residual and round again
    if (p.vec) {
      float r[8], o[8];
      S::load8(rp, r);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = r[i] + S::round(acc[i]);
      store8_policy<S, (PT_COMBINE_NT & 2) != 0>(op, o);
    } else {
      for (int i = 0; i < nval; ++i)
        S::store1(op + i * S::kBytes, S::load1(rp + i * S::kBytes) + S::round(acc[i]));
    }
  }
}

template <typename S>
__global__ __launch_bounds__(256) void moe_combine_bwd_kernel(CombineArgs p) {
  __shared__ float s_part[4][kMaxTopK];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float* w = p.w + t * p.k;
  float part[kMaxTopK];
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) part[j] = 0.f;
  for (uint32_t c = threadIdx.x; c < p.chunks; c += 256) {
    const uint32_t col = c * 8u;
    const int nval = (p.H - col) < 8u ? (int)(p.H - col) : 8;
    const int64_t cb = (int64_t)col * S::kBytes;
    float g[8];
    const char* gp = p.go + t * p.ld_go + cb;
    if (p.vec) load8_policy<S, (PT_COMBINE_NT & 1) != 0>(gp, g);
    else {
#pragma unroll
      for (int i = 0; i < 8; ++i) g[i] = i < nval ? S::load1(gp + i * S::kBytes) : 0.f;
    }
    if (p.vec) {
      // The rows of eight slots are requested together (a slot without a row reads the gradient
      // chunk again, memory that certainly exists, and neither stores nor accumulates).
#pragma unroll
      for (int j0 = 0; j0 < kMaxTopK; j0 += 8) {
        if (j0 < p.k) {
          int64_t row[8];
          float m[8][8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int j = j0 + u;
            int64_t r = -1;
            if (j < p.k) r = p.slot_row ? (int64_t)p.slot_row[t * p.k + j] : t * p.k + j;
            if (p.slot_row && r >= p.rows) r = -1;
            row[u] = r;
          }
#pragma unroll
          for (int u = 0; u < 8; ++u)
            load8_policy<S, (PT_COMBINE_NT & 1) != 0>(row[u] >= 0 ? p.moe + row[u] * p.ld_moe + cb : gp, m[u]);
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const bool ok = row[u] >= 0;
            const float wj = w[j0 + u < p.k ? j0 + u : 0];
            float d[8];
            float acc = part[j0 + u];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              d[i] = g[i] * wj;
              acc = fmaf(g[i], m[u][i], acc);
            }
            part[j0 + u] = ok ? acc : part[j0 + u];
            if (ok) store8_policy<S, (PT_COMBINE_NT & 2) != 0>(p.dmoe + row[u] * p.ld_dmoe + cb, d);
          }
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < kMaxTopK; ++j) {
        if (j < p.k) {
          const int64_t row = p.slot_row ? (int64_t)p.slot_row[t * p.k + j] : t * p.k + j;
          if (row < 0 || (p.slot_row && row >= p.rows)) continue;  // slot without a row: its weight gradient stays zero
          const char* mp = p.moe + row * p.ld_moe + cb;
          char* dp = p.dmoe + row * p.ld_dmoe + cb;
          const float wj = w[j];
          float acc = part[j];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float mi = i < nval ? S::load1(mp + i * S::kBytes) : 0.f;
            acc = fmaf(g[i], mi, acc);
            if (i < nval) S::store1(dp + i * S::kBytes, g[i] * wj);
          }
          part[j] = acc;
        }
      }
    }
  }
  // fixed-order reduction: lanes of a wave (xor butterfly), then the four waves in order
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) {
    if (j < p.k) {
      float v = part[j];
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
      if (lane == 0) s_part[wave][j] = v;
    }
  }
  __syncthreads();
  if ((int)threadIdx.x < p.k)
    p.dw[t * p.k + threadIdx.x] = ((s_part[0][threadIdx.x] + s_part[1][threadIdx.x]) + s_part[2][threadIdx.x]) + s_part[3][threadIdx.x];
}

static bool al16(const void* q) { return ((uintptr_t)q & 15) == 0; }

template <typename S, bool BWD>
static void launch_combine_typed(CombineArgs& a, int64_t T, hipStream_t stream) {
  if (BWD) hipLaunchKernelGGL(moe_combine_bwd_kernel<S>, dim3((unsigned)T), dim3(256), 0, stream, a);
  else if (a.slot_row) hipLaunchKernelGGL(moe_combine_ep_fwd_kernel<S>, dim3((unsigned)T), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(moe_combine_fwd_kernel<S>, dim3((unsigned)T), dim3(256), 0, stream, a);
}

template <bool BWD>
static int launch_combine(CombineArgs& a, int64_t T, int dtype, hipStream_t stream) {
  PT_REQUIRE(T < (1ll << 31), "moe_combine: too many tokens");
  switch (dtype) {
    case PT_BF16: launch_combine_typed<st_bf16, BWD>(a, T, stream); break;
    case PT_F16: launch_combine_typed<st_f16, BWD>(a, T, stream); break;
    case PT_F32: launch_combine_typed<st_f32, BWD>(a, T, stream); break;
    default: PT_REQUIRE(false, "moe_combine: unsupported dtype %d", dtype);
  }
  return check_launch(BWD ? "moe_combine_bwd_kernel" : "moe_combine_fwd_kernel");
}

}  // namespace pt

using namespace pt;

extern "C" int pt_moe_combine_fwd(const void* moe, int64_t ld_moe, const float* topk_weight, const void* residual,
                                  int64_t ld_res, void* out, int64_t ld_out, int64_t T, int32_t k, int64_t H, int dtype,
                                  pt_stream_t stream) {
  PT_REQUIRE(T >= 0 && H >= 0 && k >= 1 && k <= kMaxTopK, "moe_combine_fwd: bad sizes (1 <= k <= %d)", kMaxTopK);
  if (T == 0 || H == 0) return PT_OK;
  PT_REQUIRE(moe && topk_weight && out, "moe_combine_fwd: null pointer");
  PT_REQUIRE(ld_moe >= H && (!residual || ld_res >= H) && ld_out >= H && H < (1ll << 31), "moe_combine_fwd: bad leading dimension");
  const int eb = dtype == PT_F32 ? 4 : 2;
  CombineArgs a = {};
  a.moe = (const char*)moe; a.res = (const char*)residual; a.out = (char*)out; a.w = topk_weight;
  a.ld_moe = ld_moe * eb; a.ld_res = ld_res * eb; a.ld_out = ld_out * eb;
  a.k = k; a.H = (uint32_t)H; a.chunks = (uint32_t)cdiv(H, 8);
  a.vec = H % 8 == 0 && al16(moe) && al16(residual) && al16(out) && a.ld_moe % 16 == 0 && (!residual || a.ld_res % 16 == 0) && a.ld_out % 16 == 0;
  return launch_combine<false>(a, T, dtype, (hipStream_t)stream);
}

extern "C" int pt_moe_combine_bwd(const void* grad_out, int64_t ld_go, const void* moe, int64_t ld_moe,
                                  const float* topk_weight, void* d_moe, int64_t ld_dmoe, float* d_weight, int64_t T,
                                  int32_t k, int64_t H, int dtype, pt_stream_t stream) {
  PT_REQUIRE(T >= 0 && H >= 0 && k >= 1 && k <= kMaxTopK, "moe_combine_bwd: bad sizes (1 <= k <= %d)", kMaxTopK);
  if (T == 0) return PT_OK;
  PT_REQUIRE(grad_out && moe && topk_weight && d_moe && d_weight, "moe_combine_bwd: null pointer");
  PT_REQUIRE(ld_go >= H && ld_moe >= H && ld_dmoe >= H && H < (1ll << 31), "moe_combine_bwd: bad leading dimension");
  const int eb = dtype == PT_F32 ? 4 : 2;
  CombineArgs a = {};
  a.go = (const char*)grad_out; a.moe = (const char*)moe; a.dmoe = (char*)d_moe; a.w = topk_weight; a.dw = d_weight;
  a.ld_go = ld_go * eb; a.ld_moe = ld_moe * eb; a.ld_dmoe = ld_dmoe * eb;
  a.k = k; a.H = (uint32_t)H; a.chunks = (uint32_t)cdiv(H, 8);
  a.vec = H % 8 == 0 && al16(grad_out) && al16(moe) && al16(d_moe) && a.ld_go % 16 == 0 && a.ld_moe % 16 == 0 && a.ld_dmoe % 16 == 0;
  return launch_combine<true>(a, T, dtype, (hipStream_t)stream);
}

extern "C" int pt_moe_combine_ep_index(const int64_t* local_idxs, int64_t rows, int64_t slots, int32_t* slot_row,
                                       pt_stream_t stream) {
  PT_REQUIRE(rows >= 0 && slots >= 0 && rows < (1ll << 31) && slots < (1ll << 31), "moe_combine_ep_index: bad sizes");
  if (slots == 0) return PT_OK;
  PT_REQUIRE(slot_row && (local_idxs || rows == 0), "moe_combine_ep_index: null pointer");
  hipLaunchKernelGGL(combine_slot_fill_kernel, dim3((unsigned)cdiv(slots, 256)), dim3(256), 0, (hipStream_t)stream,
                     slot_row, slots);
  if (rows)
    hipLaunchKernelGGL(combine_slot_index_kernel, dim3((unsigned)cdiv(rows, 256)), dim3(256), 0, (hipStream_t)stream,
                       local_idxs, rows, slots, slot_row);
  return check_launch("combine_slot_index_kernel");
}

extern "C" int pt_moe_combine_ep_fwd(const void* moe, int64_t ld_moe, int64_t rows, const int32_t* slot_row,
                                     const float* topk_weight, const void* residual, int64_t ld_res, void* out,
                                     int64_t ld_out, int64_t T, int32_t k, int64_t H, int dtype, pt_stream_t stream) {
  PT_REQUIRE(T >= 0 && H >= 0 && rows >= 0 && k >= 1 && k <= kMaxTopK, "moe_combine_ep_fwd: bad sizes (1 <= k <= %d)", kMaxTopK);
  if (T == 0 || H == 0) return PT_OK;
  PT_REQUIRE(slot_row && topk_weight && residual && out && (moe || rows == 0), "moe_combine_ep_fwd: null pointer");
  PT_REQUIRE(ld_moe >= H && ld_res >= H && ld_out >= H && H < (1ll << 31), "moe_combine_ep_fwd: bad leading dimension");
  PT_REQUIRE(rows <= T * k, "moe_combine_ep_fwd: %lld rows for %lld slots", (long long)rows, (long long)(T * k));
  const int eb = dtype == PT_F32 ? 4 : 2;
  CombineArgs a = {};
  a.moe = (const char*)moe; a.res = (const char*)residual; a.out = (char*)out; a.w = topk_weight; a.slot_row = slot_row;
  a.rows = rows;
  a.ld_moe = ld_moe * eb; a.ld_res = ld_res * eb; a.ld_out = ld_out * eb;
  a.k = k; a.H = (uint32_t)H; a.chunks = (uint32_t)cdiv(H, 8);
  a.vec = H % 8 == 0 && al16(moe) && al16(residual) && al16(out) && a.ld_moe % 16 == 0 && a.ld_res % 16 == 0 && a.ld_out % 16 == 0;
  return launch_combine<false>(a, T, dtype, (hipStream_t)stream);
}

extern "C" int pt_moe_combine_ep_bwd(const void* grad_out, int64_t ld_go, const void* moe, int64_t ld_moe, int64_t rows,
                                     const int32_t* slot_row, const float* topk_weight, void* d_moe, int64_t ld_dmoe,
                                     float* d_weight, int64_t T, int32_t k, int64_t H, int dtype, pt_stream_t stream) {
  PT_REQUIRE(T >= 0 && H >= 0 && rows >= 0 && k >= 1 && k <= kMaxTopK, "moe_combine_ep_bwd: bad sizes (1 <= k <= %d)", kMaxTopK);
  if (T == 0) return PT_OK;
  PT_REQUIRE(grad_out && slot_row && topk_weight && d_weight && ((moe && d_moe) || rows == 0), "moe_combine_ep_bwd: null pointer");
  PT_REQUIRE(ld_go >= H && ld_moe >= H && ld_dmoe >= H && H < (1ll << 31), "moe_combine_ep_bwd: bad leading dimension");
  PT_REQUIRE(rows <= T * k, "moe_combine_ep_bwd: %lld rows for %lld slots", (long long)rows, (long long)(T * k));
  const int eb = dtype == PT_F32 ? 4 : 2;
  CombineArgs a = {};
  a.go = (const char*)grad_out; a.moe = (const char*)moe; a.dmoe = (char*)d_moe; a.w = topk_weight; a.dw = d_weight;
  a.slot_row = slot_row; a.rows = rows;
  a.ld_go = ld_go * eb; a.ld_moe = ld_moe * eb; a.ld_dmoe = ld_dmoe * eb;
  a.k = k; a.H = (uint32_t)H; a.chunks = (uint32_t)cdiv(H, 8);
  a.vec = H % 8 == 0 && al16(grad_out) && al16(moe) && al16(d_moe) && a.ld_go % 16 == 0 && a.ld_moe % 16 == 0 && a.ld_dmoe % 16 == 0;
  return launch_combine<true>(a, T, dtype, (hipStream_t)stream);
}
