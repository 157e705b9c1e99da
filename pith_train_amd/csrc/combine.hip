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
#include "common.h"

namespace pt {

static constexpr int kMaxTopK = 16;

struct CombineArgs {
  const char *moe, *res, *go;
  char *out, *dmoe;
  const float* w;
  float* dw;
  int64_t ld_moe, ld_res, ld_out, ld_go, ld_dmoe;  // bytes
  int32_t k;
  uint32_t H, chunks;  // chunks of 8 elements per row
  int vec;
};

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
    for (int j = 0; j < p.k; ++j) {
      const char* mp = p.moe + (t * p.k + j) * p.ld_moe + cb;
      float m[8];
      if (p.vec) S::load8(mp, m);
      else {
#pragma unroll
        for (int i = 0; i < 8; ++i) m[i] = i < nval ? S::load1(mp + i * S::kBytes) : 0.f;
      }
      const float wj = w[j];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = acc[i] + m[i] * wj;
    }
    const char* rp = p.res + t * p.ld_res + cb;
    char* op = p.out + t * p.ld_out + cb;
    // round the sum to the storage type, then add the residual and round again
    if (p.vec) {
      float r[8], o[8];
      S::load8(rp, r);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = r[i] + S::round(acc[i]);
      S::store8(op, o);
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
    if (p.vec) S::load8(gp, g);
    else {
#pragma unroll
      for (int i = 0; i < 8; ++i) g[i] = i < nval ? S::load1(gp + i * S::kBytes) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < kMaxTopK; ++j) {
      if (j < p.k) {
        const char* mp = p.moe + (t * p.k + j) * p.ld_moe + cb;
        char* dp = p.dmoe + (t * p.k + j) * p.ld_dmoe + cb;
        float m[8], d[8];
        if (p.vec) S::load8(mp, m);
        else {
#pragma unroll
          for (int i = 0; i < 8; ++i) m[i] = i < nval ? S::load1(mp + i * S::kBytes) : 0.f;
        }
        const float wj = w[j];
        float acc = part[j];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          d[i] = g[i] * wj;
          acc = fmaf(g[i], m[i], acc);
        }
        part[j] = acc;
        if (p.vec) S::store8(dp, d);
        else
          for (int i = 0; i < nval; ++i) S::store1(dp + i * S::kBytes, d[i]);
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

template <bool BWD>
static int launch_combine(CombineArgs& a, int64_t T, int dtype, hipStream_t stream) {
  PT_REQUIRE(T < (1ll << 31), "moe_combine: too many tokens");
  switch (dtype) {
    case PT_BF16:
      if (BWD) hipLaunchKernelGGL(moe_combine_bwd_kernel<st_bf16>, dim3((unsigned)T), dim3(256), 0, stream, a);
      else hipLaunchKernelGGL(moe_combine_fwd_kernel<st_bf16>, dim3((unsigned)T), dim3(256), 0, stream, a);
      break;
    case PT_F16:
      if (BWD) hipLaunchKernelGGL(moe_combine_bwd_kernel<st_f16>, dim3((unsigned)T), dim3(256), 0, stream, a);
      else hipLaunchKernelGGL(moe_combine_fwd_kernel<st_f16>, dim3((unsigned)T), dim3(256), 0, stream, a);
      break;
    case PT_F32:
      if (BWD) hipLaunchKernelGGL(moe_combine_bwd_kernel<st_f32>, dim3((unsigned)T), dim3(256), 0, stream, a);
      else hipLaunchKernelGGL(moe_combine_fwd_kernel<st_f32>, dim3((unsigned)T), dim3(256), 0, stream, a);
      break;
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
  PT_REQUIRE(moe && topk_weight && residual && out, "moe_combine_fwd: null pointer");
  PT_REQUIRE(ld_moe >= H && ld_res >= H && ld_out >= H && H < (1ll << 31), "moe_combine_fwd: bad leading dimension");
  const int eb = dtype == PT_F32 ? 4 : 2;
  CombineArgs a = {};
  a.moe = (const char*)moe; a.res = (const char*)residual; a.out = (char*)out; a.w = topk_weight;
  a.ld_moe = ld_moe * eb; a.ld_res = ld_res * eb; a.ld_out = ld_out * eb;
  a.k = k; a.H = (uint32_t)H; a.chunks = (uint32_t)cdiv(H, 8);
  a.vec = H % 8 == 0 && al16(moe) && al16(residual) && al16(out) && a.ld_moe % 16 == 0 && a.ld_res % 16 == 0 && a.ld_out % 16 == 0;
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
