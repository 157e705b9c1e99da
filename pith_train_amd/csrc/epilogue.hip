// Fused activation / bias epilogues of the expert path (HBM-bound elementwise kernels).
//
// Every thread moves 8 elements per step with 16-byte loads/stores (two for fp32); math is
// fp32 with one rounding to the storage type.  Grids are sized to the element count so that a
// launch has many more workgroups than the 256 CUs.
#include "common.h"

namespace pt {

// sigmoidf_fast / silu_mul_f / silu_mul_b live in common.h (shared with the fused quantisation).

template <typename S>
__global__ __launch_bounds__(256) void silu_mul_fwd_kernel(const char* gate, const char* up, char* out, int64_t n) {
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i0 >= n) return;
  if (i0 + 8 <= n) {
    float g[8], u[8], o[8];
    S::load8(gate + i0 * S::kBytes, g);
    S::load8(up + i0 * S::kBytes, u);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = silu_mul_f(g[j], u[j]);
    S::store8(out + i0 * S::kBytes, o);
  } else {
    for (int64_t i = i0; i < n; ++i) {
      const float g = S::load1(gate + i * S::kBytes), u = S::load1(up + i * S::kBytes);
      S::store1(out + i * S::kBytes, silu_mul_f(g, u));
    }
  }
}

template <typename S>
__global__ __launch_bounds__(256) void silu_mul_bwd_kernel(const char* go, const char* gate, const char* up,
                                                           char* dgate, char* dup, int64_t n) {
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i0 >= n) return;
  auto one = [](float d, float g, float u, float& dg, float& du) { silu_mul_b(d, g, u, dg, du); };
  if (i0 + 8 <= n) {
    float d[8], g[8], u[8], dg[8], du[8];
    S::load8(go + i0 * S::kBytes, d);
    S::load8(gate + i0 * S::kBytes, g);
    S::load8(up + i0 * S::kBytes, u);
#pragma unroll
    for (int j = 0; j < 8; ++j) one(d[j], g[j], u[j], dg[j], du[j]);
    S::store8(dgate + i0 * S::kBytes, dg);
    S::store8(dup + i0 * S::kBytes, du);
  } else {
    for (int64_t i = i0; i < n; ++i) {
      float dg, du;
      one(S::load1(go + i * S::kBytes), S::load1(gate + i * S::kBytes), S::load1(up + i * S::kBytes), dg, du);
      S::store1(dgate + i * S::kBytes, dg);
      S::store1(dup + i * S::kBytes, du);
    }
  }
}

// ---- silu_mul on row-strided operands ---------------------------------------------------------------
// gate / up / out (and their gradients) are [rows, cols] views with their own leading dimensions
// (in elements), e.g. the two halves of a fused gate_up buffer.  One thread per 8-element chunk.
struct Silu2dArgs {
  const char *go, *gate, *up;
  char *out, *dgate, *dup;
  int64_t ld_go, ld_gate, ld_up, ld_out, ld_dgate, ld_dup;  // bytes
  uint32_t rows, cols, chunks_per_row, total_chunks;
  int vec;
};

template <typename S, bool BWD>
__global__ __launch_bounds__(256) void silu_mul_2d_kernel(Silu2dArgs p) {
  const uint32_t c = blockIdx.x * 256u + threadIdx.x;
  if (c >= p.total_chunks) return;
  const uint32_t r = c / p.chunks_per_row;
  const uint32_t col = (c - r * p.chunks_per_row) * 8u;
  const int64_t cb = (int64_t)col * S::kBytes;
  const char* gp = p.gate + r * p.ld_gate + cb;
  const char* upp = p.up + r * p.ld_up + cb;
  float g[8], u[8];
  const int nval = (p.cols - col) < 8u ? (int)(p.cols - col) : 8;
  if (p.vec) {
    S::load8(gp, g);
    S::load8(upp, u);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      g[j] = j < nval ? S::load1(gp + j * S::kBytes) : 0.f;
      u[j] = j < nval ? S::load1(upp + j * S::kBytes) : 0.f;
    }
  }
  if (!BWD) {
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = silu_mul_f(g[j], u[j]);
    char* op = p.out + r * p.ld_out + cb;
    if (p.vec) S::store8(op, o);
    else
      for (int j = 0; j < nval; ++j) S::store1(op + j * S::kBytes, o[j]);
  } else {
    float d[8], dg[8], du[8];
    const char* dp = p.go + r * p.ld_go + cb;
    if (p.vec) S::load8(dp, d);
    else {
#pragma unroll
      for (int j = 0; j < 8; ++j) d[j] = j < nval ? S::load1(dp + j * S::kBytes) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) silu_mul_b(d[j], g[j], u[j], dg[j], du[j]);
    char* dgp = p.dgate + r * p.ld_dgate + cb;
    char* dup = p.dup + r * p.ld_dup + cb;
    if (p.vec) {
      S::store8(dgp, dg);
      S::store8(dup, du);
    } else {
      for (int j = 0; j < nval; ++j) {
        S::store1(dgp + j * S::kBytes, dg[j]);
        S::store1(dup + j * S::kBytes, du[j]);
      }
    }
  }
}

// ---- clamped SwiGLU (interleaved gate/up) ---------------------------------------------------------
// cswiglu_f / cswiglu_b live in common.h (shared with the fused quantisation).
template <typename S>
__global__ __launch_bounds__(256) void clamped_swiglu_fwd_kernel(const char* gu, char* out, int64_t n, float alpha, float limit) {
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i0 >= n) return;
  if (i0 + 8 <= n) {
    float a[8], b[8], o[8];
    S::load8(gu + (2 * i0) * S::kBytes, a);
    S::load8(gu + (2 * i0 + 8) * S::kBytes, b);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[j] = cswiglu_f(a[2 * j], a[2 * j + 1], alpha, limit);
      o[4 + j] = cswiglu_f(b[2 * j], b[2 * j + 1], alpha, limit);
    }
    S::store8(out + i0 * S::kBytes, o);
  } else {
    for (int64_t i = i0; i < n; ++i)
      S::store1(out + i * S::kBytes,
                cswiglu_f(S::load1(gu + (2 * i) * S::kBytes), S::load1(gu + (2 * i + 1) * S::kBytes), alpha, limit));
  }
}

template <typename S>
__global__ __launch_bounds__(256) void clamped_swiglu_bwd_kernel(const char* go, const char* gu, char* dgu, int64_t n,
                                                                 float alpha, float limit) {
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i0 >= n) return;
  if (i0 + 8 <= n) {
    float d[8], a[8], b[8], da[8], db[8];
    S::load8(go + i0 * S::kBytes, d);
    S::load8(gu + (2 * i0) * S::kBytes, a);
    S::load8(gu + (2 * i0 + 8) * S::kBytes, b);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      cswiglu_b(d[j], a[2 * j], a[2 * j + 1], alpha, limit, da[2 * j], da[2 * j + 1]);
      cswiglu_b(d[4 + j], b[2 * j], b[2 * j + 1], alpha, limit, db[2 * j], db[2 * j + 1]);
    }
    S::store8(dgu + (2 * i0) * S::kBytes, da);
    S::store8(dgu + (2 * i0 + 8) * S::kBytes, db);
  } else {
    for (int64_t i = i0; i < n; ++i) {
      float dg, du;
      cswiglu_b(S::load1(go + i * S::kBytes), S::load1(gu + (2 * i) * S::kBytes), S::load1(gu + (2 * i + 1) * S::kBytes),
                alpha, limit, dg, du);
      S::store1(dgu + (2 * i) * S::kBytes, dg);
      S::store1(dgu + (2 * i + 1) * S::kBytes, du);
    }
  }
}

// ---- x + bias[group_ids] -----------------------------------------------------------------------------
template <typename S>
__global__ __launch_bounds__(256) void bias_add_kernel(const char* x, const char* bias, const int64_t* gid, char* out,
                                                       int64_t M, int64_t H, int vec) {
  if (vec) {
    const int64_t chunks = H / 8;
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= M * chunks) return;
    const int64_t r = c / chunks, h = (c - r * chunks) * 8;
    float a[8], b[8];
    S::load8(x + (r * H + h) * S::kBytes, a);
    S::load8(bias + (gid[r] * H + h) * S::kBytes, b);
#pragma unroll
    for (int j = 0; j < 8; ++j) a[j] += b[j];
    S::store8(out + (r * H + h) * S::kBytes, a);
  } else {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= M * H) return;
    const int64_t r = i / H, h = i - r * H;
    S::store1(out + i * S::kBytes, S::load1(x + i * S::kBytes) + S::load1(bias + (gid[r] * H + h) * S::kBytes));
  }
}

// ---- per-group row sums -----------------------------------------------------------------------------
// grid (ceil(H/128), G); 16 column chunks x 16 row lanes; fp32 accumulate, fixed order.
// row_index (optional): grouped row r is x[row_index[r]] (negative: a padding row, nothing to add),
// i.e. the sum runs over the grouped order while x stays un-permuted.
template <typename S, typename O>
__global__ __launch_bounds__(256) void segment_sum_kernel(const char* x, const int32_t* offs, char* out, int64_t M,
                                                          int64_t H, int vec, const int32_t* row_index, int64_t x_rows) {
  __shared__ float s[16][129];
  const int g = blockIdx.y;
  const int cc = threadIdx.x & 15, rl = threadIdx.x >> 4;
  int64_t start = g == 0 ? 0 : (int64_t)offs[g - 1];
  int64_t end = offs[g];
  if (end > M) end = M;
  if (start > M) start = M;
  const int64_t h0 = (int64_t)blockIdx.x * 128 + cc * 8;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (vec) {
    // Eight rows of the thread in flight at a time, and the row indices of the next eight are
    // requested before this batch's data is waited for (an index and the row it names are two
    // dependent memory latencies otherwise).  The additions stay in row order, so the sum has the
    // bits of a one-row-at-a-time loop.
    constexpr int U = 8;
    auto indices = [&](int64_t r, int64_t (&src)[U]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t ru = r + 16 * u;
        src[u] = ru < end ? (row_index ? (int64_t)row_index[ru] : ru) : -1;
        if (src[u] >= x_rows) src[u] = -1;
      }
    };
    if (h0 < H) {
      int64_t src[U], nxt[U];
      indices(start + rl, src);
      for (int64_t r = start + rl; r < end; r += 16 * U) {
        // (rows that do not exist read row 0 and are not added: no branch around a load)
        float v[U][8];
#pragma unroll
        for (int u = 0; u < U; ++u) S::load8(x + ((src[u] >= 0 ? src[u] : 0) * H + h0) * S::kBytes, v[u]);
        indices(r + 16 * U, nxt);
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j] = src[u] >= 0 ? acc[j] + v[u][j] : acc[j];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) src[u] = nxt[u];
      }
    }
  } else {
    for (int64_t r = start + rl; r < end; r += 16) {
      const int64_t src = row_index ? (int64_t)row_index[r] : r;
      if (src < 0 || src >= x_rows) continue;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (h0 + j < H) acc[j] += S::load1(x + (src * H + h0 + j) * S::kBytes);
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) s[rl][cc * 8 + j] = acc[j];
  __syncthreads();
  if (threadIdx.x < 128) {
    const int64_t h = (int64_t)blockIdx.x * 128 + threadIdx.x;
    if (h < H) {
      float t = 0.f;
#pragma unroll
      for (int q = 0; q < 16; ++q) t += s[q][threadIdx.x];
      O::store1(out + ((int64_t)g * H + h) * O::kBytes, t);
    }
  }
}

static inline unsigned blocks8(int64_t n) { return (unsigned)cdiv(cdiv(n, 8), 256); }

#define PT_DISPATCH_ST(dtype, NAME, ...)                                   \
  switch (dtype) {                                                         \
    case PT_BF16: NAME<st_bf16> __VA_ARGS__; break;                        \
    case PT_F16:  NAME<st_f16> __VA_ARGS__; break;                         \
    case PT_F32:  NAME<st_f32> __VA_ARGS__; break;                         \
    default: PT_REQUIRE(false, "unsupported dtype %d", dtype);             \
  }

}  // namespace pt

using namespace pt;

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

extern "C" int pt_silu_mul_fwd(const void* gate, const void* up, void* out, int64_t n, int dtype, pt_stream_t stream) {
  if (n == 0) return PT_OK;
  PT_REQUIRE(n > 0 && gate && up && out, "silu_mul_fwd: bad arguments");
  PT_REQUIRE(aligned16(gate) && aligned16(up) && aligned16(out), "silu_mul_fwd: pointers must be 16-byte aligned");
  PT_REQUIRE(cdiv(n, 2048) < (1ll << 31), "silu_mul_fwd: too many elements");
  hipStream_t s = (hipStream_t)stream;
  PT_DISPATCH_ST(dtype, silu_mul_fwd_kernel, <<<blocks8(n), 256, 0, s>>>((const char*)gate, (const char*)up, (char*)out, n));
  return check_launch("silu_mul_fwd");
}

extern "C" int pt_silu_mul_bwd(const void* go, const void* gate, const void* up, void* dgate, void* dup, int64_t n,
                               int dtype, pt_stream_t stream) {
  if (n == 0) return PT_OK;
  PT_REQUIRE(n > 0 && go && gate && up && dgate && dup, "silu_mul_bwd: bad arguments");
  PT_REQUIRE(aligned16(go) && aligned16(gate) && aligned16(up) && aligned16(dgate) && aligned16(dup),
             "silu_mul_bwd: pointers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  PT_DISPATCH_ST(dtype, silu_mul_bwd_kernel,
                 <<<blocks8(n), 256, 0, s>>>((const char*)go, (const char*)gate, (const char*)up, (char*)dgate, (char*)dup, n));
  return check_launch("silu_mul_bwd");
}

static int silu_2d_setup(Silu2dArgs& a, int64_t rows, int64_t cols, int dtype, const char* what) {
  PT_REQUIRE(rows > 0 && cols > 0, "%s: bad shape", what);
  const int64_t cpr = cdiv(cols, 8);
  PT_REQUIRE(rows * cpr < (1ll << 31), "%s: too many elements", what);
  a.rows = (uint32_t)rows; a.cols = (uint32_t)cols; a.chunks_per_row = (uint32_t)cpr;
  a.total_chunks = (uint32_t)(rows * cpr);
  (void)dtype;
  return PT_OK;
}

extern "C" int pt_silu_mul_fwd_2d(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* out,
                                  int64_t ld_out, int64_t rows, int64_t cols, int dtype, pt_stream_t stream) {
  if (rows == 0 || cols == 0) return PT_OK;
  PT_REQUIRE(gate && up && out && ld_gate >= cols && ld_up >= cols && ld_out >= cols, "silu_mul_fwd_2d: bad arguments");
  const int eb = dtype == PT_F32 ? 4 : 2;
  Silu2dArgs a{};
  if (int rc = silu_2d_setup(a, rows, cols, dtype, "silu_mul_fwd_2d")) return rc;
  a.gate = (const char*)gate; a.up = (const char*)up; a.out = (char*)out;
  a.ld_gate = ld_gate * eb; a.ld_up = ld_up * eb; a.ld_out = ld_out * eb;
  a.vec = cols % 8 == 0 && aligned16(gate) && aligned16(up) && aligned16(out) && a.ld_gate % 16 == 0 &&
          a.ld_up % 16 == 0 && a.ld_out % 16 == 0;
  hipStream_t s = (hipStream_t)stream;
  const unsigned blocks = (unsigned)cdiv((int64_t)a.total_chunks, 256);
  switch (dtype) {
    case PT_BF16: silu_mul_2d_kernel<st_bf16, false><<<blocks, 256, 0, s>>>(a); break;
    case PT_F16:  silu_mul_2d_kernel<st_f16, false><<<blocks, 256, 0, s>>>(a); break;
    case PT_F32:  silu_mul_2d_kernel<st_f32, false><<<blocks, 256, 0, s>>>(a); break;
    default: PT_REQUIRE(false, "silu_mul_fwd_2d: unsupported dtype %d", dtype);
  }
  return check_launch("silu_mul_fwd_2d");
}

extern "C" int pt_silu_mul_bwd_2d(const void* go, int64_t ld_go, const void* gate, int64_t ld_gate, const void* up,
                                  int64_t ld_up, void* dgate, int64_t ld_dgate, void* dup, int64_t ld_dup, int64_t rows,
                                  int64_t cols, int dtype, pt_stream_t stream) {
  if (rows == 0 || cols == 0) return PT_OK;
  PT_REQUIRE(go && gate && up && dgate && dup && ld_go >= cols && ld_gate >= cols && ld_up >= cols && ld_dgate >= cols &&
                 ld_dup >= cols, "silu_mul_bwd_2d: bad arguments");
  const int eb = dtype == PT_F32 ? 4 : 2;
  Silu2dArgs a{};
  if (int rc = silu_2d_setup(a, rows, cols, dtype, "silu_mul_bwd_2d")) return rc;
  a.go = (const char*)go; a.gate = (const char*)gate; a.up = (const char*)up; a.dgate = (char*)dgate; a.dup = (char*)dup;
  a.ld_go = ld_go * eb; a.ld_gate = ld_gate * eb; a.ld_up = ld_up * eb; a.ld_dgate = ld_dgate * eb; a.ld_dup = ld_dup * eb;
  a.vec = cols % 8 == 0 && aligned16(go) && aligned16(gate) && aligned16(up) && aligned16(dgate) && aligned16(dup) &&
          a.ld_go % 16 == 0 && a.ld_gate % 16 == 0 && a.ld_up % 16 == 0 && a.ld_dgate % 16 == 0 && a.ld_dup % 16 == 0;
  hipStream_t s = (hipStream_t)stream;
  const unsigned blocks = (unsigned)cdiv((int64_t)a.total_chunks, 256);
  switch (dtype) {
    case PT_BF16: silu_mul_2d_kernel<st_bf16, true><<<blocks, 256, 0, s>>>(a); break;
    case PT_F16:  silu_mul_2d_kernel<st_f16, true><<<blocks, 256, 0, s>>>(a); break;
    case PT_F32:  silu_mul_2d_kernel<st_f32, true><<<blocks, 256, 0, s>>>(a); break;
    default: PT_REQUIRE(false, "silu_mul_bwd_2d: unsupported dtype %d", dtype);
  }
  return check_launch("silu_mul_bwd_2d");
}

extern "C" int pt_clamped_swiglu_fwd(const void* gate_up, void* out, int64_t n, float alpha, float limit, int dtype,
                                     pt_stream_t stream) {
  if (n == 0) return PT_OK;
  PT_REQUIRE(n > 0 && gate_up && out, "clamped_swiglu_fwd: bad arguments");
  PT_REQUIRE(aligned16(gate_up) && aligned16(out), "clamped_swiglu_fwd: pointers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  PT_DISPATCH_ST(dtype, clamped_swiglu_fwd_kernel, <<<blocks8(n), 256, 0, s>>>((const char*)gate_up, (char*)out, n, alpha, limit));
  return check_launch("clamped_swiglu_fwd");
}

extern "C" int pt_clamped_swiglu_bwd(const void* go, const void* gate_up, void* dgu, int64_t n, float alpha, float limit,
                                     int dtype, pt_stream_t stream) {
  if (n == 0) return PT_OK;
  PT_REQUIRE(n > 0 && go && gate_up && dgu, "clamped_swiglu_bwd: bad arguments");
  PT_REQUIRE(aligned16(go) && aligned16(gate_up) && aligned16(dgu), "clamped_swiglu_bwd: pointers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  PT_DISPATCH_ST(dtype, clamped_swiglu_bwd_kernel,
                 <<<blocks8(n), 256, 0, s>>>((const char*)go, (const char*)gate_up, (char*)dgu, n, alpha, limit));
  return check_launch("clamped_swiglu_bwd");
}

extern "C" int pt_indexed_bias_add_fwd(const void* x, const void* bias, const int64_t* group_ids, void* out, int64_t M,
                                       int64_t H, int dtype, pt_stream_t stream) {
  if (M == 0 || H == 0) return PT_OK;
  PT_REQUIRE(M > 0 && H > 0 && x && bias && group_ids && out, "indexed_bias_add_fwd: bad arguments");
  const int vec = (H % 8 == 0) && aligned16(x) && aligned16(bias) && aligned16(out);
  const int64_t work = vec ? M * (H / 8) : M * H;
  PT_REQUIRE(cdiv(work, 256) < (1ll << 31), "indexed_bias_add_fwd: too many elements");
  hipStream_t s = (hipStream_t)stream;
  PT_DISPATCH_ST(dtype, bias_add_kernel,
                 <<<(unsigned)cdiv(work, 256), 256, 0, s>>>((const char*)x, (const char*)bias, group_ids, (char*)out, M, H, vec));
  return check_launch("indexed_bias_add_fwd");
}

static int segment_sum_impl(const void* x, int64_t x_rows, const int32_t* row_index, const int32_t* offs, int32_t num_groups,
                            void* out, int64_t M, int64_t H, int dtype, int out_dtype, pt_stream_t stream) {
  if (num_groups == 0 || H == 0) return PT_OK;
  PT_REQUIRE(num_groups > 0 && num_groups <= 65535 && H > 0 && M >= 0 && x_rows >= 0 && x && offs && out, "segment_sum: bad arguments");
  const int vec = (H % 8 == 0) && aligned16(x);
  dim3 grid((unsigned)cdiv(H, 128), (unsigned)num_groups);
  hipStream_t s = (hipStream_t)stream;
#define PT_SEG(SI, SO) segment_sum_kernel<SI, SO><<<grid, 256, 0, s>>>((const char*)x, offs, (char*)out, M, H, vec, row_index, x_rows)
  if (dtype == PT_BF16 && out_dtype == PT_BF16) PT_SEG(st_bf16, st_bf16);
  else if (dtype == PT_BF16 && out_dtype == PT_F32) PT_SEG(st_bf16, st_f32);
  else if (dtype == PT_F16 && out_dtype == PT_F16) PT_SEG(st_f16, st_f16);
  else if (dtype == PT_F16 && out_dtype == PT_F32) PT_SEG(st_f16, st_f32);
  else if (dtype == PT_F32 && out_dtype == PT_F32) PT_SEG(st_f32, st_f32);
  else if (dtype == PT_F32 && out_dtype == PT_BF16) PT_SEG(st_f32, st_bf16);
  else PT_REQUIRE(false, "segment_sum: unsupported dtype pair %d -> %d", dtype, out_dtype);
#undef PT_SEG
  return check_launch("segment_sum");
}

extern "C" int pt_segment_sum(const void* x, const int32_t* offs, int32_t num_groups, void* out, int64_t M, int64_t H,
                              int dtype, int out_dtype, pt_stream_t stream) {
  return segment_sum_impl(x, M, nullptr, offs, num_groups, out, M, H, dtype, out_dtype, stream);
}

extern "C" int pt_segment_sum_rows(const void* x, int64_t x_rows, const int32_t* row_index, const int32_t* offs,
                                   int32_t num_groups, void* out, int64_t M, int64_t H, int dtype, int out_dtype,
                                   pt_stream_t stream) {
  PT_REQUIRE(row_index, "segment_sum_rows: null row_index");
  return segment_sum_impl(x, x_rows, row_index, offs, num_groups, out, M, H, dtype, out_dtype, stream);
}
