// In-place fused cross-entropy of the loss head: one pass for the row's softmax statistics, one
// that overwrites the logits with the gradient of the mean loss, as the reference's kernel does
// (operators/cross_entropy.py:16-78):
//
//   n    = max(1, #rows with target != ignore_index)
//   m, d = max_i x_i, sum_i exp(x_i - m)                               (fp32)
//   loss_row = -(x_y - m - log d);  ignored rows: loss_row = 0, gradient row = 0
//   x_i <- S((exp(x_i - m) / d) / n);   x_y <- S(float(x_y) - 1/n)      (S = the logits' type)
//   loss = sum(loss_row) / n
//
// One 1024-thread workgroup per row (vocabularies are 130-200 k entries: 150+ elements per
// thread), 16-byte accesses.  The second read of the row (300-400 KB) comes out of the caches, so
// HBM sees one read and one write of the logits.  exp is the hardware's exp2 of x * log2(e): at
// 1.2 G elements per step a library exp would cost as much as the memory traffic.  The row
// statistics combine per-thread (m, d) pairs in a fixed order: the result is the same on every run.
// Backward (CrossEntropy.backward, operators/cross_entropy.py:120-124): the stored gradient times
// the incoming scalar rounded to S, in place.
#include "common.h"
#include <stdlib.h>
#include <string.h>

// Cache policy of the logits' accesses (1 = non-temporal loads, 2 = non-temporal stores; build
// switch, make EXTRA=-DPT_CE_NT=<bits>): a [N, V] logits matrix is larger than every cache and each
// pass touches an element once.  Both on: the in-place backward runs 10 % faster (4096 x 151 936
// bf16: 478 -> 428 us), the forward is level; either one alone changes nothing.
#ifndef PT_CE_NT
#define PT_CE_NT 3
#endif
#if PT_CE_NT & 1
#define PT_CE_LDS_LOAD_NT " nt"
#else
#define PT_CE_LDS_LOAD_NT ""
#endif

namespace pt {

static constexpr int kCeThreads = 1024;
static constexpr float kLog2e = 1.4426950408889634f;

struct CeArgs {
  char* x;
  int64_t ld;  // bytes
  const int64_t* target;
  int64_t N, V, ignore_index;
  float* loss_rows;
  float* loss;
  int64_t* n_non_ignore;
  const float* grad_output;
  uint32_t chunks;
  int vec;
};

__device__ __forceinline__ float fast_exp(float v) { return __builtin_amdgcn_exp2f(v * kLog2e); }

__global__ __launch_bounds__(1024) void ce_count_kernel(const int64_t* target, int64_t N, int64_t ignore_index,
                                                        int64_t* n_non_ignore) {
  __shared__ int64_t s_part[16];
  int64_t c = 0;
  for (int64_t i = threadIdx.x; i < N; i += 1024) c += target[i] != ignore_index;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) c += __shfl_xor((int)c, d);  // a wave counts at most N / 16 < 2^31 rows
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    int64_t t = 0;
    for (int w = 0; w < 16; ++w) t += s_part[w];
    *n_non_ignore = t < 1 ? 1 : t;
  }
}

// (m, d) of two disjoint parts of a row -> (m, d) of their union
__device__ __forceinline__ void merge_md(float& m, float& d, float m2, float d2) {
  const float mn = fmaxf(m, m2);
  // a part that saw nothing has m = -inf and d = 0: its term is 0 * exp(-inf - mn) = 0
  const float a = m == -INFINITY ? 0.f : d * fast_exp(m - mn);
  const float b = m2 == -INFINITY ? 0.f : d2 * fast_exp(m2 - mn);
  m = mn;
  d = a + b;
}

template <typename S>
__global__ __launch_bounds__(1024) void ce_fwd_kernel(CeArgs p) {
  __shared__ float s_m[16], s_d[16];
  const int64_t row = blockIdx.x;
  char* x = p.x + row * p.ld;
  const int64_t y = p.target[row];
  const int tid = threadIdx.x;
  if (y == p.ignore_index) {
    if (p.vec) {
      const uint4 z = {0, 0, 0, 0};
      for (uint32_t c = tid; c < p.chunks; c += kCeThreads) {
        if (S::kBytes == 4) {
          ((uint4*)x)[2 * c] = z;
          ((uint4*)x)[2 * c + 1] = z;
        } else {
          ((uint4*)x)[c] = z;
        }
      }
    } else {
      for (int64_t i = tid; i < p.V; i += kCeThreads) S::store1(x + i * S::kBytes, 0.f);
    }
    if (tid == 0) p.loss_rows[row] = 0.f;
    return;
  }
  // pass 1: per-thread running (m, d), rescaled once per 8-element chunk
  float m = -INFINITY, d = 0.f;
  if (p.vec) {
    for (uint32_t c = tid; c < p.chunks; c += kCeThreads) {
      float v[8];
      S::load8(x + (int64_t)c * 8 * S::kBytes, v);
      float cm = v[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) cm = fmaxf(cm, v[i]);
      if (cm > m) {
        d = d * fast_exp(m - cm);  // m = -inf on the first chunk: d is 0 and exp2(-inf) is 0
        m = cm;
      }
      if (m != -INFINITY) {  // a chunk of -inf logits (masked vocabulary) adds nothing
        const float mb = m * kLog2e;
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) s += __builtin_amdgcn_exp2f(v[i] * kLog2e - mb);
        d += s;
      }
    }
  } else {
    for (int64_t i = tid; i < p.V; i += kCeThreads) {
      const float v = S::load1(x + i * S::kBytes);
      if (v > m) {
        d = d * fast_exp(m - v);
        m = v;
      }
      if (m != -INFINITY) d += fast_exp(v - m);
    }
  }
  // fixed-order combination: xor butterfly inside the wave, then the 16 waves in order
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) {
    const float m2 = __shfl_xor(m, s), d2 = __shfl_xor(d, s);
    merge_md(m, d, m2, d2);
  }
  if ((tid & 63) == 0) {
    s_m[tid >> 6] = m;
    s_d[tid >> 6] = d;
  }
  __syncthreads();
  m = s_m[0];
  d = s_d[0];
  for (int w = 1; w < 16; ++w) merge_md(m, d, s_m[w], s_d[w]);
  const float n = (float)*p.n_non_ignore;
  const bool y_ok = y >= 0 && y < p.V;
  if (tid == 0) {
    // a target outside the vocabulary (and not the ignore value) has no logit: the loss says so
    const float xy = y_ok ? S::load1(x + y * S::kBytes) : NAN;
    p.loss_rows[row] = -(xy - m - logf(d));
  }
  __syncthreads();  // the target's logit is read before anyone overwrites it
  // pass 2: gradient of the mean loss, in place
  const float mb = m * kLog2e;
  // The two divisions of the reference become multiplications by reciprocals computed once per
  // row: an fp32 division per element costs more issue cycles than everything else in the pass.
  const float inv_d = 1.0f / d, inv_n = 1.0f / n;
  const float neg_inv_n = -1.0f / n;
  if (p.vec) {
    for (uint32_t c = tid; c < p.chunks; c += kCeThreads) {
      float v[8];
      char* q = x + (int64_t)c * 8 * S::kBytes;
      S::load8(q, v);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (__builtin_amdgcn_exp2f(v[i] * kLog2e - mb) * inv_d) * inv_n;
      const int64_t off = y - (int64_t)c * 8;
      if (off >= 0 && off < 8) {
        // the reference stores the softmax term first and corrects the stored value afterwards
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (i == (int)off) v[i] = S::round(v[i]) + neg_inv_n;
      }
      S::store8(q, v);
    }
  } else {
    for (int64_t i = tid; i < p.V; i += kCeThreads) {
      float g = (fast_exp(S::load1(x + i * S::kBytes) - m) * inv_d) * inv_n;
      if (i == y) g = S::round(g) + neg_inv_n;
      S::store1(x + i * S::kBytes, g);
    }
  }
}

// The same computation with the row held on chip between the passes: 16-bit logits, up to
// kCeRegChunks 16-byte chunks per thread in registers and the chunks past those in LDS, so the
// logits cross the memory bus once each way (the generic kernel's second read of a 300 KB row
// mostly misses the caches when 256 rows are in flight).
static constexpr int kCeRegChunks = 15;                                  // 15 x 1024 x 8 = 122 880 elements
static constexpr int kCeLdsChunks = (160 * 1024 - 256) / 16;             // + 81 792 elements in the rest of the 160 KiB of LDS

typedef int ce_v4i __attribute__((ext_vector_type(4)));

template <typename S>
__device__ __forceinline__ void unpack8(const ce_v4i& w, float* v) {
  static_assert(S::kBytes == 2, "16-bit storage only");
  S::load8(&w, v);
}

// 16 bytes per lane from base + voff (per lane) + soff (uniform) into LDS at lds_off + 16 * lane.
__device__ __forceinline__ void ce_load_to_lds(ce_v4i rsrc, uint32_t voff, uint32_t soff, uint32_t lds_off) {
  soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
  lds_off = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_off);
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen" PT_CE_LDS_LOAD_NT " lds" ::"v"(voff), "s"(rsrc), "s"(soff),
               "s"(lds_off)
               : "memory");
}

template <typename S>
__global__ __launch_bounds__(1024) void ce_fwd_onchip_kernel(CeArgs p) {
  extern __shared__ ce_v4i s_over[];
  __shared__ float s_m[16], s_d[16];
  const int64_t row = blockIdx.x;
  char* x = p.x + row * p.ld;
  const int64_t y = p.target[row];
  const int tid = threadIdx.x;
  if (y == p.ignore_index) {
    const uint4 z = {0, 0, 0, 0};
    for (uint32_t c = tid; c < p.chunks; c += kCeThreads) ((uint4*)x)[c] = z;
    if (tid == 0) p.loss_rows[row] = 0.f;
    return;
  }
  // Raw buffer descriptor over the row: a lane's byte offset is tid * 16 for every chunk, the
  // chunk's i * 16 KiB goes into the uniform offset, and accesses past the row's end are dropped by
  // the hardware (loads return 0) instead of needing an address and a predicate per chunk.
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(x, 0, (int)(p.V * S::kBytes), 0x00020000);
  ce_v4i rsrc_words;  // the same descriptor as plain words, for the inline-assembly load
  {
    const uint64_t a = (uint64_t)(uintptr_t)x;
    rsrc_words[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    rsrc_words[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xFFFF));
    rsrc_words[2] = __builtin_amdgcn_readfirstlane((int)(p.V * S::kBytes));
    rsrc_words[3] = 0x00020000;
  }
  const uint32_t voff = (uint32_t)tid * 16u;
  ce_v4i cache[kCeRegChunks];
  float m = -INFINITY, d = 0.f;
  auto absorb = [&](const ce_v4i& w) {
    float v[8];
    unpack8<S>(w, v);
    float cm = v[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) cm = fmaxf(cm, v[i]);
    if (cm > m) {
      d = d * fast_exp(m - cm);
      m = cm;
    }
    if (m != -INFINITY) {
      const float mb = m * kLog2e;
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) s += __builtin_amdgcn_exp2f(v[i] * kLog2e - mb);
      d += s;
    }
    __builtin_amdgcn_sched_barrier(0);  // one chunk's temporaries at a time: the cache owns the registers
  };
  // The chunks past the registers go straight from memory into LDS (direct-to-LDS loads: a wave's
  // 64 lanes fill 1 KiB, lane l the 16 bytes of the chunk thread l of that wave owns), issued first
  // so that they travel while the register part is loaded and absorbed.
  {
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) ce_v4i*)s_over;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#pragma unroll 1
    for (uint32_t c0 = kCeRegChunks * kCeThreads + wave * 64; c0 < p.chunks; c0 += kCeThreads)
      ce_load_to_lds(rsrc_words, (uint32_t)(tid & 63) * 16u, c0 * 16u, lds_base + (c0 - kCeRegChunks * kCeThreads) * 16u);
  }
#pragma unroll
  for (int i = 0; i < kCeRegChunks; ++i) cache[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, i * kCeThreads * 16, (PT_CE_NT & 1) ? 2 : 0);
#pragma unroll
  for (int i = 0; i < kCeRegChunks; ++i)
    if ((uint32_t)i * kCeThreads + tid < p.chunks) absorb(cache[i]);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the LDS part has landed (each thread reads only its own chunks)
#pragma unroll 1
  for (uint32_t c = kCeRegChunks * kCeThreads + tid; c < p.chunks; c += kCeThreads) absorb(s_over[c - kCeRegChunks * kCeThreads]);
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) {
    const float m2 = __shfl_xor(m, s), d2 = __shfl_xor(d, s);
    merge_md(m, d, m2, d2);
  }
  if ((tid & 63) == 0) {
    s_m[tid >> 6] = m;
    s_d[tid >> 6] = d;
  }
  __syncthreads();
  m = s_m[0];
  d = s_d[0];
  for (int w = 1; w < 16; ++w) merge_md(m, d, s_m[w], s_d[w]);
  const float n = (float)*p.n_non_ignore;
  if (tid == 0) {
    const float xy = (y >= 0 && y < p.V) ? S::load1(x + y * S::kBytes) : NAN;
    p.loss_rows[row] = -(xy - m - logf(d));
  }
  __syncthreads();
  const float mb = m * kLog2e;
  // The two divisions of the reference become multiplications by reciprocals computed once per
  // row: an fp32 division per element costs more issue cycles than everything else in the pass.
  const float inv_d = 1.0f / d, inv_n = 1.0f / n;
  const float neg_inv_n = -1.0f / n;
  // gradient of one chunk, packed for a 16-byte store
  auto grad_of = [&](const ce_v4i& w, uint32_t c) {
    float v[8];
    unpack8<S>(w, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (__builtin_amdgcn_exp2f(v[i] * kLog2e - mb) * inv_d) * inv_n;
    const int64_t off = y - (int64_t)c * 8;
    if (off >= 0 && off < 8) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i == (int)off) v[i] = S::round(v[i]) + neg_inv_n;
    }
    ce_v4i out;
    S::store8(&out, v);
    return out;
  };
#pragma unroll
  for (int i = 0; i < kCeRegChunks; ++i) {
    const uint32_t c = (uint32_t)i * kCeThreads + tid;
    // a chunk past the row's end computes on zeros and its store is dropped by the descriptor
    __builtin_amdgcn_raw_buffer_store_b128(grad_of(cache[i], c), rsrc, voff, i * kCeThreads * 16, (PT_CE_NT & 2) ? 2 : 0);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll 1
  for (uint32_t c = kCeRegChunks * kCeThreads + tid; c < p.chunks; c += kCeThreads)
    if (PT_CE_NT & 2) __builtin_nontemporal_store(grad_of(s_over[c - kCeRegChunks * kCeThreads], c), (ce_v4i*)(x + (int64_t)c * 16));
    else *(ce_v4i*)(x + (int64_t)c * 16) = grad_of(s_over[c - kCeRegChunks * kCeThreads], c);
}

__global__ __launch_bounds__(1024) void ce_finish_kernel(const float* loss_rows, int64_t N, const int64_t* n_non_ignore,
                                                         float* loss) {
  __shared__ double s_part[16];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < N; i += 1024) acc += (double)loss_rows[i];
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const int lo = __shfl_xor(__double2loint(acc), d), hi = __shfl_xor(__double2hiint(acc), d);
    acc += __hiloint2double(hi, lo);
  }
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double t = 0.0;
    for (int w = 0; w < 16; ++w) t += s_part[w];
    *loss = (float)t / (float)*n_non_ignore;
  }
}

// Backward: four 16-byte chunks per thread, 4 KiB apart, so a wave's accesses stay contiguous and
// every thread has four loads in flight.
template <typename S>
__global__ __launch_bounds__(256) void ce_scale_kernel(CeArgs p, uint32_t blocks_per_row) {
  const float s = S::round(*p.grad_output);
  if (s == 1.0f) return;  // the stored gradient is already the answer
  const uint32_t row = blockIdx.x / blocks_per_row, rb = blockIdx.x % blocks_per_row;
  char* x = p.x + (int64_t)row * p.ld;
  if (p.vec) {
    const uint32_t c0 = rb * 1024 + threadIdx.x;
    float v[4][8];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (c0 + q * 256 < p.chunks) {
        if (S::kBytes == 2 && (PT_CE_NT & 1)) {
          const ce_v4i w = __builtin_nontemporal_load((const ce_v4i*)(x + (int64_t)(c0 + q * 256) * 16));
          S::load8(&w, v[q]);
        } else {
          S::load8(x + (int64_t)(c0 + q * 256) * 8 * S::kBytes, v[q]);
        }
      }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (c0 + q * 256 < p.chunks) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[q][i] = v[q][i] * s;
        if (S::kBytes == 2 && (PT_CE_NT & 2)) {
          ce_v4i w;
          S::store8(&w, v[q]);
          __builtin_nontemporal_store(w, (ce_v4i*)(x + (int64_t)(c0 + q * 256) * 16));
        } else {
          S::store8(x + (int64_t)(c0 + q * 256) * 8 * S::kBytes, v[q]);
        }
      }
    }
  } else {
    for (int64_t i = (int64_t)rb * 256 + threadIdx.x; i < p.V; i += (int64_t)blocks_per_row * 256)
      S::store1(x + i * S::kBytes, S::load1(x + i * S::kBytes) * s);
  }
}

static int ce_args(CeArgs& a, const char* who, void* logits, int64_t ld, int dtype, int64_t N, int64_t V) {
  PT_REQUIRE(N >= 0 && V >= 1 && N < (1ll << 31) && V < (1ll << 34), "%s: bad sizes", who);
  PT_REQUIRE(ld >= V, "%s: bad leading dimension", who);
  PT_REQUIRE(dtype == PT_BF16 || dtype == PT_F16 || dtype == PT_F32, "%s: unsupported dtype %d", who, dtype);
  const int eb = dtype == PT_F32 ? 4 : 2;
  a.x = (char*)logits; a.ld = ld * eb; a.N = N; a.V = V;
  a.chunks = (uint32_t)cdiv(V, 8);
  a.vec = V % 8 == 0 && ((uintptr_t)logits & 15) == 0 && a.ld % 16 == 0;
  return PT_OK;
}

}  // namespace pt

using namespace pt;

extern "C" int pt_cross_entropy_fwd(void* logits, int64_t ld, int dtype, const int64_t* target, int64_t N, int64_t V,
                                    int64_t ignore_index, float* loss_rows, float* loss, int64_t* n_non_ignore,
                                    pt_stream_t stream) {
  CeArgs a = {};
  if (int rc = ce_args(a, "cross_entropy_fwd", logits, ld, dtype, N, V)) return rc;
  PT_REQUIRE(loss && n_non_ignore && (N == 0 || (logits && target && loss_rows)), "cross_entropy_fwd: null pointer");
  a.target = target; a.ignore_index = ignore_index; a.loss_rows = loss_rows; a.loss = loss; a.n_non_ignore = n_non_ignore;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, s, target, N, ignore_index, n_non_ignore);
  const int64_t over = (int64_t)a.chunks - (int64_t)kCeRegChunks * kCeThreads;
  // PITHTRAIN_CE_KERNEL=twopass keeps the generic kernel for every shape (for measurements)
  static const bool onchip_allowed = [] {
    const char* e = getenv("PITHTRAIN_CE_KERNEL");
    return !(e && strcmp(e, "twopass") == 0);
  }();
  if (N && a.vec && dtype != PT_F32 && over <= kCeLdsChunks && onchip_allowed) {
    const size_t lds = over > 0 ? (size_t)over * 16 : 0;
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once per process
    static const hipError_t allow = [] {
      hipError_t e = hipFuncSetAttribute((const void*)ce_fwd_onchip_kernel<st_bf16>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kCeLdsChunks * 16);
      if (e != hipSuccess) return e;
      return hipFuncSetAttribute((const void*)ce_fwd_onchip_kernel<st_f16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                 kCeLdsChunks * 16);
    }();
    PT_REQUIRE(allow == hipSuccess, "cross_entropy_fwd: hipFuncSetAttribute failed: %s", hipGetErrorString(allow));
    if (dtype == PT_BF16) hipLaunchKernelGGL(ce_fwd_onchip_kernel<st_bf16>, dim3((unsigned)N), dim3(kCeThreads), lds, s, a);
    else hipLaunchKernelGGL(ce_fwd_onchip_kernel<st_f16>, dim3((unsigned)N), dim3(kCeThreads), lds, s, a);
  } else if (N) {
    switch (dtype) {
      case PT_BF16: hipLaunchKernelGGL(ce_fwd_kernel<st_bf16>, dim3((unsigned)N), dim3(kCeThreads), 0, s, a); break;
      case PT_F16: hipLaunchKernelGGL(ce_fwd_kernel<st_f16>, dim3((unsigned)N), dim3(kCeThreads), 0, s, a); break;
      default: hipLaunchKernelGGL(ce_fwd_kernel<st_f32>, dim3((unsigned)N), dim3(kCeThreads), 0, s, a); break;
    }
  }
  hipLaunchKernelGGL(ce_finish_kernel, dim3(1), dim3(1024), 0, s, loss_rows, N, n_non_ignore, loss);
  return check_launch("ce_fwd_kernel");
}

extern "C" int pt_cross_entropy_bwd(void* grad, int64_t ld, int dtype, int64_t N, int64_t V, const float* grad_output,
                                    pt_stream_t stream) {
  CeArgs a = {};
  if (int rc = ce_args(a, "cross_entropy_bwd", grad, ld, dtype, N, V)) return rc;
  if (N == 0) return PT_OK;
  PT_REQUIRE(grad && grad_output, "cross_entropy_bwd: null pointer");
  a.grad_output = grad_output;
  const int64_t bx = a.vec ? cdiv(a.chunks, 1024) : (cdiv(V, 256) < 1024 ? cdiv(V, 256) : 1024);
  PT_REQUIRE(N * bx < (1ll << 31), "cross_entropy_bwd: too many rows for one launch");
  const dim3 grid((unsigned)(N * bx));
  switch (dtype) {
    case PT_BF16: hipLaunchKernelGGL(ce_scale_kernel<st_bf16>, grid, dim3(256), 0, (hipStream_t)stream, a, (uint32_t)bx); break;
    case PT_F16: hipLaunchKernelGGL(ce_scale_kernel<st_f16>, grid, dim3(256), 0, (hipStream_t)stream, a, (uint32_t)bx); break;
    default: hipLaunchKernelGGL(ce_scale_kernel<st_f32>, grid, dim3(256), 0, (hipStream_t)stream, a, (uint32_t)bx); break;
  }
  return check_launch("ce_scale_kernel");
}
