// Routing-driven permute / unpermute and expert-parallel dedup index construction (gfx950).
//
// Ordering is made deterministic with a stable counting sort: every wavefront owns a contiguous
// chunk of keys, (1) counts them into a private LDS histogram, (2) one workgroup turns the
// [chunk][group] counts into exclusive bases, (3) every wavefront replays its chunk 64 keys at a
// time, ranking equal keys inside the wave with ballot masks (one ballot per key bit) on top of
// its running LDS counters.  No global atomics decide a position, so the result is the
// ascending-source-row order inside every group on every run.
//
// Row movement is a separate pass over the *destination* rows (one wavefront per row, 16-byte
// accesses) so that padding rows are zeroed and data rows copied in one coalesced sweep.
#include "common.h"
#include <mutex>

// Cache policy of the row movers (build switch, make EXTRA=-DPT_PERMUTE_NT=<bits>): 1 = non-temporal
// loads of source rows, 2 = non-temporal stores of destination rows.  Source rows are read once
// (or a few times, close together, by the expanding gather) and the results are the next
// operator's input, so only the loads are non-temporal: 65 536 rows x 4 KiB, timed alone,
// permute 112 -> 104 us, gather 105 -> 80 us, gather backward 133 -> 121 us.
#ifndef PT_PERMUTE_NT
#define PT_PERMUTE_NT 1
#endif

namespace pt {

static constexpr int kWaveKeys = 256;    // keys per wavefront chunk (4 steps of 64)
static constexpr int kMaxGroups = 2048;  // LDS: 4 waves x 2048 x 4 B = 32 KiB

__device__ __forceinline__ uint64_t lanemask_lt() {
  const int lane = threadIdx.x & 63;
  return lane == 0 ? 0ull : (~0ull >> (64 - lane));
}

// lanes (among `active`) whose key equals this lane's key
__device__ __forceinline__ uint64_t wave_match(uint32_t key, bool active, int nbits) {
  uint64_t m = __ballot(active);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (key >> b) & 1u;
    const uint64_t bal = __ballot(active && bit);
    m &= bit ? bal : ~bal;
  }
  return m;
}

static inline int bits_for(int n) { int b = 0; while ((1 << b) < n) ++b; return b < 1 ? 1 : b; }

// ---------------------------------------------------------------------------------------------
// group_rows: counts -> bases -> ranks
// ---------------------------------------------------------------------------------------------
// Also marks every entry of src_of as "no row" (the rank kernel, three launches later, overwrites
// the entries that name one).
__global__ __launch_bounds__(256) void gr_hist_kernel(const int64_t* keys, int64_t m, int G, int32_t* counts /*[W][G]*/,
                                                      int32_t* src_of, int64_t cap) {
  extern __shared__ int32_t s_hist[];  // [4][G]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < cap; i += (int64_t)gridDim.x * 256) src_of[i] = -1;
  int32_t* h = s_hist + wave * G;
  for (int g = lane; g < G; g += 64) h[g] = 0;
  __builtin_amdgcn_wave_barrier();
  const int64_t w = (int64_t)blockIdx.x * 4 + wave;
  const int64_t base = w * kWaveKeys;
  for (int s = 0; s < kWaveKeys; s += 64) {
    const int64_t i = base + s + lane;
    if (i < m) {
      const int64_t k = keys[i];
      if (k >= 0 && k < G) atomicAdd(&h[k], 1);
    }
  }
  __builtin_amdgcn_wave_barrier();
  if (base < m)
    for (int g = lane; g < G; g += 64) counts[w * G + g] = h[g];
}

// counts[W][G] -> exclusive bases over the chunks in place, one wavefront per group (64 chunks per
// step, ranked with a wave prefix sum); the group's total goes to totals[g].
__global__ __launch_bounds__(256) void gr_scan_chunks_kernel(int32_t* counts, int64_t W, int G, int32_t* totals) {
  const int lane = threadIdx.x & 63;
  const int g = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= G) return;
  int32_t run = 0;
  for (int64_t w0 = 0; w0 < W; w0 += 64) {
    const int64_t w = w0 + lane;
    const int32_t c = w < W ? counts[w * G + g] : 0;
    int32_t incl = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (w < W) counts[w * G + g] = run + incl - c;
    run += __shfl(incl, 63);
  }
  if (lane == 0) totals[g] = run;
}

// one workgroup: per-group totals (read from group_start) -> padded sizes, inclusive offsets, starts
__global__ __launch_bounds__(1024) void gr_scan_groups_kernel(int G, int alignment, int32_t* offs, int32_t* ks,
                                                              int32_t* group_start /*[G]: totals in, starts out*/) {
  __shared__ int32_t s_part[1024];
  const int t = threadIdx.x;
  // thread t owns groups 2t and 2t+1 (G <= 2048)
  int32_t p0 = 0, p1 = 0;
  if (2 * t < G) p0 = (int32_t)(((int64_t)group_start[2 * t] + alignment - 1) / alignment * alignment);
  if (2 * t + 1 < G) p1 = (int32_t)(((int64_t)group_start[2 * t + 1] + alignment - 1) / alignment * alignment);
  s_part[t] = p0 + p1;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int32_t add = t >= d ? s_part[t - d] : 0;
    __syncthreads();
    s_part[t] += add;
    __syncthreads();
  }
  const int32_t excl = s_part[t] - (p0 + p1);
  if (2 * t < G) {
    group_start[2 * t] = excl;
    offs[2 * t] = excl + p0;
    ks[2 * t] = p0;
  }
  if (2 * t + 1 < G) {
    group_start[2 * t + 1] = excl + p0;
    offs[2 * t + 1] = excl + p0 + p1;
    ks[2 * t + 1] = p1;
  }
}

__global__ __launch_bounds__(256) void gr_rank_kernel(const int64_t* keys, int64_t m, int G, int nbits,
                                                      const int32_t* bases /*[W][G]*/, const int32_t* group_start,
                                                      int64_t* reverse, int32_t* src_of, int64_t cap) {
  extern __shared__ int32_t s_run[];  // [4][G]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int32_t* run = s_run + wave * G;
  const int64_t w = (int64_t)blockIdx.x * 4 + wave;
  const int64_t base = w * kWaveKeys;
  if (base >= m) return;
  for (int g = lane; g < G; g += 64) run[g] = bases[w * G + g] + group_start[g];
  __builtin_amdgcn_wave_barrier();
  const uint64_t lt = lanemask_lt();
  for (int s = 0; s < kWaveKeys; s += 64) {
    const int64_t i = base + s + lane;
    int64_t k = (i < m) ? keys[i] : 0;
    const bool active = (i < m) && k >= 0 && k < G;
    if (!active) k = 0;
    const uint64_t mask = wave_match((uint32_t)k, active, nbits);
    const int rank = __popcll(mask & lt);
    const int32_t b = run[k];
    __builtin_amdgcn_wave_barrier();
    if (active && rank == 0) run[k] = b + __popcll(mask);
    __builtin_amdgcn_wave_barrier();
    if (active) {
      const int64_t pos = (int64_t)b + rank;
      reverse[i] = pos;
      if (pos < cap) src_of[pos] = (int32_t)i;
    } else if (i < m) {
      // a key outside [0, G) belongs to no group: the row is dropped (no src_of entry names it) and
      // its reverse entry is a valid row, so that a later gather through it stays in bounds
      reverse[i] = 0;
    }
  }
}

__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// ---------------------------------------------------------------------------------------------
// row movement: one wavefront per destination row
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ nt_u4 row_ld(const nt_u4* p) { return (PT_PERMUTE_NT & 1) ? __builtin_nontemporal_load(p) : *p; }
__device__ __forceinline__ void row_st(nt_u4* p, nt_u4 v) {
  if (PT_PERMUTE_NT & 2) __builtin_nontemporal_store(v, p);
  else *p = v;
}
template <bool VEC>
__device__ __forceinline__ void copy_row(const char* src, char* dst, int64_t row_bytes, int lane) {
  if (VEC) {
    const int64_t chunks = row_bytes >> 4;
    int64_t c = lane;
    for (; c + 192 < chunks; c += 256) {  // four 16-byte loads in flight per lane
      const nt_u4 a0 = row_ld((const nt_u4*)src + c), a1 = row_ld((const nt_u4*)src + c + 64);
      const nt_u4 a2 = row_ld((const nt_u4*)src + c + 128), a3 = row_ld((const nt_u4*)src + c + 192);
      row_st((nt_u4*)dst + c, a0); row_st((nt_u4*)dst + c + 64, a1); row_st((nt_u4*)dst + c + 128, a2); row_st((nt_u4*)dst + c + 192, a3);
    }
    for (; c < chunks; c += 64) row_st((nt_u4*)dst + c, row_ld((const nt_u4*)src + c));
  } else {
    for (int64_t b = lane; b < row_bytes; b += 64) dst[b] = src[b];
  }
}
template <bool VEC>
__device__ __forceinline__ void zero_row(char* dst, int64_t row_bytes, int lane) {
  if (VEC) {
    const int64_t chunks = row_bytes >> 4;
    for (int64_t c = lane; c < chunks; c += 64) ((uint4*)dst)[c] = make_uint4(0, 0, 0, 0);
  } else {
    for (int64_t b = lane; b < row_bytes; b += 64) dst[b] = 0;
  }
}

template <bool VEC>
__global__ __launch_bounds__(256) void permute_rows_kernel(const char* in, int64_t ld_in_b, char* out, int64_t ld_out_b,
                                                           const int32_t* src_of, const int64_t* pre,
                                                           const int32_t* offs_last, int tail_alignment, int64_t cap,
                                                           int64_t row_bytes) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  int64_t rows_out = cap;
  if (offs_last) {
    const int64_t last = offs_last[0];
    const int64_t rounded = (last + tail_alignment - 1) / tail_alignment * tail_alignment;
    rows_out = rounded < cap ? rounded : cap;
  }
  if (r >= rows_out) return;
  int64_t s = src_of[r];
  char* dst = out + r * ld_out_b;
  if (s < 0) {
    zero_row<VEC>(dst, row_bytes, lane);
  } else {
    if (pre) s = pre[s];
    copy_row<VEC>(in + s * ld_in_b, dst, row_bytes, lane);
  }
}

template <bool VEC>
__global__ __launch_bounds__(256) void gather_rows_kernel(const char* in, int64_t ld_in_b, char* out, int64_t ld_out_b,
                                                          const int64_t* index, int64_t n, int64_t row_bytes) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= n) return;
  copy_row<VEC>(in + index[r] * ld_in_b, out + r * ld_out_b, row_bytes, lane);
}

// ---------------------------------------------------------------------------------------------
// gather backward: deterministic segmented sum (CSR of the index, entries sorted ascending)
// ---------------------------------------------------------------------------------------------
__global__ void gb_count_kernel(const int64_t* index, int64_t n, int64_t rows, int32_t* cnt) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j < n) {
    const int64_t r = index[j];
    if (r >= 0 && r < rows) atomicAdd(&cnt[r], 1);
  }
}

// three-kernel exclusive scan over int32 (1024 elements per workgroup)
__device__ __forceinline__ int32_t block_excl_scan_1024(int32_t v, int32_t* s_w /*[16]*/, int32_t& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int32_t x = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int32_t y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  if (lane == 63) s_w[wave] = x;
  __syncthreads();
  int32_t woff = 0, tot = 0;
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int32_t t = s_w[q];
    if (q < wave) woff += t;
    tot += t;
  }
  __syncthreads();
  total = tot;
  return woff + x - v;
}
__global__ __launch_bounds__(1024) void scan_block_sums_kernel(const int32_t* in, int64_t n, int32_t* block_sums) {
  __shared__ int32_t s_w[16];
  const int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  int32_t tot;
  block_excl_scan_1024(i < n ? in[i] : 0, s_w, tot);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = tot;
}
__global__ __launch_bounds__(1024) void scan_top_kernel(int32_t* block_sums, int64_t nb) {
  __shared__ int32_t s_w[16];
  int32_t carry = 0;
  for (int64_t b0 = 0; b0 < nb; b0 += 1024) {
    const int64_t i = b0 + threadIdx.x;
    int32_t tot;
    const int32_t e = block_excl_scan_1024(i < nb ? block_sums[i] : 0, s_w, tot);
    if (i < nb) block_sums[i] = e + carry;
    carry += tot;
  }
}
__global__ __launch_bounds__(1024) void scan_apply_kernel(const int32_t* in, int64_t n, const int32_t* block_sums,
                                                          int32_t* out /*[n+1]*/) {
  __shared__ int32_t s_w[16];
  const int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  int32_t tot;
  const int32_t v = i < n ? in[i] : 0;
  const int32_t e = block_excl_scan_1024(v, s_w, tot) + block_sums[blockIdx.x];
  if (i < n) out[i] = e;
  if (i == n - 1) out[n] = e + v;
}

__global__ void gb_fill_kernel(const int64_t* index, int64_t n, int64_t rows, const int32_t* seg_start, int32_t* cursor,
                               int32_t* list) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j < n) {
    const int64_t r = index[j];
    if (r >= 0 && r < rows) list[seg_start[r] + atomicAdd(&cursor[r], 1)] = (int32_t)j;
  }
}

// one wavefront per destination row; each lane owns 8-element chunks lane, lane+64, ...
template <typename S, bool VEC>
__global__ __launch_bounds__(256) void gb_sum_kernel(const char* go, int64_t ld_go_b, char* gi, int64_t ld_gi_b,
                                                     const int32_t* seg_start, int32_t* list, int64_t rows, int64_t H) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int32_t s0 = seg_start[r], cnt = seg_start[r + 1] - s0;
  // The segment was filled by atomics; sum it in ascending source order.  Up to 64 entries are
  // rank-sorted in registers, longer ones by a lane-0 insertion sort in place.
  int32_t mine = 0x7FFFFFFF;
  int rank = -1;
  if (cnt <= 64) {
    if (lane < cnt) mine = list[s0 + lane];
    rank = 0;
    for (int q = 0; q < cnt; ++q) rank += (__shfl(mine, q) < mine) ? 1 : 0;
    if (lane >= cnt) rank = -1;
  } else {
    if (lane == 0) {
      for (int a = 1; a < cnt; ++a) {
        const int32_t v = list[s0 + a];
        int b = a - 1;
        while (b >= 0 && list[s0 + b] > v) { list[s0 + b + 1] = list[s0 + b]; --b; }
        list[s0 + b + 1] = v;
      }
    }
    __threadfence();
    __builtin_amdgcn_wave_barrier();
  }
  char* dst = gi + r * ld_gi_b;
  auto source = [&](int q) -> int64_t {
    if (cnt <= 64) {
      const uint64_t b = __ballot(rank == q);
      return __shfl(mine, __ffsll((unsigned long long)b) - 1);
    }
    return ((volatile int32_t*)list)[s0 + q];
  };
  if (VEC) {
    // Four 16-byte chunks per lane and source row in flight (2048 elements of a row per pass): with
    // one, a wave waits a full memory latency per source row.  The additions keep their order:
    // sources ascending, one accumulator per element.
    for (int64_t h0 = (int64_t)lane * 8; h0 < H; h0 += 2048) {
      float acc[4][8];
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[u][e] = 0.f;
      for (int q = 0; q < cnt; ++q) {
        const char* src = go + source(q) * ld_go_b;
        // (a chunk past the end of the row reads the lane's first chunk again and is not added:
        // no branch around a load, which would make the wave wait for one before asking for the next)
        float v[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          load8_policy<S, (PT_PERMUTE_NT & 1) != 0>(src + (h0 + u * 512 < H ? h0 + u * 512 : h0) * S::kBytes, v[u]);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[u][e] = h0 + u * 512 < H ? acc[u][e] + v[u][e] : acc[u][e];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (h0 + u * 512 < H) S::store8(dst + (h0 + u * 512) * S::kBytes, acc[u]);
    }
  } else {
    for (int64_t h0 = (int64_t)lane * 8; h0 < H; h0 += 512) {
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int q = 0; q < cnt; ++q) {
        const char* src = go + source(q) * ld_go_b;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (h0 + e < H) acc[e] += S::load1(src + (h0 + e) * S::kBytes);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (h0 + e < H) S::store1(dst + (h0 + e) * S::kBytes, acc[e]);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// group indices
// ---------------------------------------------------------------------------------------------
template <typename O>
__global__ void group_indices_kernel(const int32_t* offs, int G, int64_t M, O* out) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= M) return;
  int lo = 0, hi = G;  // first g with offs[g] > r
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)offs[mid] <= r) lo = mid + 1; else hi = mid;
  }
  out[r] = (O)(lo < G - 1 ? lo : G - 1);
}

// ---------------------------------------------------------------------------------------------
// dedup dispatch
// ---------------------------------------------------------------------------------------------
static constexpr int kWaveTokens = 64;  // tokens per wave of the dedup kernels (one step of 64 lanes)
static constexpr int kMaxExperts = 1024;

__device__ __forceinline__ int64_t topk_at(const int64_t* ids, int64_t ld, int k, int64_t flat) {
  const int64_t t = flat / k;
  return ids[t * ld + (flat - t * k)];
}

__global__ __launch_bounds__(256) void dd_hist_kernel(const int64_t* ids, int64_t ld, int64_t m, int k, int E, int ep,
                                                      int epr, int32_t* cnt_e /*[W][E]*/, int32_t* cnt_g /*[W][ep]*/) {
  extern __shared__ int32_t s_h[];  // [4][E + 32]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int32_t* he = s_h + wave * (E + 32);
  int32_t* hg = he + E;
  for (int e = lane; e < E + 32; e += 64) he[e] = 0;
  __builtin_amdgcn_wave_barrier();
  const int64_t w = (int64_t)blockIdx.x * 4 + wave;
  const int64_t t0 = w * kWaveTokens;
  for (int s = 0; s < kWaveTokens; s += 64) {
    const int64_t t = t0 + s + lane;
    if (t < m) {
      uint32_t visited = 0;
      for (int j = 0; j < k; ++j) {
        const int64_t e = ids[t * ld + j];
        if (e >= 0 && e < E) {
          atomicAdd(&he[e], 1);
          const uint32_t bit = 1u << (uint32_t)(e / epr);
          if (!(visited & bit)) atomicAdd(&hg[e / epr], 1);
          visited |= bit;
        }
      }
    }
  }
  __builtin_amdgcn_wave_barrier();
  if (t0 < m) {
    for (int e = lane; e < E; e += 64) cnt_e[w * E + e] = he[e];
    for (int g = lane; g < ep; g += 64) cnt_g[w * ep + g] = hg[g];
  }
}

// Exclusive scan down one column of the per-wave count tables (column c < E: expert c, else EP rank
// c - E), one wave per column, 64 chunks per step; the column total goes to totals[c].
__global__ __launch_bounds__(256) void dd_scan_cols_kernel(int32_t* cnt_e, int32_t* cnt_g, int64_t W, int E, int ep,
                                                           int32_t* totals /*[E + ep]*/) {
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= E + ep) return;
  int32_t* col = c < E ? cnt_e + c : cnt_g + (c - E);
  const int64_t stride = c < E ? E : ep;
  int32_t run = 0;
  for (int64_t w0 = 0; w0 < W; w0 += 64) {
    const int64_t w = w0 + lane;
    const int32_t v = w < W ? col[w * stride] : 0;
    int32_t incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t y = __shfl_up(incl, d);
      if (lane >= d) incl += y;
    }
    if (w < W) col[w * stride] = run + incl - v;
    run += __shfl(incl, 63);
  }
  if (lane == 0) totals[c] = run;
}

// Starts of the experts and of the EP ranks from the column totals, and the per-rank metadata.
__global__ __launch_bounds__(64) void dd_scan_totals_kernel(const int32_t* totals, int E, int ep, int epr,
                                                            int64_t* tokens_per_ep_rank, int64_t* dedup_tokens_per_gpu,
                                                            int64_t* send_meta, int32_t* expert_starts, int32_t* gpu_starts) {
  const int lane = threadIdx.x;  // one wave
  // exclusive scan over the experts, 64 at a time
  int32_t run = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const int32_t c = e < E ? totals[e] : 0;
    int32_t incl = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t y = __shfl_up(incl, d);
      if (lane >= d) incl += y;
    }
    if (e < E) {
      expert_starts[e] = run + incl - c;
      send_meta[(e / epr) * (epr + 1) + (e % epr)] = c;
    }
    run += __shfl(incl, 63);
  }
  // per EP rank: rows routed to it, unique tokens sent to it, start of its slice of the dispatch list
  const int g = lane;
  int32_t sg = 0;
  int64_t rank_total = 0;
  if (g < ep) {
    sg = totals[E + g];
    for (int e = 0; e < epr; ++e) rank_total += totals[g * epr + e];
  }
  int32_t incl = sg;
#pragma unroll
  for (int d = 1; d < 32; d <<= 1) {
    const int32_t y = __shfl_up(incl, d);
    if (lane >= d) incl += y;
  }
  if (g < ep) {
    tokens_per_ep_rank[g] = rank_total;
    dedup_tokens_per_gpu[g] = sg;
    gpu_starts[g] = incl - sg;
    send_meta[g * (epr + 1) + epr] = sg;
  }
}

__global__ __launch_bounds__(256) void dd_rank_kernel(const int64_t* ids, int64_t ld, int64_t m, int k, int E, int ep,
                                                      int epr, int nbits, const int32_t* base_e, const int32_t* base_g,
                                                      const int32_t* expert_starts, const int32_t* gpu_starts,
                                                      int64_t* dispatch, int64_t* idxs, int64_t* expand_idx) {
  extern __shared__ int32_t s_r[];  // per wave: run_e[E], run_g[32], lp[64][ep]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int per_wave = E + 32 + 64 * ep;
  int32_t* run_e = s_r + wave * per_wave;
  int32_t* run_g = run_e + E;
  int32_t* lp = run_g + 32;
  const int64_t w = (int64_t)blockIdx.x * 4 + wave;
  const int64_t t0 = w * kWaveTokens;
  if (t0 >= m) return;
  for (int e = lane; e < E; e += 64) run_e[e] = base_e[w * E + e] + expert_starts[e];
  for (int g = lane; g < ep; g += 64) run_g[g] = base_g[w * ep + g];
  __builtin_amdgcn_wave_barrier();
  const uint64_t lt = lanemask_lt();
  for (int s = 0; s < kWaveTokens; s += 64) {
    const int64_t tb = t0 + s;  // first token of this step
    if (tb >= m) break;
    // ---- phase A: first-visit dedup positions of 64 tokens ----
    const int64_t t = tb + lane;
    uint32_t visited = 0;
    if (t < m)
      for (int j = 0; j < k; ++j) {
        const int64_t e = ids[t * ld + j];
        if (e >= 0 && e < E) visited |= 1u << (uint32_t)(e / epr);
      }
    for (int g = 0; g < ep; ++g) {
      const bool v = (visited >> g) & 1u;
      const uint64_t bal = __ballot(v);
      const int32_t b = run_g[g];
      __builtin_amdgcn_wave_barrier();
      if (v) {
        const int32_t pos = b + __popcll(bal & lt);
        lp[lane * ep + g] = pos;
        dispatch[(int64_t)gpu_starts[g] + pos] = t;
      }
      if (lane == 0) run_g[g] = b + __popcll(bal);
      __builtin_amdgcn_wave_barrier();
    }
    // ---- phase B: stable counting sort of the 64*k flat entries of these tokens ----
    const int64_t ntok = (m - tb) < 64 ? (m - tb) : 64;
    const int64_t nflat = ntok * k;
    for (int64_t q = 0; q < nflat; q += 64) {
      const int64_t fl = q + lane;  // flat index local to this step
      const bool in = fl < nflat;
      const int64_t f = tb * k + fl;
      int64_t e = in ? topk_at(ids, ld, k, f) : 0;
      const bool active = in && e >= 0 && e < E;
      if (!active) e = 0;
      const uint64_t mask = wave_match((uint32_t)e, active, nbits);
      const int rank = __popcll(mask & lt);
      const int32_t b = run_e[e];
      __builtin_amdgcn_wave_barrier();
      if (active && rank == 0) run_e[e] = b + __popcll(mask);
      __builtin_amdgcn_wave_barrier();
      if (active) {
        const int64_t pos = (int64_t)b + rank;
        idxs[pos] = f;
        expand_idx[pos] = lp[(int)(fl / k) * ep + (int)(e / epr)];
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

__global__ __launch_bounds__(256) void build_expert_idxs_kernel(const int64_t* counts, int E, int ep, int epr,
                                                                int64_t max_total, int64_t* expert_idxs,
                                                                int64_t* output_splits) {
  __shared__ int64_t s_end[kMaxExperts];  // inclusive cumsum
  if (threadIdx.x == 0) {
    int64_t run = 0;
    for (int e = 0; e < E; ++e) { run += counts[e]; s_end[e] = run; }
  }
  __syncthreads();
  if (blockIdx.x == 0)
    for (int g = threadIdx.x; g < ep; g += blockDim.x)
      output_splits[g] = s_end[(g + 1) * epr - 1] - (g == 0 ? 0 : s_end[g * epr - 1]);
  const int64_t total = s_end[E - 1];
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total || i >= max_total) return;
  int lo = 0, hi = E;  // first e with s_end[e] > i
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (s_end[mid] <= i) lo = mid + 1; else hi = mid;
  }
  expert_idxs[i] = lo % epr;
}

__global__ __launch_bounds__(256) void adjust_expand_idx_kernel(const int64_t* received, int64_t* out, const int64_t* dedup,
                                                                int64_t dedup_stride, const int64_t* splits, int ep,
                                                                int64_t n) {
  __shared__ int64_t s_bound[33], s_start[33];
  if (threadIdx.x == 0) {
    int64_t b = 0, d = 0;
    for (int g = 0; g < ep; ++g) {
      s_bound[g] = b; s_start[g] = d;
      b += splits[g]; d += dedup[g * dedup_stride];
    }
    s_bound[ep] = b;
  }
  __syncthreads();
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int64_t off = 0;
  for (int g = 0; g < ep; ++g)
    if (i >= s_bound[g] && i < s_bound[g + 1]) off = s_start[g];
  out[i] = received[i] + off;
}

static inline int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

}  // namespace pt

using namespace pt;

// ------------------------------------------------------------------------------------------------
extern "C" int64_t pt_group_rows_workspace_bytes(int64_t m, int32_t num_groups) {
  const int64_t W = cdiv(m > 0 ? m : 1, kWaveKeys);
  return align_up(W * num_groups * 4, 256) + align_up((int64_t)num_groups * 4, 256);
}

// The four launches of the stable counting sort (chunk histograms, scan over the chunks, scan over
// the groups, ranks); `workspace` holds the [W][G] chunk counts and the G group starts
// (pt_group_rows_workspace_bytes), every byte of which is written before it is read.  (One kernel
// for both scans, with the last workgroup to finish doing the second, measured slower: the
// device-scope fences it needs write back and invalidate the XCD's L2, 8 us against a 4 us launch.)
static int group_rows_launch(const int64_t* keys, int64_t m, int32_t G, int32_t alignment, int32_t* offs, int32_t* ks,
                             int64_t* reverse, int32_t* src_of, int64_t cap, void* workspace, hipStream_t s) {
  const int64_t W = cdiv(m, kWaveKeys);
  int32_t* counts = (int32_t*)workspace;
  int32_t* group_start = (int32_t*)((char*)workspace + align_up(W * G * 4, 256));
  const unsigned blocks = (unsigned)cdiv(W, 4);
  const size_t lds = (size_t)4 * G * sizeof(int32_t);
  gr_hist_kernel<<<blocks, 256, lds, s>>>(keys, m, G, counts, src_of, cap);
  gr_scan_chunks_kernel<<<(unsigned)cdiv(G, 4), 256, 0, s>>>(counts, W, G, group_start);
  gr_scan_groups_kernel<<<1, 1024, 0, s>>>(G, alignment, offs, ks, group_start);
  gr_rank_kernel<<<blocks, 256, lds, s>>>(keys, m, G, bits_for(G), counts, group_start, reverse, src_of, cap);
  return check_launch("group_rows");
}

static int group_rows_check(const int64_t* keys, int64_t m, int32_t G, int32_t alignment, const int32_t* offs, const int32_t* ks,
                            const int64_t* reverse, const int32_t* src_of, int64_t cap) {
  PT_REQUIRE(m > 0 && G > 0 && G <= kMaxGroups && alignment > 0, "group_rows: m=%lld G=%d (max %d)", (long long)m, G, kMaxGroups);
  PT_REQUIRE(m + (int64_t)G * (alignment - 1) < (1ll << 31), "group_rows: row count exceeds int32");
  PT_REQUIRE(keys && offs && ks && reverse && src_of, "group_rows: null pointer");
  PT_REQUIRE(cap >= m, "group_rows: cap < m");
  return PT_OK;
}

extern "C" int pt_group_rows(const int64_t* keys, int64_t m, int32_t G, int32_t alignment, int32_t* offs, int32_t* ks,
                             int64_t* reverse, int32_t* src_of, int64_t cap, void* workspace, int64_t workspace_bytes,
                             pt_stream_t stream) {
  if (int rc = group_rows_check(keys, m, G, alignment, offs, ks, reverse, src_of, cap)) return rc;
  PT_REQUIRE(workspace, "group_rows: null pointer");
  PT_REQUIRE(workspace_bytes >= pt_group_rows_workspace_bytes(m, G), "group_rows: workspace too small");
  return group_rows_launch(keys, m, G, alignment, offs, ks, reverse, src_of, cap, workspace, (hipStream_t)stream);
}

// ---- the same sort for callers that cannot allocate: its workspace is a device array that is
// part of the loaded code object (one copy per GPU, held until the process ends).  The array's
// name is only a host-side handle; the address the kernels get is looked up once per device. ----
static constexpr int64_t kStaticScratchBytes = PT_GROUP_ROWS_STATIC_MAX_WORKSPACE;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on device d, null until looked up

static int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("group_rows_static: no current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
    return PT_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      set_error("group_rows_static: cannot find the scratch array on device %d: %s", dev, hipGetErrorString(e));
      return PT_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return PT_OK;
}

extern "C" int pt_group_rows_static(const int64_t* keys, int64_t m, int32_t G, int32_t alignment, int32_t* offs, int32_t* ks,
                                    int64_t* reverse, int32_t* src_of, int64_t cap, pt_stream_t stream) {
  if (int rc = group_rows_check(keys, m, G, alignment, offs, ks, reverse, src_of, cap)) return rc;
  const int64_t need = pt_group_rows_workspace_bytes(m, G);
  PT_REQUIRE(need <= kStaticScratchBytes,
             "group_rows_static: m=%lld keys in %d groups need %lld bytes of scratch, the built-in array holds %lld "
             "(use pt_group_rows with a workspace)",
             (long long)m, G, (long long)need, (long long)kStaticScratchBytes);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  return group_rows_launch(keys, m, G, alignment, offs, ks, reverse, src_of, cap, ws, (hipStream_t)stream);
}

extern "C" int pt_permute_rows(const void* in, int64_t ld_in, void* out, int64_t ld_out, const int32_t* src_of,
                               const int64_t* pre, const int32_t* offs_last, int32_t tail_alignment, int64_t cap, int64_t H,
                               int32_t elem_bytes, pt_stream_t stream) {
  if (cap == 0 || H == 0) return PT_OK;
  PT_REQUIRE(cap > 0 && H > 0 && in && out && src_of && elem_bytes > 0 && tail_alignment > 0, "permute_rows: bad arguments");
  const int64_t rb = H * elem_bytes, lib = ld_in * elem_bytes, lob = ld_out * elem_bytes;
  const bool vec = (rb % 16 == 0) && (lib % 16 == 0) && (lob % 16 == 0) && ((uintptr_t)in % 16 == 0) && ((uintptr_t)out % 16 == 0);
  const unsigned blocks = (unsigned)cdiv(cap, 4);
  hipStream_t s = (hipStream_t)stream;
  if (vec) permute_rows_kernel<true><<<blocks, 256, 0, s>>>((const char*)in, lib, (char*)out, lob, src_of, pre, offs_last, tail_alignment, cap, rb);
  else     permute_rows_kernel<false><<<blocks, 256, 0, s>>>((const char*)in, lib, (char*)out, lob, src_of, pre, offs_last, tail_alignment, cap, rb);
  return check_launch("permute_rows");
}

extern "C" int pt_gather_rows(const void* in, int64_t ld_in, void* out, int64_t ld_out, const int64_t* index, int64_t n,
                              int64_t H, int32_t elem_bytes, pt_stream_t stream) {
  if (n == 0 || H == 0) return PT_OK;
  PT_REQUIRE(n > 0 && H > 0 && in && out && index && elem_bytes > 0, "gather_rows: bad arguments");
  const int64_t rb = H * elem_bytes, lib = ld_in * elem_bytes, lob = ld_out * elem_bytes;
  const bool vec = (rb % 16 == 0) && (lib % 16 == 0) && (lob % 16 == 0) && ((uintptr_t)in % 16 == 0) && ((uintptr_t)out % 16 == 0);
  const unsigned blocks = (unsigned)cdiv(n, 4);
  hipStream_t s = (hipStream_t)stream;
  if (vec) gather_rows_kernel<true><<<blocks, 256, 0, s>>>((const char*)in, lib, (char*)out, lob, index, n, rb);
  else     gather_rows_kernel<false><<<blocks, 256, 0, s>>>((const char*)in, lib, (char*)out, lob, index, n, rb);
  return check_launch("gather_rows");
}

extern "C" int64_t pt_gather_rows_backward_workspace_bytes(int64_t n, int64_t rows) {
  // cnt[rows], cursor[rows], seg_start[rows+1], block_sums[ceil(rows/1024)], list[n]
  return align_up(rows * 4, 256) * 2 + align_up((rows + 1) * 4, 256) + align_up(cdiv(rows > 0 ? rows : 1, 1024) * 4, 256) +
         align_up((n > 0 ? n : 1) * 4, 256);
}

extern "C" int pt_gather_rows_backward(const void* grad_out, int64_t ld_go, void* grad_in, int64_t ld_gi,
                                       const int64_t* index, int64_t n, int64_t rows, int64_t H, int dtype, void* workspace,
                                       int64_t workspace_bytes, pt_stream_t stream) {
  if (rows == 0 || H == 0) return PT_OK;
  PT_REQUIRE(rows > 0 && n >= 0 && H > 0 && grad_in && workspace, "gather_rows_backward: bad arguments");
  PT_REQUIRE(n == 0 || (grad_out && index), "gather_rows_backward: null pointer");
  PT_REQUIRE(n < (1ll << 31) && rows < (1ll << 31), "gather_rows_backward: sizes exceed int32");
  PT_REQUIRE(workspace_bytes >= pt_gather_rows_backward_workspace_bytes(n, rows), "gather_rows_backward: workspace too small");
  hipStream_t s = (hipStream_t)stream;
  char* wsp = (char*)workspace;
  int32_t* cnt = (int32_t*)wsp; wsp += align_up(rows * 4, 256);
  int32_t* cursor = (int32_t*)wsp; wsp += align_up(rows * 4, 256);
  int32_t* seg_start = (int32_t*)wsp; wsp += align_up((rows + 1) * 4, 256);
  int32_t* block_sums = (int32_t*)wsp; wsp += align_up(cdiv(rows, 1024) * 4, 256);
  int32_t* list = (int32_t*)wsp;
  const int64_t nb = cdiv(rows, 1024);
  fill_i32_kernel<<<(unsigned)cdiv(2 * align_up(rows * 4, 256) / 4, 256), 256, 0, s>>>(cnt, 2 * align_up(rows * 4, 256) / 4, 0);
  if (n > 0) gb_count_kernel<<<(unsigned)cdiv(n, 256), 256, 0, s>>>(index, n, rows, cnt);
  scan_block_sums_kernel<<<(unsigned)nb, 1024, 0, s>>>(cnt, rows, block_sums);
  scan_top_kernel<<<1, 1024, 0, s>>>(block_sums, nb);
  scan_apply_kernel<<<(unsigned)nb, 1024, 0, s>>>(cnt, rows, block_sums, seg_start);
  if (n > 0) gb_fill_kernel<<<(unsigned)cdiv(n, 256), 256, 0, s>>>(index, n, rows, seg_start, cursor, list);
  const unsigned blocks = (unsigned)cdiv(rows, 4);
  const int eb = dtype == PT_F32 ? 4 : 2;
  const bool vec = (H % 8 == 0) && ((ld_go * eb) % 16 == 0) && ((ld_gi * eb) % 16 == 0) && ((uintptr_t)grad_out % 16 == 0) &&
                   ((uintptr_t)grad_in % 16 == 0);
#define PT_GB(S)                                                                                                         \
  do {                                                                                                                   \
    if (vec) gb_sum_kernel<S, true><<<blocks, 256, 0, s>>>((const char*)grad_out, ld_go * eb, (char*)grad_in, ld_gi * eb, seg_start, list, rows, H); \
    else     gb_sum_kernel<S, false><<<blocks, 256, 0, s>>>((const char*)grad_out, ld_go * eb, (char*)grad_in, ld_gi * eb, seg_start, list, rows, H); \
  } while (0)
  switch (dtype) {
    case PT_BF16: PT_GB(st_bf16); break;
    case PT_F16:  PT_GB(st_f16); break;
    case PT_F32:  PT_GB(st_f32); break;
    default: PT_REQUIRE(false, "gather_rows_backward: unsupported dtype %d", dtype);
  }
#undef PT_GB
  return check_launch("gather_rows_backward");
}

extern "C" int pt_group_indices(const int32_t* offs, int32_t G, int64_t M, void* group_ids, int32_t out_bytes,
                                pt_stream_t stream) {
  if (M == 0) return PT_OK;
  PT_REQUIRE(M > 0 && G > 0 && offs && group_ids, "group_indices: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  if (out_bytes == 4) group_indices_kernel<int32_t><<<(unsigned)cdiv(M, 256), 256, 0, s>>>(offs, G, M, (int32_t*)group_ids);
  else if (out_bytes == 8) group_indices_kernel<int64_t><<<(unsigned)cdiv(M, 256), 256, 0, s>>>(offs, G, M, (int64_t*)group_ids);
  else PT_REQUIRE(false, "group_indices: out_dtype_bytes must be 4 or 8");
  return check_launch("group_indices");
}

// out[r] = expand_idx[row_map[r]] for row_map[r] in [0, n_expand), -1 otherwise: the source row of
// every grouped row when the routed rows are themselves an expansion of deduplicated rows.
__global__ __launch_bounds__(256) void compose_row_map_kernel(const int32_t* row_map, int64_t n, const int64_t* expand_idx,
                                                              int64_t n_expand, int64_t n_src, int32_t* out) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= n) return;
  const int32_t i = row_map[r];
  int64_t s = -1;
  if (i >= 0 && i < n_expand) {
    s = expand_idx[i];
    if (s < 0 || s >= n_src) s = -1;  // an index outside the source rows reads nothing
  }
  out[r] = (int32_t)s;
}

extern "C" int pt_compose_row_map(const int32_t* row_map, int64_t n, const int64_t* expand_idx, int64_t n_expand,
                                  int64_t n_src, int32_t* out, pt_stream_t stream) {
  PT_REQUIRE(n >= 0 && n_expand >= 0 && n_src >= 0 && n_src < (1ll << 31), "compose_row_map: bad sizes");
  if (n == 0) return PT_OK;
  PT_REQUIRE(row_map && out && (expand_idx || n_expand == 0), "compose_row_map: null pointer");
  compose_row_map_kernel<<<(unsigned)cdiv(n, 256), 256, 0, (hipStream_t)stream>>>(row_map, n, expand_idx, n_expand, n_src, out);
  return check_launch("compose_row_map");
}

extern "C" int64_t pt_dedup_workspace_bytes(int64_t m, int32_t k, int32_t E, int32_t ep) {
  (void)k;
  const int64_t W = cdiv(m > 0 ? m : 1, kWaveTokens);
  return align_up(W * E * 4, 256) + align_up(W * ep * 4, 256) + align_up((int64_t)E * 4, 256) + 256 +
         align_up((int64_t)(E + ep) * 4, 256);
}

extern "C" int pt_dedup_prepare_dispatch(const int64_t* topk_ids, int64_t ld_ids, int64_t m, int32_t k, int32_t E,
                                         int32_t ep, int32_t epr, int64_t* tokens_per_ep_rank, int64_t* dedup_tokens_per_gpu,
                                         int64_t* dispatch_token_idxs, int64_t* idxs, int64_t* expand_idx, int64_t* send_meta,
                                         void* workspace, int64_t workspace_bytes, pt_stream_t stream) {
  PT_REQUIRE(m > 0 && k > 0 && E > 0 && E <= kMaxExperts && ep > 0 && ep <= 32 && ep * epr == E,
             "dedup_prepare_dispatch: m=%lld k=%d E=%d ep=%d epr=%d", (long long)m, k, E, ep, epr);
  PT_REQUIRE(m * k < (1ll << 31), "dedup_prepare_dispatch: m*k exceeds int32");
  PT_REQUIRE(topk_ids && tokens_per_ep_rank && dedup_tokens_per_gpu && dispatch_token_idxs && idxs && expand_idx &&
                 send_meta && workspace, "dedup_prepare_dispatch: null pointer");
  PT_REQUIRE(workspace_bytes >= pt_dedup_workspace_bytes(m, k, E, ep), "dedup_prepare_dispatch: workspace too small");
  hipStream_t s = (hipStream_t)stream;
  const int64_t W = cdiv(m, kWaveTokens);
  char* wsp = (char*)workspace;
  int32_t* cnt_e = (int32_t*)wsp; wsp += align_up(W * E * 4, 256);
  int32_t* cnt_g = (int32_t*)wsp; wsp += align_up(W * ep * 4, 256);
  int32_t* expert_starts = (int32_t*)wsp; wsp += align_up((int64_t)E * 4, 256);
  int32_t* gpu_starts = (int32_t*)wsp; wsp += 256;
  int32_t* totals = (int32_t*)wsp;
  const unsigned blocks = (unsigned)cdiv(W, 4);
  dd_hist_kernel<<<blocks, 256, (size_t)4 * (E + 32) * 4, s>>>(topk_ids, ld_ids, m, k, E, ep, epr, cnt_e, cnt_g);
  dd_scan_cols_kernel<<<(unsigned)cdiv(E + ep, 4), 256, 0, s>>>(cnt_e, cnt_g, W, E, ep, totals);
  dd_scan_totals_kernel<<<1, 64, 0, s>>>(totals, E, ep, epr, tokens_per_ep_rank, dedup_tokens_per_gpu, send_meta, expert_starts,
                                         gpu_starts);
  const size_t lds = (size_t)4 * (E + 32 + 64 * ep) * 4;
  dd_rank_kernel<<<blocks, 256, lds, s>>>(topk_ids, ld_ids, m, k, E, ep, epr, bits_for(E), cnt_e, cnt_g, expert_starts,
                                          gpu_starts, dispatch_token_idxs, idxs, expand_idx);
  return check_launch("dedup_prepare_dispatch");
}

extern "C" int pt_build_expert_idxs(const int64_t* counts, int32_t E, int32_t ep, int32_t epr, int64_t max_total,
                                    int64_t* expert_idxs, int64_t* output_splits, pt_stream_t stream) {
  PT_REQUIRE(E > 0 && E <= kMaxExperts && ep > 0 && ep * epr == E && counts && output_splits, "build_expert_idxs: bad arguments");
  PT_REQUIRE(max_total == 0 || expert_idxs, "build_expert_idxs: null pointer");
  const unsigned blocks = (unsigned)(max_total > 0 ? cdiv(max_total, 256) : 1);
  build_expert_idxs_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(counts, E, ep, epr, max_total, expert_idxs, output_splits);
  return check_launch("build_expert_idxs");
}

extern "C" int pt_adjust_expand_idx(const int64_t* received, int64_t* out, const int64_t* dedup_counts, int64_t dedup_stride,
                                    const int64_t* output_splits, int32_t ep, int64_t n, pt_stream_t stream) {
  if (n == 0) return PT_OK;
  PT_REQUIRE(n > 0 && ep > 0 && ep <= 32 && received && out && dedup_counts && output_splits, "adjust_expand_idx: bad arguments");
  adjust_expand_idx_kernel<<<(unsigned)cdiv(n, 256), 256, 0, (hipStream_t)stream>>>(received, out, dedup_counts, dedup_stride,
                                                                                      output_splits, ep, n);
  return check_launch("adjust_expand_idx");
}
