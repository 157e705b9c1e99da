// FP8 (e4m3) GEMMs on the gfx950 matrix cores with hardware block scaling.
//
// One kernel template serves the three GEMM shapes of the expert path:
//   dense      out[m,n]      = sum_k a[m,k] b[n,k]
//   m-grouped  out[rows_g,n] = a[rows_g,:] . b[g][n,:]            (forward, dgrad)
//   k-grouped  out[g][n,k]   = sum_{m in g} dy_t[n,m] x_t[k,m]     (wgrad)
// All are "NT": both operands are contiguous along the reduction dimension.  Every scale of
// this path is an exact power of two, so it is handed to v_mfma_scale_f32_32x32x64_f8f6f4 as
// an E8M0 exponent byte and applied inside the MFMA: one fp32 accumulator runs over the whole
// reduction and no VALU promotion step is needed.
//
// Workgroup = BM x BN output tile, 128-deep reduction steps (one scale block).  Operand tiles go
// global -> LDS with 16-byte direct-to-LDS loads (no VGPR staging), double buffered; 16-byte
// chunks are XOR-swizzled by choosing which global chunk each lane fetches, so the later
// ds_read_b128 fragment reads are spread over the banks.  Per step a wave reads all of its
// fragments, then the next tile's loads are issued, then the MFMAs run while those loads land.
#include "common.h"
#include "gemm_args.h"
#include <stdlib.h>
#include <string.h>

namespace pt {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __attribute__((aligned(16))) uint32_t g_zero_chunk[4] = {0, 0, 0, 0};

__device__ __forceinline__ void load_lds16(const uint8_t* g, uint8_t* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

template <int BM, int BN, int WGM, int WGN>
__global__ __launch_bounds__(WGM * WGN * 64) void fp8_gemm_nt_kernel(GemmArgs p) {
  constexpr int NW = WGM * WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;  // direct-to-LDS wave loads per step
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile/wave mismatch");
  constexpr int STAGE = (BM + BN) * 128;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  __shared__ int s_cnt[NW];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;

  // ---- which tile: consecutive logical tiles stay on one XCD (workgroups are dealt round-robin
  // over the 8 XCDs), and inside a group the tiles that share a b-tile are adjacent ----
  const int64_t per_xcd = (p.total_tiles + 7) / 8;
  const int64_t t = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (t >= p.total_tiles) return;

  int64_t a_row0, b_row0, a_lim, b_lim, k_begin, k_end, kb0;
  const uint8_t* bp = p.b;
  const float* sbp = p.sb;
  char* outp = (char*)p.out;
  if (p.mode == GEMM_DENSE) {
    const int ta = (int)(t % p.tiles_a), tb = (int)(t / p.tiles_a);
    a_row0 = (int64_t)ta * BM; b_row0 = (int64_t)tb * BN;
    a_lim = p.rows_a; b_lim = p.rows_b; k_begin = 0; k_end = p.red; kb0 = 0;
  } else if (p.mode == GEMM_M_GROUPED) {
    // row tile index in group-major order; groups are multiples of 128 rows and BM == 128
    const int64_t tr = t / p.tiles_b;
    const int64_t row = tr * BM;
    int cnt = 0;
    for (int g = tid; g < p.G; g += NW * 64) cnt += ((int64_t)p.offs[g] <= row) ? 1 : 0;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) cnt += __shfl_xor(cnt, d);
    if (lane == 0) s_cnt[wave] = cnt;
    __syncthreads();
    int g = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) g += s_cnt[w];
    if (g >= p.G) return;  // rows past the last group
    const int64_t gs = g == 0 ? 0 : p.offs[g - 1], ge = p.offs[g];
    const int64_t m_tiles = (ge - gs) / BM, first = (gs / BM) * p.tiles_b;
    const int64_t idx = t - first;
    const int tb = (int)(idx / m_tiles);
    a_row0 = gs + (idx % m_tiles) * BM; b_row0 = (int64_t)tb * BN;
    a_lim = ge; b_lim = p.rows_b; k_begin = 0; k_end = p.red; kb0 = 0;
    bp += (int64_t)g * p.b_stride_g; sbp += (int64_t)g * p.sb_stride_g;
  } else {
    const int64_t per_g = (int64_t)p.tiles_a * p.tiles_b;
    const int g = (int)(t / per_g);
    const int64_t idx = t % per_g;
    const int ta = (int)(idx % p.tiles_a), tb = (int)(idx / p.tiles_a);
    a_row0 = (int64_t)ta * BM; b_row0 = (int64_t)tb * BN;
    a_lim = p.rows_a; b_lim = p.rows_b;
    k_begin = g == 0 ? 0 : k_group_end(p, g - 1); k_end = k_group_end(p, g); kb0 = k_begin >> 7;
    outp += (int64_t)g * p.out_stride_g * (p.out_dtype == PT_F32 ? 4 : 2);
  }
  const int nk = (int)((k_end - k_begin + 127) >> 7);

  // ---- per-lane global source pointers of the direct-to-LDS loads ----
  // wave-load q covers tile rows 8*(wave + NW*q) .. +8; lane -> row +lane/8, physical chunk lane%8,
  // which holds logical chunk (lane%8) ^ f(row), f(row) = (row&7) ^ ((row>>3)&1).
  const int lrow = lane >> 3;
  const int lchunk = (lane & 7) ^ lrow ^ (wave & 1);
  const uint8_t* ap[LA];
  const uint8_t* bpp[LB];
#pragma unroll
  for (int q = 0; q < LA; ++q) {
    int64_t r = a_row0 + 8 * (wave + NW * q) + lrow;
    if (r >= a_lim) r = a_lim - 1;
    ap[q] = p.a + r * p.lda + k_begin + lchunk * 16;
  }
#pragma unroll
  for (int q = 0; q < LB; ++q) {
    int64_t r = b_row0 + 8 * (wave + NW * q) + lrow;
    if (r >= b_lim) r = b_lim - 1;
    bpp[q] = bp + r * p.ldb + k_begin + lchunk * 16;
  }
  const int64_t k_len = k_end - k_begin;
  const uint8_t* zero = (const uint8_t*)g_zero_chunk;

  auto issue_loads = [&](int it, int stage) {
    uint8_t* sA = lds + stage * STAGE;
    uint8_t* sB = sA + BM * 128;
    const int64_t koff = (int64_t)it * 128;
    const bool in = koff + lchunk * 16 < k_len;  // false only in a ragged last step
#pragma unroll
    for (int q = 0; q < LA; ++q) load_lds16(in ? ap[q] + koff : zero, sA + (wave + NW * q) * 1024);
#pragma unroll
    for (int q = 0; q < LB; ++q) load_lds16(in ? bpp[q] + koff : zero, sB + (wave + NW * q) * 1024);
  };

  // ---- per-lane scale sources ----
  int64_t sa_idx[TM], sb_idx[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    int64_t r = a_row0 + wm0 + i * 32 + (lane & 31);
    if (r >= a_lim) r = a_lim - 1;
    sa_idx[i] = (r >> p.sa_shift) * p.sa_rs + kb0 * p.sa_ks;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int64_t r = b_row0 + wn0 + j * 32 + (lane & 31);
    if (r >= b_lim) r = b_lim - 1;
    sb_idx[j] = (r >> p.sb_shift) * p.sb_rs + kb0 * p.sb_ks;
  }

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // fragment read offsets inside a tile (lane-constant): row (lane&31), chunk (ks*4 + (lane>>5)*2 + h) ^ f
  const int f = (lane & 7) ^ ((lane >> 3) & 1);
  const int roff = (lane & 31) * 128;
  int coff[2][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int h = 0; h < 2; ++h) coff[ks][h] = roff + (((ks * 4 + (lane >> 5) * 2 + h) ^ f) << 4);

  // Scales of step `it` are fetched (raw fp32 bits) one step ahead, before that step's tile loads
  // are issued, and only turned into E8M0 bytes after the next barrier: nothing between a step's
  // loads and its MFMAs waits on the vector-memory counter.
  float raw_a[TM], raw_b[TN];
  if (nk > 0) {
#pragma unroll
    for (int i = 0; i < TM; ++i) raw_a[i] = p.sa[sa_idx[i]];
#pragma unroll
    for (int j = 0; j < TN; ++j) raw_b[j] = sbp[sb_idx[j]];
    issue_loads(0, 0);
  }

  for (int it = 0; it < nk; ++it) {
    const int stage = it & 1;
    // Every wave drains its own direct-to-LDS loads *before* the barrier: the workgroup fence of
    // __syncthreads() does not wait on the vector-memory counter, and the other waves are about
    // to read the rows this wave fetched.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int sca[TM], scb[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) sca[i] = (int)(__float_as_uint(raw_a[i]) >> 23);
#pragma unroll
    for (int j = 0; j < TN; ++j) scb[j] = (int)(__float_as_uint(raw_b[j]) >> 23);
    const uint8_t* sA = lds + stage * STAGE + wm0 * 128;
    const uint8_t* sB = lds + stage * STAGE + BM * 128 + wn0 * 128;
    v8i af[2][TM], bf[2][TN];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const uint4 lo = *(const uint4*)(sA + i * 4096 + coff[ks][0]);
        const uint4 hi = *(const uint4*)(sA + i * 4096 + coff[ks][1]);
        af[ks][i] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint4 lo = *(const uint4*)(sB + j * 4096 + coff[ks][0]);
        const uint4 hi = *(const uint4*)(sB + j * 4096 + coff[ks][1]);
        bf[ks][j] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
      }
    }
    if (it + 1 < nk) {
#pragma unroll
      for (int i = 0; i < TM; ++i) raw_a[i] = p.sa[sa_idx[i] + (int64_t)(it + 1) * p.sa_ks];
#pragma unroll
      for (int j = 0; j < TN; ++j) raw_b[j] = sbp[sb_idx[j] + (int64_t)(it + 1) * p.sb_ks];
      issue_loads(it + 1, stage ^ 1);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[ks][i], bf[ks][j], acc[i][j], 0, 0, 0, sca[i], 0,
                                                                     scb[j]);
  }

  // ---- epilogue: lane holds column (lane&31), rows 8*(v/4) + 4*(lane>>5) + (v&3) of each 32x32 ----
  if (p.mode == GEMM_K_GROUPED && nk == 0 && p.accumulate) return;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int64_t col = b_row0 + wn0 + j * 32 + (lane & 31);
      if (col >= b_lim) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t row = a_row0 + wm0 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (row >= a_lim) continue;
        const float x = acc[i][j][v];
        if (p.out_dtype == PT_F32) {
          float* o = (float*)outp + row * p.ldo + col;
          *o = p.accumulate ? (*o + x) : x;
        } else {
          uint16_t* o = (uint16_t*)outp + row * p.ldo + col;
          uint32_t r = f32_to_bf16_bits(x);
          if (p.accumulate) r = f32_to_bf16_bits(bf16_bits_to_f32(*o) + bf16_bits_to_f32(r));
          *o = (uint16_t)r;
        }
      }
    }
}

template <int BM, int BN, int WGM, int WGN>
static int launch_gemm(const GemmArgs& a, hipStream_t stream) {
  if (a.total_tiles == 0) return PT_OK;
  constexpr int threads = WGM * WGN * 64;
  constexpr size_t lds = (size_t)2 * (BM + BN) * 128;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)fp8_gemm_nt_kernel<BM, BN, WGM, WGN>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_error("gemm: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return PT_ERR_LAUNCH; }
    attr_set = true;
  }
  const int64_t per_xcd = (a.total_tiles + 7) / 8;
  const int64_t blocks = per_xcd * 8;
  PT_REQUIRE(blocks < (1ll << 31), "gemm: grid too large");
  hipLaunchKernelGGL((fp8_gemm_nt_kernel<BM, BN, WGM, WGN>), dim3((unsigned)blocks), dim3(threads), lds, stream, a);
  return check_launch("fp8_gemm_nt_kernel");
}

// PT_GEMM_IMPL overrides the choice of kernel for measurements: "t" = one 128x128 tile per
// workgroup, "p0" = persistent two-phase kernel, "q0" / "q1" = persistent software-pipelined kernel
// (8 / 4 waves), "r0" = persistent kernel with the row-split loop.  Unset: chosen per call from the shape (below).
enum { IMPL_UNSET = -3, IMPL_AUTO = -2, IMPL_TILE = -1, IMPL_PIPELINED = 100, IMPL_ROWSPLIT = 200 };
static int g_impl = IMPL_UNSET;
static bool parse_impl(const char* e, int& impl) {
  if (!e || !*e || !strcmp(e, "auto")) impl = IMPL_AUTO;
  else if (!strcmp(e, "t")) impl = IMPL_TILE;
  else if (!strcmp(e, "p0")) impl = 0;
  else if (!strcmp(e, "q0") || !strcmp(e, "q1")) impl = IMPL_PIPELINED + (e[1] - '0');
  else if (!strcmp(e, "r0")) impl = IMPL_ROWSPLIT;
  else return false;
  return true;
}
static int gemm_impl() {
  if (g_impl == IMPL_UNSET) {
    int impl;
    g_impl = parse_impl(getenv("PT_GEMM_IMPL"), impl) ? impl : IMPL_AUTO;
  }
  return g_impl;
}

// Choice of the persistent kernel, from measurements on MI355X inside a training step (operands
// freshly written, i.e. partly cache-resident):
//   m-grouped, k-grouped  the row-split loop: its loads never pause, which matters most where
//              operands come from HBM (every group has its own b operand), and waves of a half-empty
//              tile skip their MFMAs.  +1..5 % per layer over the better of the other two.
//   dense      the software-pipelined loop from K = 512 on (+5 % at 512, +13..20 % from 2048 on
//              over the two-phase loop, +5..8 % over the row-split loop); below, the two-phase loop,
//              which has no fill/drain of one 128-block per tile.
enum { KERNEL_TWO_PHASE, KERNEL_PIPELINED, KERNEL_ROWSPLIT };
static int preferred_kernel(const GemmArgs& g) {
  if (g.mode != GEMM_DENSE) return KERNEL_ROWSPLIT;
  return g.red >= 512 ? KERNEL_PIPELINED : KERNEL_TWO_PHASE;
}

// The persistent kernels address operands through 32-bit buffer offsets (signed range for the
// loads, whose out-of-range marker is bit 31) and the result through an unsigned 32-bit byte
// offset from the start of the output (of one group's block in the k-grouped mode, of the
// scattered output when rows are stored through an index).  Larger problems go to the
// tile-per-workgroup kernel, which uses 64-bit pointers.
static bool fits_persistent(const GemmArgs& g) {
  const int64_t lim = (1ll << 31) - 1;
  const int64_t esz = g.out_dtype == PT_F32 ? 4 : 2;
  const int64_t out_rows = g.out_row_index ? g.out_rows : g.rows_a;
  const int64_t out_extent = out_rows * g.ldo * esz;
  return g.a_bytes < lim && g.b_bytes < lim && g.sa_bytes < lim && g.sb_bytes < lim && g.rows_a < lim && g.rows_b < lim &&
         g.red < lim && out_extent < (1ll << 32);
}

static int dispatch_gemm(const GemmArgs& g, hipStream_t stream) {
  const int impl = gemm_impl();
  const bool fits = fits_persistent(g);
  if (g.b_kmajor) {  // one kernel reads this layout, whatever kernel was selected for the others
    PT_REQUIRE(fits, "gemm: the reduction-major b operand needs the row-split kernel, which addresses operands below 2 GiB "
                     "and an output below 4 GiB through 32-bit byte offsets; larger problems take the NT entry point on the "
                     "transposed operand");
    return launch_gemm_rowsplit(g, 0, stream);
  }
  PT_REQUIRE((!g.out_row_index && !g.bias) || (impl != IMPL_TILE && fits),
             "gemm: scattered output rows and the fused bias need the persistent kernels, which address every operand and "
             "the output (one group's block of it in the k-grouped mode) through 32-bit byte offsets: operands below 2 GiB, "
             "output below 4 GiB");
  if (impl == IMPL_TILE || !fits) return launch_gemm<128, 128, 2, 2>(g, stream);
  if (impl == IMPL_AUTO) {
    switch (preferred_kernel(g)) {
      case KERNEL_ROWSPLIT: return launch_gemm_rowsplit(g, 0, stream);
      case KERNEL_PIPELINED: return launch_gemm_pipelined(g, 0, stream);
      default: return launch_gemm_persistent(g, 0, stream);
    }
  }
  if (impl >= IMPL_ROWSPLIT) return launch_gemm_rowsplit(g, impl - IMPL_ROWSPLIT, stream);
  if (impl >= IMPL_PIPELINED) return launch_gemm_pipelined(g, impl - IMPL_PIPELINED, stream);
  return launch_gemm_persistent(g, impl, stream);
}

}  // namespace pt

using namespace pt;

extern "C" int pt_gemm_select_kernel(const char* name) {
  int impl;
  PT_REQUIRE(parse_impl(name, impl), "gemm_select_kernel: unknown kernel '%s' (auto, p0, q0, q1, r0, t)", name);
  g_impl = impl;
  return PT_OK;
}

static bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

static int gemm_nt_dense_impl(const void* a_fp8, int64_t lda, const float* a_scale, const void* b_fp8, int64_t ldb,
                              const float* b_scale, void* out, int out_dtype, int64_t M, int64_t N, int64_t K,
                              pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && N >= 0 && K >= 0, "gemm_nt_dense: negative size");
  if (M == 0 || N == 0) return PT_OK;
  PT_REQUIRE(K > 0 && K % 16 == 0, "gemm_nt_dense: K=%lld must be a positive multiple of 16", (long long)K);
  PT_REQUIRE(lda >= K && ldb >= K && lda % 16 == 0 && ldb % 16 == 0, "gemm_nt_dense: row pitches must be multiples of 16 and at least K");
  PT_REQUIRE(a_fp8 && a_scale && b_fp8 && b_scale && out && al16(a_fp8) && al16(b_fp8), "gemm_nt_dense: null or misaligned pointer");
  PT_REQUIRE(out_dtype == PT_BF16 || out_dtype == PT_F32, "gemm_nt_dense: out_dtype must be bf16 or fp32");
  const int64_t KB = cdiv(K, 128);
  GemmArgs g = {};
  g.a = (const uint8_t*)a_fp8; g.lda = lda; g.b = (const uint8_t*)b_fp8; g.ldb = ldb;
  g.sa = a_scale; g.sa_rs = KB; g.sa_ks = 1; g.sa_shift = 0;
  g.sb = b_scale; g.sb_rs = KB; g.sb_ks = 1; g.sb_shift = 7;
  g.out = out; g.ldo = N; g.out_dtype = out_dtype; g.accumulate = 0;
  g.rows_a = M; g.rows_b = N; g.red = K; g.mode = GEMM_DENSE;
  g.a_bytes = (M - 1) * lda + K; g.b_bytes = (N - 1) * ldb + K; g.sa_bytes = M * KB * 4; g.sb_bytes = cdiv(N, 128) * KB * 4;
  g.tiles_a = (int)cdiv(M, 128); g.tiles_b = (int)cdiv(N, 128);
  g.total_tiles = (int64_t)g.tiles_a * g.tiles_b;
  return dispatch_gemm(g, (hipStream_t)stream);
}

extern "C" int pt_gemm_nt_dense(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale, void* out,
                                int out_dtype, int64_t M, int64_t N, int64_t K, pt_stream_t stream) {
  return gemm_nt_dense_impl(a_fp8, K, a_scale, b_fp8, K, b_scale, out, out_dtype, M, N, K, stream);
}

extern "C" int pt_gemm_nt_dense_ld(const void* a_fp8, int64_t lda, const float* a_scale, const void* b_fp8, int64_t ldb,
                                   const float* b_scale, void* out, int out_dtype, int64_t M, int64_t N, int64_t K,
                                   pt_stream_t stream) {
  return gemm_nt_dense_impl(a_fp8, lda, a_scale, b_fp8, ldb, b_scale, out, out_dtype, M, N, K, stream);
}

// ---- split-K: a dense GEMM whose output has too few tiles to fill the GPU ------------------------
// The reduction is cut into `splits` ranges of split_len (a multiple of 128, so every range starts
// on a scale block); range s is computed like a group of the k-grouped mode into the fp32 slab
// partial[s] (M x N), and pt_sum_partials adds the slabs in the order of s.
static int gemm_nt_dense_splitk_impl(const void* a_fp8, int64_t lda, const float* a_scale, const void* b_fp8, int64_t ldb,
                                     const float* b_scale, float* partial, int32_t splits, int64_t split_len, int64_t M,
                                     int64_t N, int64_t K, pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && N >= 0 && K >= 0, "gemm_nt_dense_splitk: negative size");
  if (M == 0 || N == 0) return PT_OK;
  PT_REQUIRE(K > 0 && K % 16 == 0, "gemm_nt_dense_splitk: K=%lld must be a positive multiple of 16", (long long)K);
  PT_REQUIRE(lda >= K && ldb >= K && lda % 16 == 0 && ldb % 16 == 0,
             "gemm_nt_dense_splitk: row pitches must be multiples of 16 and at least K");
  PT_REQUIRE(splits >= 1 && split_len > 0 && split_len % 128 == 0 && (int64_t)splits * split_len >= K &&
                 (int64_t)(splits - 1) * split_len < K,
             "gemm_nt_dense_splitk: %d ranges of %lld (a multiple of 128) must cover K=%lld with none empty", splits,
             (long long)split_len, (long long)K);
  PT_REQUIRE(a_fp8 && a_scale && b_fp8 && b_scale && partial && al16(a_fp8) && al16(b_fp8),
             "gemm_nt_dense_splitk: null or misaligned pointer");
  const int64_t KB = cdiv(K, 128);
  GemmArgs g = {};
  g.a = (const uint8_t*)a_fp8; g.lda = lda; g.b = (const uint8_t*)b_fp8; g.ldb = ldb;
  g.sa = a_scale; g.sa_rs = KB; g.sa_ks = 1; g.sa_shift = 0;
  g.sb = b_scale; g.sb_rs = KB; g.sb_ks = 1; g.sb_shift = 7;
  g.out = partial; g.ldo = N; g.out_dtype = PT_F32; g.accumulate = 0;
  g.rows_a = M; g.rows_b = N; g.red = K; g.mode = GEMM_K_GROUPED; g.offs = nullptr; g.G = splits; g.split_len = split_len;
  g.out_stride_g = M * N;
  g.a_bytes = (M - 1) * lda + K; g.b_bytes = (N - 1) * ldb + K; g.sa_bytes = M * KB * 4; g.sb_bytes = cdiv(N, 128) * KB * 4;
  g.tiles_a = (int)cdiv(M, 128); g.tiles_b = (int)cdiv(N, 128);
  g.total_tiles = (int64_t)g.tiles_a * g.tiles_b * splits;
  return dispatch_gemm(g, (hipStream_t)stream);
}

extern "C" int pt_gemm_nt_dense_splitk(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale,
                                       float* partial, int32_t splits, int64_t split_len, int64_t M, int64_t N, int64_t K,
                                       pt_stream_t stream) {
  return gemm_nt_dense_splitk_impl(a_fp8, K, a_scale, b_fp8, K, b_scale, partial, splits, split_len, M, N, K, stream);
}

extern "C" int pt_gemm_nt_dense_splitk_ld(const void* a_fp8, int64_t lda, const float* a_scale, const void* b_fp8, int64_t ldb,
                                          const float* b_scale, float* partial, int32_t splits, int64_t split_len, int64_t M,
                                          int64_t N, int64_t K, pt_stream_t stream) {
  return gemm_nt_dense_splitk_impl(a_fp8, lda, a_scale, b_fp8, ldb, b_scale, partial, splits, split_len, M, N, K, stream);
}

namespace pt {
template <typename S>
__global__ __launch_bounds__(256) void sum_partials_kernel(const float* partial, int splits, int64_t n, char* out) {
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;  // n is a multiple of 8
  if (i0 >= n) return;
  float acc[8];
  st_f32::load8(partial + i0, acc);
  for (int s = 1; s < splits; ++s) {
    float v[8];
    st_f32::load8(partial + (int64_t)s * n + i0, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] += v[j];
  }
  S::store8(out + i0 * S::kBytes, acc);
}
}  // namespace pt

extern "C" int pt_sum_partials(const float* partial, int32_t splits, int64_t n, void* out, int out_dtype, pt_stream_t stream) {
  PT_REQUIRE(splits >= 1 && n >= 0, "sum_partials: bad sizes");
  if (n == 0) return PT_OK;
  PT_REQUIRE(partial && out && al16(partial) && al16(out) && n % 8 == 0, "sum_partials: null or misaligned pointer, or n not a multiple of 8");
  PT_REQUIRE(out_dtype == PT_BF16 || out_dtype == PT_F32, "sum_partials: out_dtype must be bf16 or fp32");
  const int64_t blocks = cdiv(n, 2048);
  PT_REQUIRE(blocks < (1ll << 31), "sum_partials: too many elements");
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == PT_BF16) hipLaunchKernelGGL((sum_partials_kernel<st_bf16>), dim3((unsigned)blocks), dim3(256), 0, st, partial, splits, n, (char*)out);
  else hipLaunchKernelGGL((sum_partials_kernel<st_f32>), dim3((unsigned)blocks), dim3(256), 0, st, partial, splits, n, (char*)out);
  return check_launch("sum_partials_kernel");
}

static int gemm_m_grouped_impl(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale, void* out,
                               int out_dtype, const int32_t* offs, int32_t G, int64_t M, int64_t N, int64_t K,
                               const int32_t* out_row_index, int64_t out_rows, const void* bias, pt_stream_t stream,
                               bool b_kmajor = false) {
  PT_REQUIRE(M >= 0 && N >= 0 && K >= 0 && G > 0, "gemm_m_grouped_nt: bad sizes");
  if (M == 0 || N == 0) return PT_OK;
  PT_REQUIRE(M % 128 == 0, "gemm_m_grouped_nt: M=%lld must be a multiple of 128", (long long)M);
  PT_REQUIRE(K > 0 && K % 16 == 0, "gemm_m_grouped_nt: K=%lld must be a positive multiple of 16", (long long)K);
  PT_REQUIRE(a_fp8 && a_scale && b_fp8 && b_scale && out && offs && al16(a_fp8) && al16(b_fp8), "gemm_m_grouped_nt: null or misaligned pointer");
  PT_REQUIRE(out_dtype == PT_BF16, "gemm_m_grouped_nt: out_dtype must be bf16");
  PT_REQUIRE((N * K) % 16 == 0, "gemm_m_grouped_nt: N*K must be a multiple of 16");
  const int64_t KB = cdiv(K, 128), NB = cdiv(N, 128);
  GemmArgs g = {};
  g.a = (const uint8_t*)a_fp8; g.lda = K; g.b = (const uint8_t*)b_fp8; g.ldb = K;
  g.sa = a_scale; g.sa_rs = KB; g.sa_ks = 1; g.sa_shift = 0;
  g.sb = b_scale; g.sb_rs = KB; g.sb_ks = 1; g.sb_shift = 7;
  g.out = out; g.ldo = N; g.out_dtype = out_dtype; g.accumulate = 0;
  g.rows_a = M; g.rows_b = N; g.red = K; g.mode = GEMM_M_GROUPED; g.offs = offs; g.G = G;
  g.b_stride_g = N * K; g.sb_stride_g = NB * KB;
  g.a_bytes = M * K; g.b_bytes = N * K; g.sa_bytes = M * KB * 4; g.sb_bytes = NB * KB * 4;
  g.tiles_a = (int)(M / 128); g.tiles_b = (int)NB;
  g.total_tiles = (int64_t)g.tiles_a * g.tiles_b;
  if (b_kmajor) {
    // b[g] is [K, N] (row pitch N), its scales [ceil(K/128), ceil(N/128)]: scale(b row n, block kb) = sb[kb * NB + n / 128]
    PT_REQUIRE(N % 16 == 0, "gemm_m_grouped_nn: N=%lld must be a multiple of 16", (long long)N);
    // (b_bytes = K * N is the exact extent of one group's matrix: the kernel leaves the rows past
    // the end of a ragged reduction to the buffer descriptor's range check)
    g.b_kmajor = 1; g.ldb = N; g.sb_rs = 1; g.sb_ks = NB;
  }
  if (out_row_index) {
    PT_REQUIRE(out_rows >= 0 && N % 8 == 0 && al16(out) && out_rows * N * 2 < (1ll << 32),
               "gemm_m_grouped_nt_scatter: needs N %% 8 == 0, a 16-byte aligned output smaller than 4 GiB");
    g.out_row_index = out_row_index; g.out_rows = out_rows;
  }
  if (bias) {
    PT_REQUIRE(N % 8 == 0 && al16(out) && al16(bias),
               "gemm_m_grouped_nt_bias: needs N %% 8 == 0 and 16-byte aligned output and bias");
    g.bias = bias;
  }
  return dispatch_gemm(g, (hipStream_t)stream);
}

extern "C" int pt_gemm_m_grouped_nt(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale,
                                    void* out, int out_dtype, const int32_t* offs, int32_t G, int64_t M, int64_t N, int64_t K,
                                    pt_stream_t stream) {
  return gemm_m_grouped_impl(a_fp8, a_scale, b_fp8, b_scale, out, out_dtype, offs, G, M, N, K, nullptr, 0, nullptr, stream);
}

extern "C" int pt_gemm_m_grouped_nt_scatter(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale,
                                            void* out, int out_dtype, const int32_t* offs, int32_t G, int64_t M, int64_t N,
                                            int64_t K, const int32_t* out_row_index, int64_t out_rows, pt_stream_t stream) {
  PT_REQUIRE(out_row_index, "gemm_m_grouped_nt_scatter: null out_row_index");
  return gemm_m_grouped_impl(a_fp8, a_scale, b_fp8, b_scale, out, out_dtype, offs, G, M, N, K, out_row_index, out_rows, nullptr,
                             stream);
}

extern "C" int pt_gemm_m_grouped_nt_scatter_bias(const void* a_fp8, const float* a_scale, const void* b_fp8,
                                                 const float* b_scale, void* out, int out_dtype, const int32_t* offs, int32_t G,
                                                 int64_t M, int64_t N, int64_t K, const int32_t* out_row_index, int64_t out_rows,
                                                 const void* bias, pt_stream_t stream) {
  PT_REQUIRE(out_row_index && bias, "gemm_m_grouped_nt_scatter_bias: null out_row_index or bias");
  return gemm_m_grouped_impl(a_fp8, a_scale, b_fp8, b_scale, out, out_dtype, offs, G, M, N, K, out_row_index, out_rows, bias,
                             stream);
}

extern "C" int pt_gemm_m_grouped_nn(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale,
                                    void* out, int out_dtype, const int32_t* offs, int32_t G, int64_t M, int64_t N, int64_t K,
                                    pt_stream_t stream) {
  return gemm_m_grouped_impl(a_fp8, a_scale, b_fp8, b_scale, out, out_dtype, offs, G, M, N, K, nullptr, 0, nullptr, stream, true);
}

extern "C" int pt_gemm_m_grouped_nn_scatter(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale,
                                            void* out, int out_dtype, const int32_t* offs, int32_t G, int64_t M, int64_t N,
                                            int64_t K, const int32_t* out_row_index, int64_t out_rows, pt_stream_t stream) {
  PT_REQUIRE(out_row_index, "gemm_m_grouped_nn_scatter: null out_row_index");
  return gemm_m_grouped_impl(a_fp8, a_scale, b_fp8, b_scale, out, out_dtype, offs, G, M, N, K, out_row_index, out_rows, nullptr,
                             stream, true);
}

extern "C" int pt_gemm_m_grouped_nt_bias(const void* a_fp8, const float* a_scale, const void* b_fp8, const float* b_scale,
                                         void* out, int out_dtype, const int32_t* offs, int32_t G, int64_t M, int64_t N,
                                         int64_t K, const void* bias, pt_stream_t stream) {
  PT_REQUIRE(bias, "gemm_m_grouped_nt_bias: null bias");
  return gemm_m_grouped_impl(a_fp8, a_scale, b_fp8, b_scale, out, out_dtype, offs, G, M, N, K, nullptr, 0, bias, stream);
}

static int gemm_k_grouped_wgrad_impl(const void* dy_t_fp8, const float* dy_scale, int64_t ld_dy_scale, const void* x_t_fp8,
                                     const float* x_scale, int64_t ld_x_scale, void* out, int out_dtype, int accumulate,
                                     const int32_t* offs, int32_t G, int64_t M, int64_t N, int64_t K, pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && N >= 0 && K >= 0 && G > 0, "gemm_k_grouped_wgrad: bad sizes");
  if (N == 0 || K == 0) return PT_OK;
  PT_REQUIRE(M % 128 == 0, "gemm_k_grouped_wgrad: M=%lld must be a multiple of 128", (long long)M);
  PT_REQUIRE(out && offs, "gemm_k_grouped_wgrad: null pointer");
  PT_REQUIRE(M == 0 || (dy_t_fp8 && dy_scale && x_t_fp8 && x_scale && al16(dy_t_fp8) && al16(x_t_fp8)),
             "gemm_k_grouped_wgrad: null or misaligned pointer");
  PT_REQUIRE(out_dtype == PT_BF16 || out_dtype == PT_F32, "gemm_k_grouped_wgrad: out_dtype must be bf16 or fp32");
  PT_REQUIRE(ld_dy_scale >= N && ld_x_scale >= K, "gemm_k_grouped_wgrad: scale row length smaller than the row count");
  GemmArgs g = {};
  g.a = (const uint8_t*)dy_t_fp8; g.lda = M; g.b = (const uint8_t*)x_t_fp8; g.ldb = M;
  g.sa = dy_scale; g.sa_rs = 1; g.sa_ks = ld_dy_scale; g.sa_shift = 0;
  g.sb = x_scale; g.sb_rs = 1; g.sb_ks = ld_x_scale; g.sb_shift = 0;
  g.out = out; g.ldo = K; g.out_dtype = out_dtype; g.accumulate = accumulate;
  g.rows_a = N; g.rows_b = K; g.red = M; g.mode = GEMM_K_GROUPED; g.offs = offs; g.G = G;
  g.out_stride_g = N * K;
  g.a_bytes = N * M; g.b_bytes = K * M;
  g.sa_bytes = ((M / 128 - 1) * ld_dy_scale + N) * 4; g.sb_bytes = ((M / 128 - 1) * ld_x_scale + K) * 4;
  g.tiles_a = (int)cdiv(N, 128); g.tiles_b = (int)cdiv(K, 128);
  g.total_tiles = (int64_t)g.tiles_a * g.tiles_b * G;
  return dispatch_gemm(g, (hipStream_t)stream);
}

extern "C" int pt_gemm_k_grouped_wgrad(const void* dy_t_fp8, const float* dy_scale, const void* x_t_fp8, const float* x_scale,
                                       void* out, int out_dtype, int accumulate, const int32_t* offs, int32_t G, int64_t M,
                                       int64_t N, int64_t K, pt_stream_t stream) {
  return gemm_k_grouped_wgrad_impl(dy_t_fp8, dy_scale, N, x_t_fp8, x_scale, K, out, out_dtype, accumulate, offs, G, M, N, K, stream);
}

extern "C" int pt_gemm_k_grouped_wgrad_ld(const void* dy_t_fp8, const float* dy_scale, int64_t ld_dy_scale, const void* x_t_fp8,
                                          const float* x_scale, int64_t ld_x_scale, void* out, int out_dtype, int accumulate,
                                          const int32_t* offs, int32_t G, int64_t M, int64_t N, int64_t K, pt_stream_t stream) {
  return gemm_k_grouped_wgrad_impl(dy_t_fp8, dy_scale, ld_dy_scale, x_t_fp8, x_scale, ld_x_scale, out, out_dtype, accumulate,
                                   offs, G, M, N, K, stream);
}
