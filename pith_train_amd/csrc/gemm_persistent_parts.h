// Parts shared by the two persistent FP8 GEMM kernels (two-phase and software-pipelined main
// loops): buffer descriptors and direct-to-LDS loads, the work list (group scan, tile geometry),
// the result stores, and the launch of one workgroup per CU.
#pragma once
#include "common.h"
#include "gemm_args.h"
#include <stdlib.h>

namespace pt {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

static constexpr int kMaxGroupsGemm = 2048;
#ifdef PT_GEMM_ABLATE_STORES
static constexpr bool kAblateStores = true;
#else
static constexpr bool kAblateStores = false;
#endif
static constexpr uint32_t kOob = 0x80000000u;  // per-lane offset that is out of range for every descriptor used here
// Cache-policy bits of the wide result stores (buffer instruction aux operand: 1 = sc0, 2 = nt,
// 16 = sc1), for the weight-gradient mode and for the others.  Non-temporal by default: a GEMM
// launched alone runs the same either way, but inside a training step the results (the weight
// gradients above all: 1.2 GB per step for a 128-expert layer, read by nobody soon) otherwise
// push the next kernels' operands out of the memory-side cache.  Measured on the Qwen3-30B-A3B
// step: weight gradients only -1.7 %, all modes -2.2 %, all but the weight gradients -0.3 %.
#ifndef PT_GEMM_STORE_AUX_WGRAD
#define PT_GEMM_STORE_AUX_WGRAD 2
#endif
#ifndef PT_GEMM_STORE_AUX
#define PT_GEMM_STORE_AUX 2
#endif
template <int MODE> static constexpr int kStoreAux = MODE == GEMM_K_GROUPED ? PT_GEMM_STORE_AUX_WGRAD : PT_GEMM_STORE_AUX;
static constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format

// Raw buffer descriptor over [base, base + bytes) for the inline-assembly loads.
__device__ __forceinline__ v4i make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t a = (uint64_t)(uintptr_t)base;
  v4i r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xFFFF));
  r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  r[3] = kRsrcFlags;
  return r;
}

// Direct-to-LDS buffer loads: address = base + voff (per lane) + soff (uniform); lane l's data lands
// at lds_off + 16*l (dwordx4) or lds_off + 4*l (dword).  lds_off is a wave-uniform LDS byte address.
// (PT_GEMM_LOAD_A_MOD / PT_GEMM_LOAD_B_MOD, measurement builds: cache-policy modifiers, e.g. " nt", of
// the row-split kernel's a and b operand loads.)
#ifndef PT_GEMM_LOAD_A_MOD
#define PT_GEMM_LOAD_A_MOD ""
#endif
#ifndef PT_GEMM_LOAD_B_MOD
#define PT_GEMM_LOAD_B_MOD ""
#endif
__device__ __forceinline__ void dma16(v4i rsrc, uint32_t voff, uint32_t soff, uint32_t lds_off) {
  soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);  // uniform by construction; pin them to SGPRs
  lds_off = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_off);
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voff), "s"(rsrc), "s"(soff),
               "s"(lds_off)
               : "memory");
}
template <int OPERAND>  // 0: a, 1: b
__device__ __forceinline__ void dma16_op(v4i rsrc, uint32_t voff, uint32_t soff, uint32_t lds_off) {
  soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
  lds_off = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_off);
  if (OPERAND == 0)
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen" PT_GEMM_LOAD_A_MOD " lds" ::"v"(voff), "s"(rsrc),
                 "s"(soff), "s"(lds_off)
                 : "memory");
  else
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen" PT_GEMM_LOAD_B_MOD " lds" ::"v"(voff), "s"(rsrc),
                 "s"(soff), "s"(lds_off)
                 : "memory");
}
__device__ __forceinline__ void dma4(v4i rsrc, uint32_t voff, uint32_t soff, uint32_t lds_off) {
  soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
  lds_off = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_off);
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dword %0, %1, %2 offen lds" ::"v"(voff), "s"(rsrc), "s"(soff),
               "s"(lds_off)
               : "memory");
}
__device__ __forceinline__ void wait_all_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  const bf16x2 h = __builtin_convertvector(f32x2{lo, hi}, bf16x2);
  return __builtin_bit_cast(uint32_t, h);
}

// ---- epilogue of one 32x32 accumulator tile.  The lane holds column (lane&31) and rows
// 8*(v/4) + 4*(lane>>5) + (v&3).  voff is the lane's byte offset inside the tile (kOob if its
// column is out of range); soff the uniform byte offset of the tile's row 0, column 0; pitch the
// row pitch in bytes. ----
__device__ __forceinline__ void store_f32(const v16f& a, __amdgpu_buffer_rsrc_t out, uint32_t voff, uint32_t soff,
                                          uint32_t pitch, bool accumulate) {
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const uint32_t s = soff + (8 * (v >> 2) + (v & 3)) * pitch;
    float x = a[v];
    if (accumulate) x += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(out, voff, s, 0));
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, x), out, voff, s, 0);
  }
}
// bf16: lanes 2c and 2c+1 trade one value of each register pair so that each stores two adjacent
// columns of one row as a dword (the odd lane writes one row below the even lane; voff already
// says so).  Needs an even row pitch in elements.
__device__ __forceinline__ void store_pairs_bf16(const v16f& a, __amdgpu_buffer_rsrc_t out, uint32_t voff, uint32_t soff,
                                                 uint32_t pitch, bool accumulate, bool odd) {
#pragma unroll
  for (int v = 0; v < 16; v += 2) {
    const float x0 = a[v], x1 = a[v + 1];
    const float send = odd ? x0 : x1;
    const float recv = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send), 0xB1, 0xF, 0xF, false));
    const uint32_t s = soff + (8 * (v >> 2) + (v & 3)) * pitch;
    // round the GEMM result to bf16 first, then add: the two roundings of `grad += wgrad.to(bf16)`
    uint32_t w = odd ? pack2_bf16(recv, x1) : pack2_bf16(x0, recv);
    if (accumulate) {
      const uint32_t old = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(out, voff, s, 0);
      w = pack2_bf16(bf16_lo(old) + bf16_lo(w), bf16_hi(old) + bf16_hi(w));
    }
    __builtin_amdgcn_raw_buffer_store_b32((int)w, out, voff, s, 0);
  }
}
// bf16 through a per-wave LDS staging tile: the accumulator layout (a lane owns one column) is
// turned into rows so that every lane stores 16 contiguous bytes.  Two horizontally adjacent
// 32x32 blocks (64 columns: one 128-byte line per row) go through the 2 KiB tile 16 rows at a
// time, and each store instruction then writes 8 whole 128-byte lines.  (Half lines - one block,
// 16 rows x 64 B per instruction - cost a tenth of the dense and a quarter of the weight-gradient
// GEMM's time in the write path; the memory pipeline spends the same time on a 4-byte and on a
// 16-byte store instruction, which is why the stores are wide in the first place.)  Only this wave
// touches its staging tile, and the LDS executes one wave's operations in order, so the phases
// need compiler fences only.
// voff[q]: the lane's byte offset for tile rows 8q + lane/8, q = 0..3 (row start + 16-byte chunk
// lane%8, or kOob); soff: uniform byte offset added to all of them.
// bias (with has_bias): the 8 values of the lane's columns, added in the output type after the
// result has been rounded to it (x + bias[group] as a second operation on the rounded x).
template <int AUX = 0>
__device__ __forceinline__ void store_staged_bf16_lines(const v16f& a0, const v16f& a1, __amdgpu_buffer_rsrc_t out, uint8_t* stg,
                                                        const uint32_t (&voff)[4], uint32_t soff, bool accumulate, int lane,
                                                        bool has_bias = false, v4i bias = v4i{0, 0, 0, 0}) {
  const bool odd = lane & 1;
  uint8_t* wr = stg + (4 * (lane >> 5) + (odd ? 1 : 0)) * 128 + ((lane & 31) >> 1) * 4;
  const uint8_t* rd = stg + (lane >> 3) * 128 + (lane & 7) * 16;
  // p = (row r | row r+1) of the lane's column; the even lane of a pair takes both low halves (row r,
  // columns c and c+1), the odd lane both high halves (row r+1): one byte permute of own and neighbour
  const uint32_t sel = odd ? 0x03020706u : 0x05040100u;
#ifdef PT_GEMM_ABLATE_STAGING
  // measurement build: the stores carry raw accumulator bits, no conversion and no staging
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const v16f& a = hf ? a1 : a0;
      v4i w = v4i{__float_as_int(a[8 * h]), __float_as_int(a[8 * h + 1]), __float_as_int(a[8 * h + 2]), __float_as_int(a[8 * h + 3])};
      __builtin_amdgcn_raw_buffer_store_b128(w, out, voff[2 * hf + h], soff, AUX);
      asm volatile("s_nop 4" ::"v"(w) : "memory");
    }
  return;
#endif
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {  // tile rows 0-15, then 16-31
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const v16f& a = b ? a1 : a0;
#pragma unroll
      for (int v = 8 * hf; v < 8 * hf + 8; v += 2) {
        const uint32_t pk = pack2_bf16(a[v], a[v + 1]);
        const uint32_t nb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)pk, 0xB1, 0xF, 0xF, false);
        *(uint32_t*)(wr + (8 * ((v >> 2) & 1) + (v & 3)) * 128 + b * 64) = __builtin_amdgcn_perm(nb, pk, sel);
      }
    }
    asm volatile("" ::: "memory");  // the reads below alias the writes above
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      v4i w = *(const v4i*)(rd + h * 1024);
      const uint32_t vo = voff[2 * hf + h];
      if (has_bias) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          w[q] = (int)pack2_bf16(bf16_lo((uint32_t)w[q]) + bf16_lo((uint32_t)bias[q]), bf16_hi((uint32_t)w[q]) + bf16_hi((uint32_t)bias[q]));
      }
      if (accumulate) {
        const v4i old = __builtin_amdgcn_raw_buffer_load_b128(out, vo, soff, 0);
#pragma unroll
        for (int q = 0; q < 4; ++q)
          w[q] = (int)pack2_bf16(bf16_lo((uint32_t)old[q]) + bf16_lo((uint32_t)w[q]), bf16_hi((uint32_t)old[q]) + bf16_hi((uint32_t)w[q]));
      }
      __builtin_amdgcn_raw_buffer_store_b128(w, out, vo, soff, AUX);
      // A 16-byte store reads its data registers for a few cycles after it issues; the compiler
      // only guards that window for stores without a scalar offset, so hold the registers here.
      asm volatile("s_nop 4" ::"v"(w) : "memory");
    }
    asm volatile("" ::: "memory");  // the next half's writes alias these reads
  }
}

__device__ __forceinline__ void store_single_bf16(const v16f& a, __amdgpu_buffer_rsrc_t out, uint32_t voff, uint32_t soff,
                                                  uint32_t pitch, bool accumulate) {
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const uint32_t s = soff + (8 * (v >> 2) + (v & 3)) * pitch;
    uint32_t r = f32_to_bf16_bits(a[v]);
    if (accumulate) {
      const uint32_t old = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(out, voff, s, 0);
      r = f32_to_bf16_bits(bf16_bits_to_f32(old) + bf16_bits_to_f32(r));
    }
    __builtin_amdgcn_raw_buffer_store_b16((short)r, out, voff, s, 0);
  }
}

// One tile of the work list; everything is wave-uniform (SGPRs).
struct Tile {
  int a_row0, b_row0, a_lim, b_lim, k_begin, k_len, kb0, g;
};

// Scaled MFMA whose scale bytes are byte `ia` of sa and byte `ib` of sb (byte index = op_sel bit +
// 2 * op_sel_hi bit, one pair per operand).  Issued as volatile inline assembly with a memory
// clobber: the compiler keeps such statements, and every memory operation between them, in source
// order, which is what pins the interleaving of MFMAs, LDS reads and direct-to-LDS loads in the
// main loop.  AGPR: the accumulator lives in the accumulation registers ("a" constraint), which a
// wave with 256 accumulator values needs; with 128 it lives in ordinary registers ("v"), where the
// epilogue reads it without a copy and shares one register pool with everything else.
template <bool AGPR>
__device__ __forceinline__ void mfma_sel(const v8i& a, const v8i& b, v16f& c, int ia, int sa, int ib, int sb) {
#define PT_MFMA_TEXT(S0, S1, H0, H1) \
  "v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[" #S0 "," #S1 ",0] op_sel_hi:[" #H0 "," #H1 ",0]"
#define PT_MFMA(IA, IB, S0, S1, H0, H1)                                                                                  \
  case IA * 4 + IB:                                                                                                      \
    if constexpr (AGPR) asm volatile(PT_MFMA_TEXT(S0, S1, H0, H1) : "+a"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb) : "memory"); \
    else asm volatile(PT_MFMA_TEXT(S0, S1, H0, H1) : "+v"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb) : "memory");               \
    break;
  switch (ia * 4 + ib) {
    PT_MFMA(0, 0, 0, 0, 0, 0) PT_MFMA(0, 1, 0, 1, 0, 0) PT_MFMA(0, 2, 0, 0, 0, 1) PT_MFMA(0, 3, 0, 1, 0, 1)
    PT_MFMA(1, 0, 1, 0, 0, 0) PT_MFMA(1, 1, 1, 1, 0, 0) PT_MFMA(1, 2, 1, 0, 0, 1) PT_MFMA(1, 3, 1, 1, 0, 1)
    PT_MFMA(2, 0, 0, 0, 1, 0) PT_MFMA(2, 1, 0, 1, 1, 0) PT_MFMA(2, 2, 0, 0, 1, 1) PT_MFMA(2, 3, 0, 1, 1, 1)
    PT_MFMA(3, 0, 1, 0, 1, 0) PT_MFMA(3, 1, 1, 1, 1, 0) PT_MFMA(3, 2, 1, 0, 1, 1) PT_MFMA(3, 3, 1, 1, 1, 1)
  }
#undef PT_MFMA
#undef PT_MFMA_TEXT
}

// s_pref[g] = sum of weight(g') over groups g' < g (s_pref[G] = the total, s_pref[G + 1] = the largest
// weight); computed by the first wave, followed by a workgroup barrier.
template <class E, class W>
__device__ __forceinline__ void scan_groups(const GemmArgs& p, int* s_pref, int tid, int lane, E end_of, W weight) {
  if (tid < 64) {
    // Lane l owns groups [l * per, (l + 1) * per): one global read per group, running sums kept in
    // LDS, then the lanes' totals are scanned and added to each lane's own entries.
    const int per = (p.G + 63) / 64;
    const int g0 = tid * per;
    int sum = 0, mx = 0;
    if (per <= 4) {
      // up to 256 groups: the lane's five group ends are requested together (one memory latency)
      const int last = p.G - 1;
      int e[5];
#pragma unroll
      for (int q = 0; q < 5; ++q) {
        int g = g0 - 1 + q;
        g = g < 0 ? 0 : (g > last ? last : g);
        e[q] = end_of(g);
      }
      if (g0 == 0) e[0] = 0;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int g = g0 + q;
        if (q < per && g < p.G) {
          const int w = weight(e[q + 1] - e[q]);
          sum += w;
          mx = w > mx ? w : mx;
          s_pref[g + 1] = sum;
        }
      }
    } else {
      int prev = (g0 > 0 && g0 <= p.G) ? end_of(g0 - 1) : 0;
      for (int q = 0; q < per; ++q) {
        const int g = g0 + q;
        if (g < p.G) {
          const int cur = end_of(g);
          const int w = weight(cur - prev);
          sum += w;
          mx = w > mx ? w : mx;
          prev = cur;
          s_pref[g + 1] = sum;
        }
      }
    }
    int incl = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int y = __shfl_up(incl, d);
      if (lane >= d) incl += y;
    }
    const int base = incl - sum;
    for (int q = 0; q < per; ++q) {
      const int g = g0 + q;
      if (g < p.G) s_pref[g + 1] += base;
    }
    if (tid == 0) s_pref[0] = 0;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int y = __shfl_xor(mx, d);
      mx = y > mx ? y : mx;
    }
    if (tid == 0) s_pref[p.G + 1] = mx;  // the largest weight, after the total
  }
  __syncthreads();
}

// m-grouped: s_pref[g] = number of BM-row tiles of groups < g, from the cumulative group ends.
template <int BM>
__device__ __forceinline__ void scan_group_tiles(const GemmArgs& p, int* s_pref, int tid, int lane) {
  scan_groups(p, s_pref, tid, lane, [&](int g) { return p.offs[g]; }, [](int rows) { return (rows + BM - 1) / BM; });
}

// k-grouped: a tile of group g costs its number of 128-deep reduction blocks plus a fixed share
// for the tile switch and the result store; s_pref[g] = that cost summed over groups < g.
static constexpr int kTileFixedCost = 3;
__device__ __forceinline__ int k_group_tile_cost(int rows) { return ((rows + 127) >> 7) + kTileFixedCost; }
__device__ __forceinline__ void scan_group_costs(const GemmArgs& p, int* s_pref, int tid, int lane) {
  scan_groups(p, s_pref, tid, lane, [&](int g) { return k_group_end(p, g); }, [](int rows) { return k_group_tile_cost(rows); });
}

// First logical tile of XCD `x` (x in [0, 8]; x = 8 gives the end of the list).  Dense and
// m-grouped tiles all cost the same, so the list is cut into eight equal counts.  k-grouped tiles
// cost in proportion to their group's row count: the list (group-major) is cut where the summed
// cost reaches x/8 of the total, so that skewed group sizes do not leave most XCDs idle while one
// works through the large groups.  Cuts are rounded to multiples of `round`, the number of
// workgroups per XCD.
template <int MODE>
__device__ __forceinline__ int xcd_first_tile(const GemmArgs& p, const int* s_pref, int total_tiles, int x, int round) {
  // Groups of nearly equal cost (largest within a quarter of the mean): the plain cut by count, which
  // for a group count that is a multiple of eight also keeps whole groups on one XCD.
  const bool by_count = MODE != GEMM_K_GROUPED || (int64_t)s_pref[p.G + 1] * p.G * 4 <= (int64_t)s_pref[p.G] * 5;
  if (by_count) {
    const int per_xcd = (total_tiles + 7) / 8;
    const int t = x * per_xcd;
    return t < total_tiles ? t : total_tiles;
  }
  if (x <= 0) return 0;
  if (x >= 8) return total_tiles;
  const int per_g = p.tiles_a * p.tiles_b;
  const int64_t pos = (int64_t)s_pref[p.G] * per_g * x / 8;
  int lo = 0, hi = p.G - 1;  // last g with s_pref[g] * per_g <= pos
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int64_t)s_pref[mid] * per_g <= pos) lo = mid; else hi = mid - 1;
  }
  const int cost = s_pref[lo + 1] - s_pref[lo];
  int idx = (int)((pos - (int64_t)s_pref[lo] * per_g) / cost);
  if (idx > per_g) idx = per_g;
  // whole rounds of the XCD's workgroups: a cut a few tiles past a multiple of `round` would
  // leave most of them idle during one more round
  const int t = (lo * per_g + idx + (round >> 1)) / round * round;
  return t < total_tiles ? t : total_tiles;
}

// Geometry of logical tile t; plain per-lane arithmetic (every lane may ask for a different t).
template <int MODE, int BM, int BN>
__device__ __forceinline__ void decode_tile(const GemmArgs& p, const int* s_pref, int t, Tile& T) {
  // The 32 CUs of an XCD work on 32 consecutive logical tiles at a time.  The b-tiles are cut into
  // strips of at most 8 (of nearly equal width), and a strip is walked row by row: 32 consecutive
  // tiles then share 32 / w a-tiles and w b-tiles in that XCD's L2 (4 and 8 for a full strip)
  // instead of 32 a-tiles and 1 b-tile, whatever the number of b-tiles is.
  auto blocked = [&](int t, int& ta, int& tb) {
    const int ns = (p.tiles_b + 7) >> 3;           // strips
    const int w0 = p.tiles_b / ns, wide = p.tiles_b - w0 * ns;  // the first `wide` strips have w0 + 1 b-tiles
    const int per_wide = p.tiles_a * (w0 + 1);
    int s, r, w, b0;
    if (t < wide * per_wide) { s = t / per_wide; r = t - s * per_wide; w = w0 + 1; b0 = s * w; }
    else { const int t2 = t - wide * per_wide; s = t2 / (p.tiles_a * w0); r = t2 - s * p.tiles_a * w0; w = w0; b0 = wide * (w0 + 1) + s * w0; }
    ta = r / w;
    tb = b0 + r - ta * w;
  };
  if (MODE == GEMM_DENSE) {
    T.g = 0;
    int ta, tb;
    blocked(t, ta, tb);
    T.a_row0 = ta * BM; T.b_row0 = tb * BN;
    T.a_lim = (int)p.rows_a; T.b_lim = (int)p.rows_b; T.k_begin = 0; T.k_len = (int)p.red; T.kb0 = 0;
  } else if (MODE == GEMM_M_GROUPED) {
    const int q = t / p.tiles_b;
    int lo = 1, hi = p.G;  // first j in [1, G] with s_pref[j] > q
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (s_pref[mid] > q) hi = mid; else lo = mid + 1;
    }
    const int g = lo - 1;
    const int pg = s_pref[g], pg1 = s_pref[g + 1];
    const int gs = g ? p.offs[g - 1] : 0;
    const int m_tiles = pg1 - pg;
    const int idx = t - pg * p.tiles_b;
    T.g = g;
    T.a_row0 = gs + (idx % m_tiles) * BM; T.b_row0 = (idx / m_tiles) * BN;
    T.a_lim = p.offs[g]; T.b_lim = (int)p.rows_b; T.k_begin = 0; T.k_len = (int)p.red; T.kb0 = 0;
  } else {
    const int per_g = p.tiles_a * p.tiles_b;
    const int g = t / per_g;
    const int idx = t % per_g;
    T.g = g;
    int ta = idx % p.tiles_a, tb = idx / p.tiles_a;
    if (!p.offs) blocked(idx, ta, tb);  // split-K of a dense product: the dense order inside every range
    T.a_row0 = ta * BM; T.b_row0 = tb * BN;
    T.a_lim = (int)p.rows_a; T.b_lim = (int)p.rows_b;
    T.k_begin = g ? k_group_end(p, g - 1) : 0; T.k_len = k_group_end(p, g) - T.k_begin; T.kb0 = T.k_begin >> 7;
  }
}

// Hands one accumulator block produced by inline-assembly MFMAs to the compiler: PIN 1 = it lives
// in the accumulation registers, 2 = in ordinary registers, 0 = the compiler produced it itself.
template <int PIN>
__device__ __forceinline__ void pin_acc(v16f& a) {
  if constexpr (PIN == 1) asm volatile("" : "+a"(a));
  else if constexpr (PIN == 2) asm volatile("" : "+v"(a));
}

// Writes one wave's TM x TN blocks of 32 x 32 results of tile T (rows wm0.., columns wn0.. of the
// tile).  `stg` is the wave's 2 KiB LDS staging area.  PIN != 0: the accumulators were produced by
// inline-assembly MFMAs; each block is handed to the compiler only right before its store, so
// that it is converted and copied out one block at a time.
template <int MODE, int TM, int TN, bool ACC, int PIN>
__device__ __forceinline__ void store_tile(v16f (&acc)[TM][TN], const GemmArgs& p, const Tile& T, int wm0, int wn0, int lane,
                                           uint8_t* stg) {
  const uint32_t esz = p.out_dtype == PT_F32 ? 4 : 2;
  const uint32_t pitch = (uint32_t)p.ldo * esz;
  const bool pair_ok = p.out_dtype != PT_F32 && (p.ldo & 1) == 0 && (((uintptr_t)p.out) & 3) == 0;
  const bool wide_ok = p.out_dtype != PT_F32 && (p.ldo & 7) == 0 && (((uintptr_t)p.out) & 15) == 0 &&
                       (MODE != GEMM_K_GROUPED || (p.out_stride_g & 7) == 0);
  // The descriptor ends after the tile's last valid row: stores to ragged rows are dropped.
  // (PT_GEMM_ABLATE_STORES, measurement builds only: it ends before the first, so every store
  // instruction runs and nothing is written.)
  char* outp = (char*)p.out + (MODE == GEMM_K_GROUPED ? (int64_t)T.g * p.out_stride_g * esz : 0);
  const __amdgpu_buffer_rsrc_t rs_out = __builtin_amdgcn_make_buffer_rsrc(outp, 0, kAblateStores ? 0 : (int)((uint32_t)T.a_lim * pitch), kRsrcFlags);
  const uint32_t s_tile = (uint32_t)(T.a_row0 + wm0) * pitch + (uint32_t)(T.b_row0 + wn0) * esz;
  const int colw = T.b_row0 + wn0 + (lane & 31);
  static_assert(TN % 2 == 0, "the wide stores take column blocks in pairs");
  if (MODE == GEMM_M_GROUPED && p.out_row_index) {
    // Result row r goes to output row out_row_index[r] (the un-permute folded into the store);
    // rows of the group's padding map to a negative index and are dropped.
    const __amdgpu_buffer_rsrc_t rs_sc = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, kAblateStores ? 0 : (int)((uint32_t)p.out_rows * pitch), kRsrcFlags);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      // one index load for the block row (lane -> row lane%32), handed to the lanes that store the row
      const int r = T.a_row0 + wm0 + i * 32 + (lane & 31);
      const int dst_of_lane = r < T.a_lim ? p.out_row_index[r] : -1;
      uint32_t vrow[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int dst = __shfl(dst_of_lane, q * 8 + (lane >> 3));
        vrow[q] = dst >= 0 ? (uint32_t)dst * pitch + (uint32_t)(lane & 7) * 16 : kOob;
      }
#pragma unroll
      for (int j = 0; j < TN; j += 2) {
        const int colc = T.b_row0 + wn0 + j * 32 + (lane & 7) * 8;
        uint32_t voff[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) voff[q] = colc < T.b_lim ? vrow[q] : kOob;
        v4i bias = v4i{0, 0, 0, 0};
        if (p.bias != nullptr && colc < T.b_lim) bias = *(const v4i*)((const char*)p.bias + ((int64_t)T.g * p.rows_b + colc) * 2);
        pin_acc<PIN>(acc[i][j]); pin_acc<PIN>(acc[i][j + 1]);
        store_staged_bf16_lines<kStoreAux<MODE>>(acc[i][j], acc[i][j + 1], rs_sc, stg, voff, (uint32_t)(T.b_row0 + wn0 + j * 32) * 2, false, lane,
                                p.bias != nullptr, bias);
      }
    }
  } else if (p.out_dtype != PT_F32 && wide_ok && (T.b_lim & 7) == 0) {
    const bool has_bias = MODE == GEMM_M_GROUPED && p.bias != nullptr;
#pragma unroll
    for (int j = 0; j < TN; j += 2) {
      const int colc = T.b_row0 + wn0 + j * 32 + (lane & 7) * 8;
      v4i bias = v4i{0, 0, 0, 0};
      if (has_bias && colc < T.b_lim) bias = *(const v4i*)((const char*)p.bias + ((int64_t)T.g * p.rows_b + colc) * 2);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        uint32_t voff[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          voff[q] = colc < T.b_lim ? (uint32_t)(q * 8 + (lane >> 3)) * pitch + (uint32_t)(lane & 7) * 16 : kOob;
        pin_acc<PIN>(acc[i][j]); pin_acc<PIN>(acc[i][j + 1]);
        store_staged_bf16_lines<kStoreAux<MODE>>(acc[i][j], acc[i][j + 1], rs_out, stg, voff, s_tile + i * 32 * pitch + j * 64, ACC, lane, has_bias, bias);
      }
    }
  } else if (p.out_dtype != PT_F32 && pair_ok && (T.b_lim & 1) == 0) {
    const bool odd = lane & 1;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t voff = colw + j * 32 < T.b_lim ? (uint32_t)(4 * (lane >> 5) + odd) * pitch + (uint32_t)(((lane & 31) & ~1) + j * 32) * 2 : kOob;
#pragma unroll
      for (int i = 0; i < TM; ++i) { pin_acc<PIN>(acc[i][j]); store_pairs_bf16(acc[i][j], rs_out, voff, s_tile + i * 32 * pitch, pitch, ACC, odd); }
    }
  } else if (p.out_dtype == PT_F32) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t voff = colw + j * 32 < T.b_lim ? (uint32_t)(4 * (lane >> 5)) * pitch + (uint32_t)((lane & 31) + j * 32) * 4 : kOob;
#pragma unroll
      for (int i = 0; i < TM; ++i) { pin_acc<PIN>(acc[i][j]); store_f32(acc[i][j], rs_out, voff, s_tile + i * 32 * pitch, pitch, ACC); }
    }
  } else {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t voff = colw + j * 32 < T.b_lim ? (uint32_t)(4 * (lane >> 5)) * pitch + (uint32_t)((lane & 31) + j * 32) * 2 : kOob;
#pragma unroll
      for (int i = 0; i < TM; ++i) { pin_acc<PIN>(acc[i][j]); store_single_bf16(acc[i][j], rs_out, voff, s_tile + i * 32 * pitch, pitch, ACC); }
    }
  }
}

// One workgroup per CU (fewer when there are fewer tiles), in multiples of the 8 XCDs.  `upper` is
// an upper bound of the number of tiles.
template <class Kernel>
static int launch_persistent_grid(Kernel kernel, const char* name, const GemmArgs& a, int64_t upper, int threads, size_t lds,
                                  bool& attr_set, hipStream_t stream) {
  static int num_cus = 0;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_error("gemm: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return PT_ERR_LAUNCH; }
    attr_set = true;
  }
  if (num_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    num_cus = n;
  }
  if (upper == 0) return PT_OK;
  PT_REQUIRE(upper < (1ll << 30), "gemm: too many tiles");
  int64_t blocks = (num_cus + 7) / 8 * 8;
  if (upper < blocks) blocks = (upper + 7) / 8 * 8;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(threads), lds, stream, a);
  return check_launch(name);
}

// Fills the tile counts of `a` for BM x BN tiles and returns an upper bound of the number of tiles
// (exact except in the m-grouped mode, where the kernel counts them from the group sizes).
static inline int64_t plan_tiles(GemmArgs& a, int BM, int BN) {
  a.tiles_a = (int)cdiv(a.rows_a, BM);
  a.tiles_b = (int)cdiv(a.rows_b, BN);
  if (a.mode == GEMM_DENSE) return a.total_tiles = (int64_t)a.tiles_a * a.tiles_b;
  if (a.mode == GEMM_K_GROUPED) return a.total_tiles = (int64_t)a.tiles_a * a.tiles_b * a.G;
  return ((a.rows_a / 128 + a.G) / 2 + 1) * a.tiles_b;
}

}  // namespace pt
