// Blockwise FP8 quantisation kernels for gfx950.
//
// One workgroup (256 threads, 4 wavefronts) owns one 128x128 tile of the source: it is read
// once with 16-byte loads, reduced three ways (per row, per column, whole tile) and written as
// up to two e4m3 tensors plus their power-of-two scales.  Thread t holds the 8x8 sub-block at
// rows (t/16)*8.., columns (t%16)*8.. so that a 16-lane DPP row covers one 128-column row
// segment (row amax is a DPP all-reduce) and one thread owns 8 consecutive rows of each of its
// columns (so transposed bytes can be packed straight from registers).  Transposed twins go
// through an XOR-swizzled LDS tile so that global stores are 16 bytes wide and 128-byte
// contiguous per 8 lanes.  The kernel is HBM-bound: 2 (or 4) bytes in, 2 bytes out per element.
#include "common.h"
#include <type_traits>

// Cache policy of the streaming accesses (bits; the default is what measured best inside the
// training step, the others are measurement builds: make EXTRA=-DPT_QUANT_NT=<bits>):
//   1  non-temporal loads in the weight kernels (128x128-scaled)     4  their stores
//   2  non-temporal loads in the activation kernels (row-scaled)      8  their stores
//   16 non-temporal stores of the activation kernels' transposed twin only
//   32 non-temporal loads in the fused SwiGLU prologues
// Weights are read once per step and their FP8 form (0.6 GB for a 128-expert layer) is larger
// than the memory-side cache, so keeping either in the caches only evicts what the next GEMM
// needs: 1 + 4 take 1.5 % off the Qwen3-30B-A3B step.  gate_up and grad_h are read once by the
// SwiGLU prologues: 32 takes another 0.6 %.  Activation outputs are the next GEMM's operands and
// want to stay in the memory-side cache: 8 or 16 make the step 0.5-2 % slower although the
// kernels themselves, timed alone back to back, get up to 24 % faster.
#ifndef PT_QUANT_NT
#define PT_QUANT_NT (1 + 4 + 32)
#endif
// rows of the paired SwiGLU-backward prologue whose loads are in flight at a time
#ifndef PT_QUANT_PAIR_ROWS
#define PT_QUANT_PAIR_ROWS 2
#endif

namespace pt {

typedef uint32_t q_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t q_u2 __attribute__((ext_vector_type(2)));
template <bool W> __device__ __forceinline__ uint4 q_load16(const void* p) {
  if (PT_QUANT_NT & (W ? 1 : 2)) { const q_u4 v = __builtin_nontemporal_load(reinterpret_cast<const q_u4*>(p)); return make_uint4(v.x, v.y, v.z, v.w); }
  return *reinterpret_cast<const uint4*>(p);
}
// the loads of the fused SwiGLU prologues (bit 32)
__device__ __forceinline__ void q_load8_pro(const void* p, float* v) {
  uint4 u;
  if (PT_QUANT_NT & 32) { const q_u4 t = __builtin_nontemporal_load(reinterpret_cast<const q_u4*>(p)); u = make_uint4(t.x, t.y, t.z, t.w); }
  else u = *reinterpret_cast<const uint4*>(p);
  v[0] = bf16_lo(u.x); v[1] = bf16_hi(u.x); v[2] = bf16_lo(u.y); v[3] = bf16_hi(u.y);
  v[4] = bf16_lo(u.z); v[5] = bf16_hi(u.z); v[6] = bf16_lo(u.w); v[7] = bf16_hi(u.w);
}
template <bool W> __device__ __forceinline__ void q_store8(void* p, uint32_t lo, uint32_t hi) {
  if (PT_QUANT_NT & (W ? 4 : 8)) { __builtin_nontemporal_store(q_u2{lo, hi}, reinterpret_cast<q_u2*>(p)); return; }
  *reinterpret_cast<uint2*>(p) = make_uint2(lo, hi);
}
template <bool W> __device__ __forceinline__ void q_store16(void* p, uint4 v) {  // the transposed twin
  if (PT_QUANT_NT & (W ? 4 : 8 + 16)) { __builtin_nontemporal_store(q_u4{v.x, v.y, v.z, v.w}, reinterpret_cast<q_u4*>(p)); return; }
  *reinterpret_cast<uint4*>(p) = v;
}

enum { A_ROW = 0, A_BLOCK = 1 };                       // scaling of the same-orientation output
enum { B_COL = 0, B_BLOCK = 1 };                       // scaling of the twin
enum { BL_ROWMAJOR = 0, BL_TRANSPOSED = 1, BL_KMAJOR = 2, BL_NONE = 3 };  // layout of the twin's bytes (BL_NONE: no twin is written)
enum { BS_MB_N = 0, BS_N_MB = 1 };                     // twin scale layout for B_COL

struct QuantArgs {
  const void* x;
  int64_t M, N, ldx, x_stride_g;
  uint8_t* a_out;  int64_t a_stride_g;   // [M,N] bytes, ld = N
  float* a_scale;  int64_t a_scale_stride_g;
  uint8_t* b_out;  int64_t b_stride_g;   // rowmajor [M,N] / transposed [N,M] / kmajor flat
  float* b_scale;  int64_t b_scale_stride_g;
  int32_t tiles_m, tiles_n;
  const int32_t* offs; int32_t num_groups;  // KMAJOR only
  int32_t vec_in;     // 16-byte loads legal (alignment + N % 8 == 0)
  int32_t vec_out;    // 8-byte row-major stores legal (N % 8 == 0)
  int32_t vec_out_t;  // 16-byte transposed stores legal
  const int32_t* row_index;  // optional [M]: source row of output row r (negative: a zero row); null = identity
  const void* x2; int64_t ldx2;  // fused SwiGLU backward: the saved gate_up [M, 2*half]
  int64_t half;                  // fused SwiGLU: width of one half of gate_up
  const int32_t* row_limit;      // optional device scalar: row tiles at or past *row_limit are skipped (nothing written)
  int64_t ld_t;                  // row pitch of the transposed twin (bytes = elements); M unless it is a column slice
  int64_t bs_ld;                 // row length of the twin's block-scale grid; tiles_m unless it is a column slice
  float alpha, limit;            // fused clamped SwiGLU: its two constants
  float* col_sum;                // fused clamped SwiGLU backward: [tiles_m, N] column sums of each 128-row tile
};

template <typename T> struct Loader;
struct bf16_tag {};
template <> struct Loader<bf16_tag> {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ void load8(const void* p, float* v) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    v[0] = bf16_lo(u.x); v[1] = bf16_hi(u.x); v[2] = bf16_lo(u.y); v[3] = bf16_hi(u.y);
    v[4] = bf16_lo(u.z); v[5] = bf16_hi(u.z); v[6] = bf16_lo(u.w); v[7] = bf16_hi(u.w);
  }
  static __device__ __forceinline__ float load1(const void* p) {
    return bf16_bits_to_f32(*reinterpret_cast<const uint16_t*>(p));
  }
};
struct f16_tag {};
template <> struct Loader<f16_tag> {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ void load8(const void* p, float* v) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    v[0] = f16_bits_to_f32(u.x & 0xFFFFu); v[1] = f16_bits_to_f32(u.x >> 16); v[2] = f16_bits_to_f32(u.y & 0xFFFFu);
    v[3] = f16_bits_to_f32(u.y >> 16); v[4] = f16_bits_to_f32(u.z & 0xFFFFu); v[5] = f16_bits_to_f32(u.z >> 16);
    v[6] = f16_bits_to_f32(u.w & 0xFFFFu); v[7] = f16_bits_to_f32(u.w >> 16);
  }
  static __device__ __forceinline__ float load1(const void* p) {
    return f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(p));
  }
};
template <> struct Loader<float> {
  static constexpr int kBytes = 4;
  static __device__ __forceinline__ void load8(const void* p, float* v) {
    const float4 a = reinterpret_cast<const float4*>(p)[0];
    const float4 b = reinterpret_cast<const float4*>(p)[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ float load1(const void* p) {
    return *reinterpret_cast<const float*>(p);
  }
};

// The thread's 8x8 sub-block.  bf16 sources stay packed (two values per register, unpacked at
// each use): half the registers of an fp32 copy, which is what lets enough wavefronts be
// resident to keep HBM busy.
template <typename T> struct Frag;
template <> struct Frag<bf16_tag> {
  uint32_t w[8][4];
  template <bool W = false> __device__ __forceinline__ void load_row(int i, const void* p) {
    const uint4 u = q_load16<W>(p);
    w[i][0] = u.x; w[i][1] = u.y; w[i][2] = u.z; w[i][3] = u.w;
  }
  __device__ __forceinline__ void zero_row(int i) { w[i][0] = w[i][1] = w[i][2] = w[i][3] = 0u; }
  __device__ __forceinline__ void set(int i, int j, const void* p) {
    const uint32_t b = *reinterpret_cast<const uint16_t*>(p);
    w[i][j >> 1] = (j & 1) ? ((w[i][j >> 1] & 0x0000FFFFu) | (b << 16)) : ((w[i][j >> 1] & 0xFFFF0000u) | b);
  }
  __device__ __forceinline__ float get(int i, int j) const { return (j & 1) ? bf16_hi(w[i][j >> 1]) : bf16_lo(w[i][j >> 1]); }
  // Compiler fence on the packed registers: values unpacked before it cannot be kept live
  // across it, so each phase of the kernel unpacks again instead of holding 64 floats.
  __device__ __forceinline__ void fence() {
#pragma unroll
    for (int i = 0; i < 8; ++i) fence_row(i);
  }
  __device__ __forceinline__ void fence_row(int i) {
#pragma unroll
    for (int k = 0; k < 4; ++k) asm volatile("" : "+v"(w[i][k]));
  }
};
// fp16 sources (the reference's quantisers take any float type): packed like bf16, unpacked with
// the half-to-float conversion; none of the packed-bf16 shortcuts apply.
template <> struct Frag<f16_tag> {
  uint32_t w[8][4];
  template <bool W = false> __device__ __forceinline__ void load_row(int i, const void* p) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    w[i][0] = u.x; w[i][1] = u.y; w[i][2] = u.z; w[i][3] = u.w;
  }
  __device__ __forceinline__ void zero_row(int i) { w[i][0] = w[i][1] = w[i][2] = w[i][3] = 0u; }
  __device__ __forceinline__ void set(int i, int j, const void* p) {
    const uint32_t b = *reinterpret_cast<const uint16_t*>(p);
    w[i][j >> 1] = (j & 1) ? ((w[i][j >> 1] & 0x0000FFFFu) | (b << 16)) : ((w[i][j >> 1] & 0xFFFF0000u) | b);
  }
  __device__ __forceinline__ float get(int i, int j) const {
    return f16_bits_to_f32((j & 1) ? (w[i][j >> 1] >> 16) : (w[i][j >> 1] & 0xFFFFu));
  }
  __device__ __forceinline__ void fence() {
#pragma unroll
    for (int i = 0; i < 8; ++i) fence_row(i);
  }
  __device__ __forceinline__ void fence_row(int i) {
#pragma unroll
    for (int k = 0; k < 4; ++k) asm volatile("" : "+v"(w[i][k]));
  }
};
template <> struct Frag<float> {
  float v[8][8];
  template <bool W = false> __device__ __forceinline__ void load_row(int i, const void* p) { Loader<float>::load8(p, v[i]); }
  __device__ __forceinline__ void zero_row(int i) {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[i][j] = 0.f;
  }
  __device__ __forceinline__ void set(int i, int j, const void* p) { v[i][j] = *reinterpret_cast<const float*>(p); }
  __device__ __forceinline__ float get(int i, int j) const { return v[i][j]; }
  __device__ __forceinline__ void fence() {}
  __device__ __forceinline__ void fence_row(int) {}
};

// what the tile is computed from
enum { PRO_NONE = 0, PRO_SILU_FWD = 1, PRO_SILU_BWD = 2, PRO_SILU_BWD_PAIR = 3, PRO_CSWIGLU_FWD = 4, PRO_CSWIGLU_BWD = 5 };

// ---- packed-bf16 arithmetic of the interior-tile path -------------------------------------------
// |x| of a bf16 is its low 15 bits, and for non-negative floats the integer order of the bits is
// the numeric order: an amax over packed pairs is one AND and one 16-bit packed integer max per two
// elements, with no unpacking.  (A NaN input compares as larger than everything here, while the
// float max of the edge-tile path skips it; the results agree for every finite and infinite input.)
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_abs(uint32_t w) { return w & 0x7FFF7FFFu; }
__device__ __forceinline__ uint32_t pk_umax(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}
// the larger half of a packed pair, as the fp32 with those bf16 bits
__device__ __forceinline__ float pk_hmax_f32(uint32_t m) {
  const uint32_t lo = m << 16, hi = m & 0xFFFF0000u;
  return __uint_as_float(lo > hi ? lo : hi);
}
// Two packed bf16 -> two e4m3 bytes of x / scale (scale a power of two, so the quotient is exact and
// equals x * (1/scale)), placed in the low or high half of `old`.  One instruction instead of two
// unpacks, two multiplies and a conversion; bit-identical to them for every bf16 value that the
// scale rule allows (|x| / scale <= 448), checked exhaustively on the hardware.
template <bool HI>
__device__ __forceinline__ uint32_t cvt2_e4m3_scaled(uint32_t old, uint32_t pair, float scale) {
  const s16x2 r = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(__builtin_bit_cast(s16x2, old), __builtin_bit_cast(bf16x2_t, pair),
                                                            scale, HI);
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t cvt4_e4m3_scaled(uint32_t p01, uint32_t p23, float scale) {
  return cvt2_e4m3_scaled<true>(cvt2_e4m3_scaled<false>(0u, p01, scale), p23, scale);
}

// One 128x128 tile.  FULL: the tile lies inside the tensor and every vector access is legal, so no
// bounds are checked; for bf16 sources it also selects the packed arithmetic above.
template <typename T, int AM, int BMODE, int BL, int BS, int PRO, bool FULL>
__device__ __forceinline__ void quant_tile_body(const QuantArgs& p, float (*s_colmax)[128], float* s_blk, uint8_t* s_t,
                                                [[maybe_unused]] float (*s_colsum)[128], const int tc, const int tr,
                                                const int64_t g) {
  constexpr bool PK = FULL && std::is_same<T, bf16_tag>::value;  // packed-bf16 arithmetic
  const int t = threadIdx.x;
  const int cc = t & 15, rg = t >> 4, wave = t >> 6, lane = t & 63;
  const int64_t row0 = (int64_t)tr * 128 + rg * 8;
  const int64_t col0 = (int64_t)tc * 128 + cc * 8;
  const char* xb = reinterpret_cast<const char*>(p.x) + g * p.x_stride_g * Loader<T>::kBytes;

  Frag<T> f;
  [[maybe_unused]] Frag<T> f_up;  // PRO_SILU_BWD_PAIR only
  if constexpr (PRO == PRO_SILU_BWD_PAIR) {
    const bool col_ok = FULL || col0 < p.half;
    // Two rows in flight: row i + 2 is addressed through a register that an empty assembly statement
    // ties to the packed results of row i.  Left alone, the compiler starts all eight rows at once
    // (24 loads and their unpacked values: the whole register file, one wave per SIMD).
    uint32_t gate[PT_QUANT_PAIR_ROWS] = {};  // always zero
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (FULL || (col_ok && row0 + i < p.M)) {
        const int64_t r = row0 + i + gate[i % PT_QUANT_PAIR_ROWS];
        float d[8], g[8], u[8], dg[8], du[8];
        q_load8_pro(xb + (r * p.ldx + col0) * 2, d);
        const char* gp = (const char*)p.x2 + (r * p.ldx2 + col0) * 2;
        q_load8_pro(gp, g);
        q_load8_pro(gp + p.half * 2, u);
#pragma unroll
        for (int j = 0; j < 8; ++j) silu_mul_b(d[j], g[j], u[j], dg[j], du[j]);
        f.w[i][0] = pack_bf16x2(dg[0], dg[1]); f.w[i][1] = pack_bf16x2(dg[2], dg[3]);
        f.w[i][2] = pack_bf16x2(dg[4], dg[5]); f.w[i][3] = pack_bf16x2(dg[6], dg[7]);
        f_up.w[i][0] = pack_bf16x2(du[0], du[1]); f_up.w[i][1] = pack_bf16x2(du[2], du[3]);
        f_up.w[i][2] = pack_bf16x2(du[4], du[5]); f_up.w[i][3] = pack_bf16x2(du[6], du[7]);
        f.fence_row(i);
        f_up.fence_row(i);
        asm volatile("" : "+v"(gate[i % PT_QUANT_PAIR_ROWS]) : "v"(f.w[i][3]), "v"(f_up.w[i][3]));
      } else {
        f.zero_row(i);
        f_up.zero_row(i);
      }
    }
  } else if constexpr (PRO == PRO_CSWIGLU_FWD) {
    // h = clamped SwiGLU of the interleaved (gate, up) pairs of gate_up = x, rounded to bf16:
    // sixteen consecutive inputs give the thread's eight outputs of a row.
    const bool col_ok = FULL || col0 < p.N;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (FULL || (col_ok && row0 + i < p.M)) {
        const char* gp = xb + ((row0 + i) * p.ldx + 2 * col0) * 2;
        float a[8], b[8], o[8];
        q_load8_pro(gp, a);
        q_load8_pro(gp + 16, b);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          o[j] = cswiglu_f(a[2 * j], a[2 * j + 1], p.alpha, p.limit);
          o[4 + j] = cswiglu_f(b[2 * j], b[2 * j + 1], p.alpha, p.limit);
        }
        f.w[i][0] = pack_bf16x2(o[0], o[1]); f.w[i][1] = pack_bf16x2(o[2], o[3]);
        f.w[i][2] = pack_bf16x2(o[4], o[5]); f.w[i][3] = pack_bf16x2(o[6], o[7]);
      } else {
        f.zero_row(i);
      }
    }
  } else if constexpr (PRO == PRO_CSWIGLU_BWD) {
    // The gradient of gate_up = x2 in its own interleaved layout, (dgate, dup) pairs rounded to
    // bf16, from grad_h = x (one column per pair): four pairs per thread and row.
    const bool col_ok = FULL || col0 < p.N;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (FULL || (col_ok && row0 + i < p.M)) {
        const int64_t r = row0 + i;
        const uint2 dw = *reinterpret_cast<const uint2*>(xb + (r * p.ldx + (col0 >> 1)) * 2);
        const float d[4] = {bf16_lo(dw.x), bf16_hi(dw.x), bf16_lo(dw.y), bf16_hi(dw.y)};
        float a[8], o[8];
        q_load8_pro((const char*)p.x2 + (r * p.ldx2 + col0) * 2, a);
#pragma unroll
        for (int j = 0; j < 4; ++j) cswiglu_b(d[j], a[2 * j], a[2 * j + 1], p.alpha, p.limit, o[2 * j], o[2 * j + 1]);
        f.w[i][0] = pack_bf16x2(o[0], o[1]); f.w[i][1] = pack_bf16x2(o[2], o[3]);
        f.w[i][2] = pack_bf16x2(o[4], o[5]); f.w[i][3] = pack_bf16x2(o[6], o[7]);
      } else {
        f.zero_row(i);
      }
    }
  } else if constexpr (PRO != PRO_NONE) {
    // The quantised tensor is the bf16-rounded SwiGLU output (forward: h = silu(gate) * up from
    // gate_up = x) or its gradient (backward: [dgate | dup] from grad_h = x and gate_up = x2),
    // computed here instead of being written to memory and read back.  bf16 only, 16-byte loads.
    const bool col_ok = FULL || col0 < p.N;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (FULL || (col_ok && row0 + i < p.M)) {
        const int64_t r = row0 + i;
        float g[8], u[8], o[8];
        if (PRO == PRO_SILU_FWD) {
          const char* gp = xb + (r * p.ldx + col0) * 2;
          q_load8_pro(gp, g);
          q_load8_pro(gp + p.half * 2, u);
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = silu_mul_f(g[j], u[j]);
        } else {
          const bool up_half = col0 >= p.half;
          const int64_t cc = col0 - (up_half ? p.half : 0);
          float d[8];
          q_load8_pro(xb + (r * p.ldx + cc) * 2, d);
          const char* gp = (const char*)p.x2 + (r * p.ldx2 + cc) * 2;
          q_load8_pro(gp, g);
          q_load8_pro(gp + p.half * 2, u);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            float dg, du;
            silu_mul_b(d[j], g[j], u[j], dg, du);
            o[j] = up_half ? du : dg;
          }
        }
        f.w[i][0] = pack_bf16x2(o[0], o[1]); f.w[i][1] = pack_bf16x2(o[2], o[3]);
        f.w[i][2] = pack_bf16x2(o[4], o[5]); f.w[i][3] = pack_bf16x2(o[6], o[7]);
      } else {
        f.zero_row(i);
      }
    }
  } else if (FULL || p.vec_in) {
    const bool col_ok = FULL || col0 < p.N;
    int32_t src[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) src[i] = 0;
    if (p.row_index) {
      if (FULL || row0 + 8 <= p.M) {  // the thread's 8 rows are consecutive: two 16-byte index loads (row0 % 8 == 0)
        const int4 lo = *reinterpret_cast<const int4*>(p.row_index + row0);
        const int4 hi = *reinterpret_cast<const int4*>(p.row_index + row0 + 4);
        src[0] = lo.x; src[1] = lo.y; src[2] = lo.z; src[3] = lo.w; src[4] = hi.x; src[5] = hi.y; src[6] = hi.z; src[7] = hi.w;
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (row0 + i < p.M) src[i] = p.row_index[row0 + i];
      }
    }
    if (FULL && !p.row_index) {
      const char* base = xb + (row0 * p.ldx + col0) * Loader<T>::kBytes;
      const int64_t pitch = p.ldx * Loader<T>::kBytes;
#pragma unroll
      for (int i = 0; i < 8; ++i) f.template load_row<AM == A_BLOCK>(i, base + i * pitch);
    } else if (FULL) {
      // Gathered rows of an interior tile: all eight loads are issued without a branch around any of
      // them (a row that does not exist reads row 0 and is zeroed afterwards); with the test in
      // front of each load the compiler waits for one row before it asks for the next.
#pragma unroll
      for (int i = 0; i < 8; ++i) f.load_row(i, xb + ((src[i] >= 0 ? (int64_t)src[i] : 0) * p.ldx + col0) * Loader<T>::kBytes);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (src[i] < 0) f.zero_row(i);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int64_t sr = p.row_index ? (int64_t)src[i] : row0 + i;
        if ((FULL || (col_ok && row0 + i < p.M)) && sr >= 0) f.load_row(i, xb + (sr * p.ldx + col0) * Loader<T>::kBytes);
        else f.zero_row(i);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      f.zero_row(i);
      int64_t sr = row0 + i;
      if (p.row_index && sr < p.M) sr = p.row_index[sr];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (row0 + i < p.M && sr >= 0 && col0 + j < p.N) f.set(i, j, xb + (sr * p.ldx + col0 + j) * Loader<T>::kBytes);
    }
  }

  // Everything after the load stage, for one 128x128 tile held in `f` at column tile `tc`.
  auto quantise_tile = [&](const int tc, const int64_t col0, Frag<T>& f) {
  // ---- reductions ------------------------------------------------------------------------
  float rowmax[8];
  if constexpr (PK) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      rowmax[i] = pk_hmax_f32(pk_umax(pk_umax(pk_abs(f.w[i][0]), pk_abs(f.w[i][1])), pk_umax(pk_abs(f.w[i][2]), pk_abs(f.w[i][3]))));
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float m = fabsf(f.get(i, 0));
#pragma unroll
      for (int j = 1; j < 8; ++j) m = fmaxf(m, fabsf(f.get(i, j)));
      rowmax[i] = m;
    }
  }
  if (AM == A_ROW) {
#pragma unroll
    for (int i = 0; i < 8; ++i) rowmax[i] = row16_allmax(rowmax[i]);
  }

  auto write_same_orientation = [&](float blk_scale, float blk_rcp) {
  f.fence();
  {
    uint8_t* ab = p.a_out + g * p.a_stride_g;
    const int64_t nb = p.tiles_n;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      f.fence_row(i);
      float rcp, s;
      if (AM == A_ROW) {
        s = fp8_scale_from_amax(rowmax[i], rcp);
        if (cc == 0 && (FULL || row0 + i < p.M)) p.a_scale[(row0 + i) * nb + tc] = s;
      } else {
        rcp = blk_rcp;
        s = blk_scale;
      }
      uint32_t lo, hi;
      if constexpr (PK) {
        lo = cvt4_e4m3_scaled(f.w[i][0], f.w[i][1], s);
        hi = cvt4_e4m3_scaled(f.w[i][2], f.w[i][3], s);
      } else {
        lo = cvt4_e4m3(f.get(i, 0) * rcp, f.get(i, 1) * rcp, f.get(i, 2) * rcp, f.get(i, 3) * rcp);
        hi = cvt4_e4m3(f.get(i, 4) * rcp, f.get(i, 5) * rcp, f.get(i, 6) * rcp, f.get(i, 7) * rcp);
      }
      if (FULL || row0 + i < p.M) {
        uint8_t* dst = ab + (row0 + i) * p.N + col0;
        if (FULL || p.vec_out) {
          if (FULL || col0 < p.N) q_store8<AM == A_BLOCK>(dst, lo, hi);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (col0 + j < p.N) dst[j] = (uint8_t)(((j < 4 ? lo : hi) >> (8 * (j & 3))) & 0xFF);
        }
      }
    }
    if (AM == A_BLOCK && t == 0)
      p.a_scale[g * p.a_scale_stride_g + (int64_t)tr * p.tiles_n + tc] = blk_scale;
  }

  };
  // Row-scaled output needs nothing from the other phases: write it now so that the row maxima
  // are dead before the column phase starts (fewer live registers, more resident waves).
  if (AM == A_ROW) write_same_orientation(0.f, 0.f);

  f.fence();
  float colmax[8];
  if (BMODE == B_COL) {
    if constexpr (PK) {
      // columns stay packed in pairs through the in-wave and the cross-wave reduction
      uint32_t* s_pair = reinterpret_cast<uint32_t*>(&s_colmax[0][0]);  // [4][64] pairs
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        uint32_t m = pk_abs(f.w[0][k]);
#pragma unroll
        for (int i = 1; i < 8; ++i) m = pk_umax(m, pk_abs(f.w[i][k]));
        m = pk_umax(m, (uint32_t)__shfl_xor((int)m, 16));
        m = pk_umax(m, (uint32_t)__shfl_xor((int)m, 32));
        if (lane < 16) s_pair[wave * 64 + cc * 4 + k] = m;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float m = fabsf(f.get(0, j));
#pragma unroll
        for (int i = 1; i < 8; ++i) m = fmaxf(m, fabsf(f.get(i, j)));
        m = fmaxf(m, __shfl_xor(m, 16));
        m = fmaxf(m, __shfl_xor(m, 32));
        colmax[j] = m;
      }
      if (lane < 16) {
#pragma unroll
        for (int j = 0; j < 8; ++j) s_colmax[wave][cc * 8 + j] = colmax[j];
      }
    }
  }
  if constexpr (PRO == PRO_CSWIGLU_BWD) {
    // Column sums of the tile's bf16 values (the bias gradient of the projection before the
    // activation is their sum over a group's tiles): rows of the thread in order, then the four
    // row groups of a wave pairwise, then the four waves after the barrier.
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float sum = f.get(0, j);
#pragma unroll
      for (int i = 1; i < 8; ++i) sum = __fadd_rn(sum, f.get(i, j));
      sum = __fadd_rn(sum, __shfl_xor(sum, 16));
      sum = __fadd_rn(sum, __shfl_xor(sum, 32));
      if (lane < 16) s_colsum[wave][cc * 8 + j] = sum;
    }
  }
  float blkmax = 0.f;
  if (AM == A_BLOCK || BMODE == B_BLOCK) {
    float m = rowmax[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) m = fmaxf(m, rowmax[i]);
    if (AM != A_ROW) m = row16_allmax(m);
    m = fmaxf(m, __shfl_xor(m, 16));
    m = fmaxf(m, __shfl_xor(m, 32));
    if (lane == 0) s_blk[wave] = m;
  }
  __syncthreads();
  if constexpr (PRO == PRO_CSWIGLU_BWD) {
    if (rg == 0) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int c = cc * 8 + j;
        if (FULL || col0 + j < p.N)
          p.col_sum[(int64_t)tr * p.N + col0 + j] =
              __fadd_rn(__fadd_rn(s_colsum[0][c], s_colsum[1][c]), __fadd_rn(s_colsum[2][c], s_colsum[3][c]));
      }
    }
  }
  if (BMODE == B_COL) {
    if constexpr (PK) {
      const uint32_t* s_pair = reinterpret_cast<const uint32_t*>(&s_colmax[0][0]);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t m = pk_umax(pk_umax(s_pair[cc * 4 + k], s_pair[64 + cc * 4 + k]),
                                   pk_umax(s_pair[128 + cc * 4 + k], s_pair[192 + cc * 4 + k]));
        colmax[2 * k] = __uint_as_float(m << 16);
        colmax[2 * k + 1] = __uint_as_float(m & 0xFFFF0000u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        colmax[j] = fmaxf(fmaxf(s_colmax[0][cc * 8 + j], s_colmax[1][cc * 8 + j]),
                          fmaxf(s_colmax[2][cc * 8 + j], s_colmax[3][cc * 8 + j]));
    }
  }
  float blk_scale = 0.f, blk_rcp = 0.f;
  if (AM == A_BLOCK || BMODE == B_BLOCK) {
    blkmax = fmaxf(fmaxf(s_blk[0], s_blk[1]), fmaxf(s_blk[2], s_blk[3]));
    blk_scale = fp8_scale_from_amax(blkmax, blk_rcp);
  }

  // ---- same-orientation output (row-scaled: already written above) ---------------------------
  if (AM != A_ROW) write_same_orientation(blk_scale, blk_rcp);
  if constexpr (BL == BL_NONE) return;

  // ---- twin ---------------------------------------------------------------------------------
  f.fence();
  float crcp[8], cs[8];
  if (BMODE == B_COL) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      cs[j] = fp8_scale_from_amax(colmax[j], crcp[j]);
      if (rg == 0 && (FULL || col0 + j < p.N)) {
        if (BS == BS_MB_N) p.b_scale[(int64_t)tr * p.N + col0 + j] = cs[j];
        else               p.b_scale[(col0 + j) * (int64_t)p.tiles_m + tr] = cs[j];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) { crcp[j] = blk_rcp; cs[j] = blk_scale; }
    if (t == 0) p.b_scale[g * p.b_scale_stride_g + (int64_t)tc * p.bs_ld + tr] = blk_scale;
  }

  if (BL == BL_ROWMAJOR) {
    uint8_t* bb = p.b_out + g * p.b_stride_g;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      f.fence_row(i);
      const uint32_t lo = cvt4_e4m3(f.get(i, 0) * crcp[0], f.get(i, 1) * crcp[1], f.get(i, 2) * crcp[2], f.get(i, 3) * crcp[3]);
      const uint32_t hi = cvt4_e4m3(f.get(i, 4) * crcp[4], f.get(i, 5) * crcp[5], f.get(i, 6) * crcp[6], f.get(i, 7) * crcp[7]);
      if (FULL || row0 + i < p.M) {
        uint8_t* dst = bb + (row0 + i) * p.N + col0;
        if (FULL || p.vec_out) {
          if (FULL || col0 < p.N) q_store8<AM == A_BLOCK>(dst, lo, hi);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (col0 + j < p.N) dst[j] = (uint8_t)(((j < 4 ? lo : hi) >> (8 * (j & 3))) & 0xFF);
        }
      }
    }
  } else {
    // pack 8 consecutive rows of each column and stage the transposed tile in LDS:
    // s_t[n][m], 16-byte chunk index XOR-swizzled with (n >> 3) & 7.
    if constexpr (PK) {
      // A byte permute puts the same column of two consecutive rows into one register pair, which
      // the scaled conversion then turns into two bytes that are already neighbours in the
      // transposed row.
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        uint32_t even[4], odd[4];  // row pairs (0,1) (2,3) (4,5) (6,7) of columns 2k and 2k+1
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          even[q] = __builtin_amdgcn_perm(f.w[2 * q + 1][k], f.w[2 * q][k], 0x05040100u);
          odd[q] = __builtin_amdgcn_perm(f.w[2 * q + 1][k], f.w[2 * q][k], 0x07060302u);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int j = 2 * k + h;
          const uint32_t* pr = h ? odd : even;
          const uint32_t lo = cvt4_e4m3_scaled(pr[0], pr[1], cs[j]);
          const uint32_t hi = cvt4_e4m3_scaled(pr[2], pr[3], cs[j]);
          const int n = cc * 8 + j;
          const int chunk = (rg >> 1) ^ ((n >> 3) & 7);
          *reinterpret_cast<uint2*>(&s_t[n * 128 + chunk * 16 + (rg & 1) * 8]) = make_uint2(lo, hi);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float r = crcp[j];
        const uint32_t lo = cvt4_e4m3(f.get(0, j) * r, f.get(1, j) * r, f.get(2, j) * r, f.get(3, j) * r);
        const uint32_t hi = cvt4_e4m3(f.get(4, j) * r, f.get(5, j) * r, f.get(6, j) * r, f.get(7, j) * r);
        const int n = cc * 8 + j;
        const int chunk = (rg >> 1) ^ ((n >> 3) & 7);
        *reinterpret_cast<uint2*>(&s_t[n * 128 + chunk * 16 + (rg & 1) * 8]) = make_uint2(lo, hi);
      }
    }
    __syncthreads();
    // destination of tile element (n, m): base + n * ld + m
    uint8_t* base;
    int64_t ld;
    if (BL == BL_TRANSPOSED) {
      base = p.b_out + g * p.b_stride_g + (int64_t)tc * 128 * p.ld_t + (int64_t)tr * 128;
      ld = p.ld_t;
    } else {
      const int64_t row_start = (int64_t)tr * 128;
      int grp = 0;
      int64_t gstart = 0;
      for (int q = 0; q < p.num_groups; ++q) {  // uniform scalar scan; groups are 128-aligned
        const int64_t e = p.offs[q];
        if (e <= row_start && q < p.num_groups - 1) { grp = q + 1; gstart = e; }
      }
      const int64_t kg = (int64_t)p.offs[grp] - gstart;
      base = p.b_out + gstart * p.N + (int64_t)tc * 128 * kg + (row_start - gstart);
      ld = kg;
    }
    const int mc = t & 7;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int n = (t >> 3) + 32 * k;
      const int64_t gn = (int64_t)tc * 128 + n;
      const int64_t gm = (int64_t)tr * 128 + mc * 16;
      if (!FULL && gn >= p.N) continue;
      const uint4 val = *reinterpret_cast<const uint4*>(&s_t[n * 128 + ((mc ^ ((n >> 3) & 7)) * 16)]);
      uint8_t* dst = base + n * ld + mc * 16;
      if (FULL || p.vec_out_t) {
        if (FULL || gm < p.M) q_store16<AM == A_BLOCK>(dst, val);
      } else {
        const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
        for (int b = 0; b < 16; ++b)
          if (gm + b < p.M) dst[b] = (uint8_t)((w[b >> 2] >> (8 * (b & 3))) & 0xFF);
      }
    }
  }
  };
  quantise_tile(tc, col0, f);
  if constexpr (PRO == PRO_SILU_BWD_PAIR) {
    __syncthreads();  // the shared staging arrays are reused by the twin
    quantise_tile(tc + p.tiles_n / 2, col0 + p.half, f_up);
  }
}

// Register budget: the kernel is bound by memory latency, so resident waves matter more than
// keeping every load of a tile in flight at once (which is what the compiler does when it is given
// the whole register file: 256 registers and one wave per SIMD for the paired SwiGLU backward).
template <typename T, int AM, int BMODE, int BL, int BS, int PRO = PRO_NONE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(PRO == PRO_SILU_BWD_PAIR ? 3 : (BL == BL_ROWMAJOR ? 5 : 6))))
void quant_tile_kernel(QuantArgs p) {
  __shared__ float s_colmax[4][128];
  __shared__ float s_blk[4];
  __shared__ __attribute__((aligned(16))) uint8_t s_t[128 * 128];
  __shared__ float s_colsum[PRO == PRO_CSWIGLU_BWD ? 4 : 1][128];

  int64_t bid = blockIdx.x;
  // PRO_SILU_BWD_PAIR: one workgroup produces the dgate tile and its dup twin (half / 128 column
  // tiles further right) from one read of grad_h, gate and up
  const int tiles_n_grid = PRO == PRO_SILU_BWD_PAIR ? p.tiles_n / 2 : p.tiles_n;
  // Row-scaled launches (one group): which XCD runs which tile decides whether the 4-byte scale
  // writes merge into whole lines.  Row scales are [M, tiles_n] floats, so the column tiles of one
  // row block write neighbouring floats; column scales in the [N, tiles_m] layout put the same
  // column of neighbouring row blocks next to each other.  Workgroup b runs on XCD b % 8: with the
  // column tile as the fastest index all of those writes would meet in eight different L2s and
  // leave as one 32-byte sector per float (8x their bytes; 12 % of the kernel's write traffic).
  // So XCD x takes octets of row blocks (octet o with o % 8 == x) and runs an octet's tiles back
  // to back, the eight row blocks of a column tile first: both kinds of neighbours are written by
  // one XCD within a few microseconds and merge in its L2.  Row blocks that do not fill eight
  // octets are dealt singly (row block r to XCD r % 8, its column tiles back to back: the row
  // scales still merge), the last tiles_m % 8 in plain order.
  int tc, tr;
  int64_t g = 0;
  const int64_t per_oct = 8 * (int64_t)tiles_n_grid;
  const int oct_rows = ((p.tiles_m >> 3) & ~7) * 8;  // row blocks in whole rounds of eight octets
  const int64_t oct_region = (int64_t)oct_rows * tiles_n_grid;
  const int64_t remapped = (int64_t)(p.tiles_m & ~7) * tiles_n_grid;
  if (AM == A_ROW && bid < oct_region) {
    const int64_t s = bid >> 3;
    const int64_t o = (s / per_oct) * 8 + (bid & 7);
    const int r = (int)(s % per_oct);
    tc = r >> 3;
    tr = (int)o * 8 + (r & 7);
  } else if (AM == A_ROW && bid < remapped) {
    const int64_t b2 = bid - oct_region, s = b2 >> 3;
    tc = (int)(s % tiles_n_grid);
    tr = oct_rows + (int)(s / tiles_n_grid) * 8 + (int)(b2 & 7);
  } else {
    tc = (int)(bid % tiles_n_grid); bid /= tiles_n_grid;
    tr = (int)(bid % p.tiles_m);
    g = bid / p.tiles_m;
  }
  // The caller may size the tensors for the largest row count a routing can produce and tell the
  // real one through device memory (no host round trip): tiles past it have nothing to do.
  if (p.row_limit && (int64_t)tr * 128 >= *p.row_limit) return;
  // interior tile with every vector access legal (uniform over the workgroup)
  const int64_t n_cols = PRO == PRO_SILU_BWD_PAIR ? p.half : p.N;
  const bool full = (int64_t)tr * 128 + 128 <= p.M && (int64_t)tc * 128 + 128 <= n_cols && p.vec_in && p.vec_out && p.vec_out_t;
  if (full) quant_tile_body<T, AM, BMODE, BL, BS, PRO, true>(p, s_colmax, s_blk, s_t, s_colsum, tc, tr, g);
  else      quant_tile_body<T, AM, BMODE, BL, BS, PRO, false>(p, s_colmax, s_blk, s_t, s_colsum, tc, tr, g);
}

template <int AM, int BMODE, int BL, int BS>
static int launch_quant(const QuantArgs& a, int dtype, int64_t G, hipStream_t stream) {
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n * G;
  if (blocks == 0) return PT_OK;
  PT_REQUIRE(blocks < (1ll << 31), "quant: grid too large (%lld tiles)", (long long)blocks);
  PT_REQUIRE(AM != A_ROW || G == 1, "quant: row-scaled launches take one group");  // the kernel's tile order relies on it
  if (dtype == PT_BF16)
    hipLaunchKernelGGL((quant_tile_kernel<bf16_tag, AM, BMODE, BL, BS>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else if (dtype == PT_F32)
    hipLaunchKernelGGL((quant_tile_kernel<float, AM, BMODE, BL, BS>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else if (dtype == PT_F16)
    hipLaunchKernelGGL((quant_tile_kernel<f16_tag, AM, BMODE, BL, BS>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else
    PT_REQUIRE(false, "quant: unsupported dtype %d (bf16, fp16 and fp32 only)", dtype);
  return check_launch("quant_tile_kernel");
}

static void fill_common(QuantArgs& a, const void* x, int dtype, int64_t M, int64_t N, int64_t ldx) {
  a.x = x; a.M = M; a.N = N; a.ldx = ldx; a.x_stride_g = 0;
  a.a_stride_g = 0; a.a_scale_stride_g = 0; a.b_stride_g = 0; a.b_scale_stride_g = 0;
  a.tiles_m = (int32_t)cdiv(M, 128); a.tiles_n = (int32_t)cdiv(N, 128);
  a.offs = nullptr; a.num_groups = 0; a.row_index = nullptr; a.x2 = nullptr; a.ldx2 = 0; a.half = 0;
  a.row_limit = nullptr; a.ld_t = M; a.bs_ld = a.tiles_m; a.alpha = 0.f; a.limit = 0.f; a.col_sum = nullptr;
  const int eb = dtype == PT_F32 ? 4 : 2;
  a.vec_in = (N % 8 == 0) && ((ldx * eb) % 16 == 0) && (((uintptr_t)x) % 16 == 0);
  a.vec_out = (N % 8 == 0);
  a.vec_out_t = (M % 16 == 0);
}

}  // namespace pt

using namespace pt;

static int quant_rowwise_colwise_impl(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx, const int32_t* row_index,
                                      void* tok_fp8, float* tok_scale, void* ch_fp8, float* ch_scale, int ch_layout,
                                      const int32_t* offs, int32_t num_groups, pt_stream_t stream);

extern "C" int pt_quant_rowwise_colwise(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                                        void* tok_fp8, float* tok_scale, void* ch_fp8,
                                        float* ch_scale, int ch_layout, const int32_t* offs,
                                        int32_t num_groups, pt_stream_t stream) {
  return quant_rowwise_colwise_impl(x, dtype, M, N, ldx, nullptr, tok_fp8, tok_scale, ch_fp8, ch_scale, ch_layout, offs,
                                    num_groups, stream);
}

extern "C" int pt_quant_rowwise_colwise_rows(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                                             const int32_t* row_index, void* tok_fp8, float* tok_scale,
                                             void* ch_fp8, float* ch_scale, int ch_layout,
                                             const int32_t* offs, int32_t num_groups, pt_stream_t stream) {
  PT_REQUIRE(row_index || M == 0, "quant_rowwise_colwise_rows: null row_index");
  return quant_rowwise_colwise_impl(x, dtype, M, N, ldx, row_index, tok_fp8, tok_scale, ch_fp8, ch_scale, ch_layout, offs,
                                    num_groups, stream);
}

static int quant_rowwise_colwise_impl(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx, const int32_t* row_index,
                                      void* tok_fp8, float* tok_scale, void* ch_fp8, float* ch_scale, int ch_layout,
                                      const int32_t* offs, int32_t num_groups, pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && N >= 0 && M % 128 == 0, "quant_rowwise_colwise: M=%lld must be a multiple of 128", (long long)M);
  PT_REQUIRE(ldx >= N, "quant_rowwise_colwise: ldx < N");
  if (M == 0 || N == 0) return PT_OK;
  PT_REQUIRE(x && tok_fp8 && tok_scale && ch_fp8 && ch_scale, "quant_rowwise_colwise: null pointer");
  QuantArgs a;
  fill_common(a, x, dtype, M, N, ldx);
  a.a_out = (uint8_t*)tok_fp8; a.a_scale = tok_scale; a.b_out = (uint8_t*)ch_fp8; a.b_scale = ch_scale;
  a.row_index = row_index;
  if (offs && num_groups > 0) a.row_limit = offs + (num_groups - 1);
  hipStream_t s = (hipStream_t)stream;
  switch (ch_layout) {
    case PT_CH_ROWMAJOR:   return launch_quant<A_ROW, B_COL, BL_ROWMAJOR, BS_MB_N>(a, dtype, 1, s);
    case PT_CH_TRANSPOSED: return launch_quant<A_ROW, B_COL, BL_TRANSPOSED, BS_MB_N>(a, dtype, 1, s);
    case PT_CH_KMAJOR:
      PT_REQUIRE(offs && num_groups > 0, "quant_rowwise_colwise: kmajor layout needs offs");
      a.offs = offs; a.num_groups = num_groups;
      return launch_quant<A_ROW, B_COL, BL_KMAJOR, BS_N_MB>(a, dtype, 1, s);
  }
  PT_REQUIRE(false, "quant_rowwise_colwise: bad ch_layout %d", ch_layout);
}

static int quant_rowwise_transpose_impl(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx, void* tok_fp8,
                                        float* tok_scale, void* t_fp8, int64_t ld_t, float* t_scale, pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && N >= 0 && ldx >= N && ld_t >= M, "quant_rowwise_transpose: bad shape");
  if (M == 0 || N == 0) return PT_OK;
  PT_REQUIRE(x && tok_fp8 && tok_scale && t_fp8 && t_scale, "quant_rowwise_transpose: null pointer");
  QuantArgs a;
  fill_common(a, x, dtype, M, N, ldx);
  a.a_out = (uint8_t*)tok_fp8; a.a_scale = tok_scale; a.b_out = (uint8_t*)t_fp8; a.b_scale = t_scale;
  a.ld_t = ld_t;
  a.vec_out_t = a.vec_out_t && ld_t % 16 == 0 && ((uintptr_t)t_fp8) % 16 == 0;
  return launch_quant<A_ROW, B_COL, BL_TRANSPOSED, BS_N_MB>(a, dtype, 1, (hipStream_t)stream);
}

extern "C" int pt_quant_rowwise_transpose(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                                          void* tok_fp8, float* tok_scale, void* t_fp8,
                                          float* t_scale, pt_stream_t stream) {
  return quant_rowwise_transpose_impl(x, dtype, M, N, ldx, tok_fp8, tok_scale, t_fp8, M, t_scale, stream);
}

extern "C" int pt_quant_rowwise_transpose_ld(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                                             void* tok_fp8, float* tok_scale, void* t_fp8, int64_t ld_t,
                                             float* t_scale, pt_stream_t stream) {
  return quant_rowwise_transpose_impl(x, dtype, M, N, ldx, tok_fp8, tok_scale, t_fp8, ld_t, t_scale, stream);
}

static int quant_rowwise_blockwise_transpose_impl(const void* x, int dtype, int64_t M, int64_t K, int64_t ldx, void* tok_fp8,
                                                  float* tok_scale, void* blk_t_fp8, int64_t ld_t, float* blk_t_scale,
                                                  pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && K >= 0 && ldx >= K && ld_t >= M, "quant_rowwise_blockwise_transpose: bad shape");
  if (M == 0 || K == 0) return PT_OK;
  PT_REQUIRE(x && tok_fp8 && tok_scale && blk_t_fp8 && blk_t_scale, "quant_rowwise_blockwise_transpose: null pointer");
  QuantArgs a;
  fill_common(a, x, dtype, M, K, ldx);
  a.a_out = (uint8_t*)tok_fp8; a.a_scale = tok_scale; a.b_out = (uint8_t*)blk_t_fp8; a.b_scale = blk_t_scale;
  a.ld_t = ld_t;
  a.vec_out_t = a.vec_out_t && ld_t % 16 == 0 && ((uintptr_t)blk_t_fp8) % 16 == 0;
  return launch_quant<A_ROW, B_BLOCK, BL_TRANSPOSED, BS_MB_N>(a, dtype, 1, (hipStream_t)stream);
}

extern "C" int pt_quant_rowwise_blockwise_transpose(const void* x, int dtype, int64_t M, int64_t K,
                                                    int64_t ldx, void* tok_fp8, float* tok_scale,
                                                    void* blk_t_fp8, float* blk_t_scale,
                                                    pt_stream_t stream) {
  return quant_rowwise_blockwise_transpose_impl(x, dtype, M, K, ldx, tok_fp8, tok_scale, blk_t_fp8, M, blk_t_scale, stream);
}

extern "C" int pt_quant_rowwise_blockwise_transpose_ld(const void* x, int dtype, int64_t M, int64_t K,
                                                       int64_t ldx, void* tok_fp8, float* tok_scale,
                                                       void* blk_t_fp8, int64_t ld_t, float* blk_t_scale,
                                                       pt_stream_t stream) {
  return quant_rowwise_blockwise_transpose_impl(x, dtype, M, K, ldx, tok_fp8, tok_scale, blk_t_fp8, ld_t, blk_t_scale, stream);
}

static int quant_blockwise_transpose_batched_impl(const void* x, int dtype, int64_t G, int64_t N, int64_t K, int64_t stride_g,
                                                  int64_t stride_row, void* fp8, int64_t fp8_stride_g, float* scale,
                                                  int64_t scale_stride_g, void* fp8_t, int64_t t_ld, int64_t t_stride_g,
                                                  float* scale_t, int64_t scale_t_ld, int64_t scale_t_stride_g,
                                                  pt_stream_t stream) {
  PT_REQUIRE(G >= 0 && N >= 0 && K >= 0 && stride_row >= K, "quant_blockwise_transpose_batched: bad shape");
  if (G == 0 || N == 0 || K == 0) return PT_OK;
  PT_REQUIRE(x && fp8 && scale && (fp8_t != nullptr) == (scale_t != nullptr), "quant_blockwise_transpose_batched: null pointer");
  QuantArgs a;
  fill_common(a, x, dtype, N, K, stride_row);
  PT_REQUIRE(fp8_stride_g >= N * K && (!fp8_t || (t_ld >= N && t_stride_g >= K * t_ld - (t_ld - N) && scale_t_ld >= a.tiles_m)),
             "quant_blockwise_transpose_batched: output strides smaller than the tensors");
  const int eb = dtype == PT_F32 ? 4 : 2;
  a.vec_in = a.vec_in && ((stride_g * eb) % 16 == 0);
  a.x_stride_g = stride_g;
  a.a_out = (uint8_t*)fp8; a.a_stride_g = fp8_stride_g; a.a_scale = scale; a.a_scale_stride_g = scale_stride_g;
  a.b_out = (uint8_t*)fp8_t; a.b_stride_g = t_stride_g; a.b_scale = scale_t; a.b_scale_stride_g = scale_t_stride_g;
  a.ld_t = t_ld; a.bs_ld = scale_t_ld;
  // 16-byte transposed stores need every row start aligned: the pitch, the group stride and the base
  a.vec_out_t = a.vec_out_t && (t_ld % 16 == 0) && (t_stride_g % 16 == 0) && (((uintptr_t)fp8_t) % 16 == 0);
  a.vec_out = a.vec_out && (fp8_stride_g % 8 == 0) && (((uintptr_t)fp8) % 8 == 0);
  if (!fp8_t) return launch_quant<A_BLOCK, B_BLOCK, BL_NONE, BS_MB_N>(a, dtype, G, (hipStream_t)stream);
  return launch_quant<A_BLOCK, B_BLOCK, BL_TRANSPOSED, BS_MB_N>(a, dtype, G, (hipStream_t)stream);
}

extern "C" int pt_quant_blockwise_transpose_batched(const void* x, int dtype, int64_t G, int64_t N,
                                                    int64_t K, int64_t stride_g, int64_t stride_row,
                                                    void* fp8, float* scale, void* fp8_t,
                                                    float* scale_t, pt_stream_t stream) {
  const int64_t nb = cdiv(N, 128), kb = cdiv(K, 128);
  return quant_blockwise_transpose_batched_impl(x, dtype, G, N, K, stride_g, stride_row, fp8, N * K, scale, nb * kb, fp8_t, N,
                                                N * K, scale_t, nb, nb * kb, stream);
}

extern "C" int pt_quant_blockwise_transpose_batched_into(const void* x, int dtype, int64_t G, int64_t N, int64_t K,
                                                         int64_t stride_g, int64_t stride_row, void* fp8,
                                                         int64_t fp8_stride_g, float* scale, int64_t scale_stride_g,
                                                         void* fp8_t, int64_t t_ld, int64_t t_stride_g, float* scale_t,
                                                         int64_t scale_t_ld, int64_t scale_t_stride_g, pt_stream_t stream) {
  return quant_blockwise_transpose_batched_impl(x, dtype, G, N, K, stride_g, stride_row, fp8, fp8_stride_g, scale,
                                                scale_stride_g, fp8_t, t_ld, t_stride_g, scale_t, scale_t_ld,
                                                scale_t_stride_g, stream);
}

// ---- SwiGLU fused into the activation quantisation --------------------------------------------
template <int PRO>
static int launch_silu_quant(const QuantArgs& a, hipStream_t stream) {
  const int64_t blocks = (int64_t)a.tiles_m * (PRO == PRO_SILU_BWD_PAIR ? a.tiles_n / 2 : a.tiles_n);
  if (blocks == 0) return PT_OK;
  PT_REQUIRE(blocks < (1ll << 31), "quant: grid too large (%lld tiles)", (long long)blocks);
  hipLaunchKernelGGL((pt::quant_tile_kernel<pt::bf16_tag, pt::A_ROW, pt::B_COL, pt::BL_TRANSPOSED, pt::BS_MB_N, PRO>),
                     dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return pt::check_launch("quant_tile_kernel(fused SwiGLU)");
}

extern "C" int pt_silu_mul_quant_rowwise_colwise(const void* gate_up, int64_t M, int64_t half, int64_t ld_gate_up,
                                                 void* tok_fp8, float* tok_scale, void* ch_t_fp8, float* ch_scale,
                                                 const int32_t* valid_rows, pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && half >= 0 && M % 128 == 0 && ld_gate_up >= 2 * half, "silu_mul_quant: bad shape");
  if (M == 0 || half == 0) return PT_OK;
  PT_REQUIRE(gate_up && tok_fp8 && tok_scale && ch_t_fp8 && ch_scale, "silu_mul_quant: null pointer");
  PT_REQUIRE(half % 8 == 0 && ld_gate_up % 8 == 0 && ((uintptr_t)gate_up) % 16 == 0,
             "silu_mul_quant: the half width and the row stride must be multiples of 8 elements, the pointer 16-byte aligned");
  QuantArgs a;
  fill_common(a, gate_up, PT_BF16, M, half, ld_gate_up);
  a.half = half; a.row_limit = valid_rows;
  a.a_out = (uint8_t*)tok_fp8; a.a_scale = tok_scale; a.b_out = (uint8_t*)ch_t_fp8; a.b_scale = ch_scale;
  return launch_silu_quant<PRO_SILU_FWD>(a, (hipStream_t)stream);
}

extern "C" int pt_silu_mul_bwd_quant_rowwise_colwise(const void* grad_h, int64_t ld_grad_h, const void* gate_up,
                                                     int64_t ld_gate_up, int64_t M, int64_t half, void* tok_fp8,
                                                     float* tok_scale, void* ch_t_fp8, float* ch_scale,
                                                     const int32_t* valid_rows, pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && half >= 0 && M % 128 == 0 && ld_gate_up >= 2 * half && ld_grad_h >= half, "silu_mul_bwd_quant: bad shape");
  if (M == 0 || half == 0) return PT_OK;
  PT_REQUIRE(grad_h && gate_up && tok_fp8 && tok_scale && ch_t_fp8 && ch_scale, "silu_mul_bwd_quant: null pointer");
  PT_REQUIRE(half % 8 == 0 && ld_gate_up % 8 == 0 && ld_grad_h % 8 == 0 && ((uintptr_t)gate_up) % 16 == 0 &&
                 ((uintptr_t)grad_h) % 16 == 0,
             "silu_mul_bwd_quant: widths and row strides must be multiples of 8 elements, pointers 16-byte aligned");
  QuantArgs a;
  fill_common(a, grad_h, PT_BF16, M, 2 * half, ld_grad_h);
  a.half = half; a.x2 = gate_up; a.ldx2 = ld_gate_up; a.row_limit = valid_rows;
  a.a_out = (uint8_t*)tok_fp8; a.a_scale = tok_scale; a.b_out = (uint8_t*)ch_t_fp8; a.b_scale = ch_scale;
  // with whole 128-column tiles per half, each workgroup makes a dgate tile and its dup twin
  if (half % 128 == 0) return launch_silu_quant<PRO_SILU_BWD_PAIR>(a, (hipStream_t)stream);
  return launch_silu_quant<PRO_SILU_BWD>(a, (hipStream_t)stream);
}

// ---- clamped SwiGLU (interleaved gate/up) fused into the activation quantisation -----------------
extern "C" int pt_clamped_swiglu_quant_rowwise_colwise(const void* gate_up, int64_t M, int64_t half, int64_t ld_gate_up,
                                                       float alpha, float limit, void* tok_fp8, float* tok_scale,
                                                       void* ch_t_fp8, float* ch_scale, const int32_t* valid_rows,
                                                       pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && half >= 0 && M % 128 == 0 && ld_gate_up >= 2 * half, "clamped_swiglu_quant: bad shape");
  if (M == 0 || half == 0) return PT_OK;
  PT_REQUIRE(gate_up && tok_fp8 && tok_scale && ch_t_fp8 && ch_scale, "clamped_swiglu_quant: null pointer");
  PT_REQUIRE(half % 8 == 0 && ld_gate_up % 8 == 0 && ((uintptr_t)gate_up) % 16 == 0,
             "clamped_swiglu_quant: the output width and the row stride must be multiples of 8 elements, the pointer 16-byte aligned");
  QuantArgs a;
  fill_common(a, gate_up, PT_BF16, M, half, ld_gate_up);
  a.half = half; a.row_limit = valid_rows; a.alpha = alpha; a.limit = limit;
  a.a_out = (uint8_t*)tok_fp8; a.a_scale = tok_scale; a.b_out = (uint8_t*)ch_t_fp8; a.b_scale = ch_scale;
  return launch_silu_quant<PRO_CSWIGLU_FWD>(a, (hipStream_t)stream);
}

extern "C" int pt_clamped_swiglu_bwd_quant_rowwise_colwise(const void* grad_h, int64_t ld_grad_h, const void* gate_up,
                                                           int64_t ld_gate_up, int64_t M, int64_t half, float alpha,
                                                           float limit, void* tok_fp8, float* tok_scale, void* ch_t_fp8,
                                                           float* ch_scale, float* col_sum, const int32_t* valid_rows,
                                                           pt_stream_t stream) {
  PT_REQUIRE(M >= 0 && half >= 0 && M % 128 == 0 && ld_gate_up >= 2 * half && ld_grad_h >= half,
             "clamped_swiglu_bwd_quant: bad shape");
  if (M == 0 || half == 0) return PT_OK;
  PT_REQUIRE(grad_h && gate_up && tok_fp8 && tok_scale && ch_t_fp8 && ch_scale && col_sum, "clamped_swiglu_bwd_quant: null pointer");
  PT_REQUIRE(half % 4 == 0 && ld_gate_up % 8 == 0 && ld_grad_h % 4 == 0 && ((uintptr_t)gate_up) % 16 == 0 &&
                 ((uintptr_t)grad_h) % 8 == 0,
             "clamped_swiglu_bwd_quant: the pair count and the gradient's row stride must be multiples of 4 elements, "
             "gate_up's row stride a multiple of 8, pointers 8- and 16-byte aligned");
  QuantArgs a;
  fill_common(a, grad_h, PT_BF16, M, 2 * half, ld_grad_h);
  a.half = half; a.x2 = gate_up; a.ldx2 = ld_gate_up; a.row_limit = valid_rows; a.alpha = alpha; a.limit = limit;
  a.col_sum = col_sum;
  a.a_out = (uint8_t*)tok_fp8; a.a_scale = tok_scale; a.b_out = (uint8_t*)ch_t_fp8; a.b_scale = ch_scale;
  return launch_silu_quant<PRO_CSWIGLU_BWD>(a, (hipStream_t)stream);
}
