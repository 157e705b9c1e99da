// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/pithtrain_hip.h"

namespace pt {

// ---- error reporting -------------------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

#define PT_REQUIRE(cond, ...)                \
  do {                                       \
    if (!(cond)) {                           \
      pt::set_error(__VA_ARGS__);            \
      return PT_ERR_INVALID;                 \
    }                                        \
  } while (0)

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- element conversion ------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

// fp32 -> bf16 round-to-nearest-even (NaN kept quiet) with the hardware conversion
// (v_cvt_pk_bf16_f32): one instruction per pair, and bit-identical to the integer sequence
// u += 0x7FFF + ((u >> 16) & 1); u >>= 16 for all 2^32 inputs (checked exhaustively on MI355X).
typedef __bf16 pt_bf16x2 __attribute__((ext_vector_type(2)));
typedef float pt_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const pt_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, pt_bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, 0.f) & 0xFFFFu; }

__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}
// The conversion is an opaque instruction on purpose: written as a cast, the compiler folds a
// preceding fp32 multiply into v_fma_mixlo_f16 (one rounding instead of fp32-then-fp16), which
// makes the result depend on how each kernel happens to be scheduled.
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  uint32_t r;
  asm("v_cvt_f16_f32_e32 %0, %1" : "=v"(r) : "v"(f));
  return r & 0xFFFFu;
}

// ---- SwiGLU arithmetic shared by the epilogue kernels and the fused activation + quantisation ----
__device__ __forceinline__ float sigmoidf_fast(float x) {
  return __builtin_amdgcn_rcpf(__fadd_rn(1.0f, __expf(-x)));
}

// The arithmetic is spelled with explicit round-to-nearest operations so that every kernel that
// uses it (flat and row-strided) produces the same bits whatever the compiler would contract.
__device__ __forceinline__ float silu_mul_f(float g, float u) {
  return __fmul_rn(__fmul_rn(g, sigmoidf_fast(g)), u);
}
__device__ __forceinline__ void silu_mul_b(float d, float g, float u, float& dg, float& du) {
  const float sig = sigmoidf_fast(g);
  const float silu = __fmul_rn(g, sig);
  du = __fmul_rn(d, silu);
  dg = __fmul_rn(__fmul_rn(__fmul_rn(d, u), sig), __fsub_rn(__fadd_rn(1.0f, g), silu));
}

// Clamped SwiGLU on one (gate, up) pair: (clamp(u, -L, L) + 1) * gc * sigmoid(alpha * gc) with
// gc = min(g, L); the backward masks each gradient where its input was clamped.
__device__ __forceinline__ float cswiglu_f(float g, float u, float alpha, float limit) {
  const float gc = fminf(g, limit);
  const float uc = fminf(fmaxf(u, -limit), limit);
  return __fmul_rn(__fadd_rn(uc, 1.0f), __fmul_rn(gc, sigmoidf_fast(__fmul_rn(alpha, gc))));
}
__device__ __forceinline__ void cswiglu_b(float d, float g, float u, float alpha, float limit, float& dg, float& du) {
  const float gc = fminf(g, limit);
  const float uc = fminf(fmaxf(u, -limit), limit);
  const float ag = __fmul_rn(alpha, gc);
  const float sig = sigmoidf_fast(ag);
  const float grad_uc = __fmul_rn(d, __fmul_rn(gc, sig));
  const float grad_gc = __fmul_rn(__fmul_rn(__fmul_rn(d, __fadd_rn(uc, 1.0f)), sig),
                                  __fadd_rn(1.0f, __fmul_rn(ag, __fsub_rn(1.0f, sig))));
  dg = (g <= limit) ? grad_gc : 0.0f;
  du = (u >= -limit && u <= limit) ? grad_uc : 0.0f;
}

// ---- storage types: 8-wide vector and scalar load/store with fp32 math ---------------------------
struct st_bf16 {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ void load8(const void* p, float* v) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    v[0] = bf16_lo(u.x); v[1] = bf16_hi(u.x); v[2] = bf16_lo(u.y); v[3] = bf16_hi(u.y);
    v[4] = bf16_lo(u.z); v[5] = bf16_hi(u.z); v[6] = bf16_lo(u.w); v[7] = bf16_hi(u.w);
  }
  static __device__ __forceinline__ void store8(void* p, const float* v) {
    uint4 u;
    u.x = pack_bf16x2(v[0], v[1]); u.y = pack_bf16x2(v[2], v[3]);
    u.z = pack_bf16x2(v[4], v[5]); u.w = pack_bf16x2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = u;
  }
  static __device__ __forceinline__ float load1(const void* p) { return bf16_bits_to_f32(*(const uint16_t*)p); }
  static __device__ __forceinline__ void store1(void* p, float v) { *(uint16_t*)p = (uint16_t)f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }  // to the storage type and back
};
struct st_f16 {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ void load8(const void* p, float* v) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[2 * i] = f16_bits_to_f32(w[i] & 0xFFFF); v[2 * i + 1] = f16_bits_to_f32(w[i] >> 16); }
  }
  static __device__ __forceinline__ void store8(void* p, const float* v) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = f32_to_f16_bits(v[2 * i]) | (f32_to_f16_bits(v[2 * i + 1]) << 16);
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  static __device__ __forceinline__ float load1(const void* p) { return f16_bits_to_f32(*(const uint16_t*)p); }
  static __device__ __forceinline__ void store1(void* p, float v) { *(uint16_t*)p = (uint16_t)f32_to_f16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }
};
struct st_f32 {
  static constexpr int kBytes = 4;
  static __device__ __forceinline__ void load8(const void* p, float* v) {
    const float4 a = ((const float4*)p)[0], b = ((const float4*)p)[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store8(void* p, const float* v) {
    ((float4*)p)[0] = make_float4(v[0], v[1], v[2], v[3]);
    ((float4*)p)[1] = make_float4(v[4], v[5], v[6], v[7]);
  }
  static __device__ __forceinline__ float load1(const void* p) { return *(const float*)p; }
  static __device__ __forceinline__ void store1(void* p, float v) { *(float*)p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};

// The same 8-wide accesses with the non-temporal cache policy (data that is touched once and is
// larger than the caches); NT = false is the plain access, so kernels can take the policy as a
// compile-time switch.
typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
template <typename S, bool NT>
__device__ __forceinline__ void load8_policy(const void* p, float* v) {
  if constexpr (!NT) {
    S::load8(p, v);
  } else if constexpr (S::kBytes == 2) {
    const nt_u4 q = __builtin_nontemporal_load(reinterpret_cast<const nt_u4*>(p));
    S::load8(&q, v);
  } else {
    nt_u4 q[2];
    q[0] = __builtin_nontemporal_load(reinterpret_cast<const nt_u4*>(p));
    q[1] = __builtin_nontemporal_load(reinterpret_cast<const nt_u4*>(p) + 1);
    S::load8(q, v);
  }
}
template <typename S, bool NT>
__device__ __forceinline__ void store8_policy(void* p, const float* v) {
  if constexpr (!NT) {
    S::store8(p, v);
  } else if constexpr (S::kBytes == 2) {
    nt_u4 q;
    S::store8(&q, v);
    __builtin_nontemporal_store(q, reinterpret_cast<nt_u4*>(p));
  } else {
    nt_u4 q[2];
    S::store8(q, v);
    __builtin_nontemporal_store(q[0], reinterpret_cast<nt_u4*>(p));
    __builtin_nontemporal_store(q[1], reinterpret_cast<nt_u4*>(p) + 1);
  }
}

// ---- FP8 scale rule ------------------------------------------------------------------------
// scale = 2^ceil(log2(max(amax,1e-4) * fl32(1/448))), clamped to 2^-126; rcp by exponent flip.
__device__ __forceinline__ float fp8_scale_from_amax(float amax, float& rcp) {
  const float s_in = fmaxf(amax, 1e-4f) * (1.0f / 448.0f);
  const uint32_t bits = __float_as_uint(s_in);
  uint32_t e = bits & 0x7F800000u;
  if (bits & 0x007FFFFFu) e += 0x00800000u;
  float s = __uint_as_float(e);
  s = fmaxf(s, 1.17549435e-38f);  // 2^-126
  rcp = __uint_as_float((254u << 23) - __float_as_uint(s));
  return s;
}

// two / four floats -> packed OCP e4m3fn bytes (round-to-nearest-even on gfx950)
__device__ __forceinline__ uint32_t cvt4_e4m3(float a, float b, float c, float d) {
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  return (uint32_t)r;
}

// ---- 16-lane (DPP row) max all-reduce ---------------------------------------------------------
__device__ __forceinline__ float row16_allmax(float v) {
  int x = __float_as_int(v);
  int y;
  y = __builtin_amdgcn_update_dpp(x, x, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
  v = fmaxf(v, __int_as_float(y)); x = __float_as_int(v);
  y = __builtin_amdgcn_update_dpp(x, x, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
  v = fmaxf(v, __int_as_float(y)); x = __float_as_int(v);
  y = __builtin_amdgcn_update_dpp(x, x, 0x141, 0xF, 0xF, false);  // row_half_mirror
  v = fmaxf(v, __int_as_float(y)); x = __float_as_int(v);
  y = __builtin_amdgcn_update_dpp(x, x, 0x140, 0xF, 0xF, false);  // row_mirror
  v = fmaxf(v, __int_as_float(y));
  return v;
}

}  // namespace pt
