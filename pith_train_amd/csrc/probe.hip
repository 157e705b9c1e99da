// Measurement aid: the rate the matrix pipe sustains when nothing else limits it.  Every wave
// issues back-to-back v_mfma_scale_f32_32x32x64_f8f6f4 on eight independent accumulators held in
// registers; no memory traffic.  The benchmark times it with events and reports the rate next to
// the published peak, because the clock the part holds under this load is below the nominal one.
#include "common.h"

namespace pt {

typedef int probe_v8i __attribute__((ext_vector_type(8)));
typedef float probe_v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_rate_probe_kernel(float* sink, int iters) {
  probe_v8i a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    // e4m3 bytes 0x30..0x3F (0.5 .. 1.875), varying by lane and register: finite sums, live operand bits
    a[i] = 0x30303030 + (((int)threadIdx.x * 0x01030507 + i * 0x02040608) & 0x0F0F0F0F);
    b[i] = 0x30303030 + (((int)threadIdx.x * 0x07050301 + i * 0x08060402) & 0x0F0F0F0F);
  }
  probe_v16f acc[8];
#pragma unroll
  for (int n = 0; n < 8; ++n)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[n][v] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 8; ++n) acc[n] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[n], 0, 0, 0, 127, 0, 127);
  }
  float s = 0.f;
#pragma unroll
  for (int n = 0; n < 8; ++n)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[n][v];
  sink[(int64_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace pt

using namespace pt;

extern "C" int pt_probe_mfma_rate(int32_t blocks, int32_t iters, float* sink, double* flop, pt_stream_t stream) {
  PT_REQUIRE(blocks >= 1 && blocks <= 65536 && iters >= 1 && sink && flop, "probe_mfma_rate: bad arguments");
  hipLaunchKernelGGL(mfma_rate_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, sink, iters);
  // 32 x 32 x 64 multiply-adds per instruction, eight per iteration, four waves per workgroup
  *flop = 2.0 * 32 * 32 * 64 * 8.0 * (double)iters * 4.0 * (double)blocks;
  return check_launch("mfma_rate_probe_kernel");
}
