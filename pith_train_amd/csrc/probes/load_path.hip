// Probe of one compute unit's vector-memory load path on gfx950 (not part of the library).
// Eight waves per workgroup, one workgroup per CU, stream 1 KiB wave-loads (8 rows x 128 bytes, the
// access shape of the GEMM's operand loads) out of a region that fits the L2 (64 KiB per workgroup)
// or out of HBM (a 1 GiB buffer walked once), with D loads per wave in flight:
//   direct-to-LDS loads, loads into registers, registers + ds_write_b128, and a mix (waves 0-3
//   direct to LDS, waves 4-7 into registers) that shows whether the two kinds share one limit.
// Prints GB/s per CU and in total for 1, 8, 64 and 256 active CUs.
// Build: hipcc -O3 --offload-arch=gfx950 load_path.hip -o load_path
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
typedef int v4i __attribute__((ext_vector_type(4)));
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1); } } while (0)
__device__ __forceinline__ v4i make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t a = (uint64_t)(uintptr_t)base;
  v4i r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xFFFF));
  r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  r[3] = 0x00020000;
  return r;
}
__device__ __forceinline__ void dma16(v4i rsrc, uint32_t voff, uint32_t soff, uint32_t lds_off) {
  soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
  lds_off = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_off);
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voff), "s"(rsrc), "s"(soff), "s"(lds_off) : "memory");
}
__device__ __forceinline__ v4i ld16(v4i rsrc, uint32_t voff, uint32_t soff) {
  soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
  v4i r;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(r) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
  return r;
}
// MODE 0: direct to LDS, 1: into registers (discarded), 2: into registers then ds_write_b128, 3: waves 0-3 as 0, waves 4-7 as 1
template <int D, int MODE>
__global__ __launch_bounds__(512, 1) void stream_kernel(const uint8_t* buf, uint32_t region_arg, uint32_t pitch, int iters, int shared, int* sink) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  uint32_t region = region_arg;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
  // shared: all workgroups of an XCD (blockIdx & 7) read the same region
  // shared == 2: every workgroup walks its own 4 MiB of the buffer once (HBM-resident data)
  // shared == 3: up to four workgroups walk 128 MiB each, starting 256 MiB into the buffer (never touched before)
  const uint8_t* base = buf + (size_t)(shared == 1 ? (blockIdx.x & 7) : blockIdx.x) * (shared == 2 ? (4u << 20) : shared == 3 ? (128u << 20) : region);
  if (shared == 2) region = 4u << 20;
  if (shared == 3) { region = 128u << 20; base += (size_t)256 << 20; }
  const v4i rs = make_rsrc(base, region);
  const uint32_t voff = (uint32_t)(lane >> 3) * pitch + (lane & 7) * 16;
  const uint32_t rows = region / pitch, cols = pitch / 128, row_groups = rows / 8;
  uint32_t n = wave;
  const uint32_t total = row_groups * cols;
  int acc = 0;
  for (int it = 0; it < iters; ++it) {
    v4i r[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const uint32_t q = n % total;
      const uint32_t rg = q % row_groups, c = q / row_groups;
      if (MODE == 0 || (MODE == 3 && wave < 4)) dma16(rs, voff, rg * 8 * pitch + c * 128, lds_base + ((wave * D + d) & 127) * 1024);
      else r[d] = ld16(rs, voff, rg * 8 * pitch + c * 128);
      n += 8;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (MODE == 1 || (MODE == 3 && wave >= 4)) {
#pragma unroll
      for (int d = 0; d < D; ++d) asm volatile("" ::"v"(r[d]));
    }
    if (MODE == 2) {
#pragma unroll
      for (int d = 0; d < D; ++d) *(v4i*)(lds + ((wave * D + d) & 127) * 1024 + lane * 16) = r[d];
    }
  }
  if (threadIdx.x == 0 && sink) sink[blockIdx.x] = lds[17] + acc;
}
template <int D, int MODE>
static double run(const uint8_t* buf, uint32_t region, uint32_t pitch, int iters, int blocks, int shared) {
  CHECK(hipFuncSetAttribute((const void*)stream_kernel<D, MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
  hipEvent_t a, b; CHECK(hipEventCreate(&a)); CHECK(hipEventCreate(&b));
  if (shared != 3) stream_kernel<D, MODE><<<blocks, 512, 128 * 1024>>>(buf, region, pitch, iters / 4 + 1, shared, nullptr);
  CHECK(hipEventRecord(a));
  stream_kernel<D, MODE><<<blocks, 512, 128 * 1024>>>(buf, region, pitch, iters, shared, nullptr);
  CHECK(hipEventRecord(b)); CHECK(hipEventSynchronize(b));
  float ms; CHECK(hipEventElapsedTime(&ms, a, b));
  return (double)iters * 8 * D * 1024 / (ms * 1e-3) / 1e9;
}
int main() {
  uint8_t* buf; CHECK(hipMalloc(&buf, (size_t)1 << 30)); CHECK(hipMemset(buf, 1, (size_t)1 << 30));
  const uint32_t pitch = 2048, region = 64u << 10;
  const int target = 64 << 20;
  const char* names[4] = {"direct-to-LDS", "to registers", "registers + ds_write", "4 waves LDS + 4 waves regs"};
  const char* where[3] = {"private 64 KiB regions (L2 hits)", "per-XCD shared 64 KiB regions (L2 hits)", "4 MiB per workgroup walked once (HBM)"};
  for (int shared = 0; shared < 3; ++shared)
    for (int blocks : {1, 8, 64, 256}) {
      printf("blocks %3d, %s:\n", blocks, where[shared]);
      const int tgt = shared == 2 ? (4 << 20) : target;
#define RUN(D, MODE) { const int iters = tgt / (8 * D * 1024); double g = run<D, MODE>(buf, region, pitch, iters, blocks, shared); printf("   %-28s D=%2d: %6.1f GB/s per CU, %5.2f TB/s\n", names[MODE], D, g, g * blocks / 1e3); fflush(stdout); }
      RUN(4, 0) RUN(8, 0) RUN(16, 0) RUN(4, 1) RUN(8, 1) RUN(16, 1) RUN(4, 2) RUN(16, 3)
    }
  // cold data: nothing of these regions is in any cache (the buffer was written once, long ago, and is four times the
  // memory-side cache); every variant walks the same region, so all but the first may find it in the memory-side cache
  for (int blocks : {1, 4}) {
    printf("blocks %3d, 128 MiB per workgroup walked once (cold):\n", blocks);
    const int shared = 3;
    const int tgt = 128 << 20;
    RUN(16, 1) RUN(16, 0) RUN(4, 1) RUN(1, 1)
  }
  return 0;
}
