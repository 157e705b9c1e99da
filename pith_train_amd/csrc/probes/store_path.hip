// Probe of the write path on gfx950 (not part of the library): how the rate at which compute
// units can write result tiles depends on how many XCDs and how many CUs per XCD write at once.
// One workgroup per CU (256 launched; workgroup b runs on XCD b % 8), eight waves each, every
// wave-store writes 8 rows x 128 bytes (the shape of the GEMM's result stores: 16 bytes per lane,
// row pitch 4096 bytes).  Active workgroups write 4 MiB each, the others return at once.
// A last section keeps all 256 CUs writing and varies the shape of a wave-store (R rows x 1024/R
// bytes) and the order of a workgroup's wave-stores (down the rows of one column chunk first, or
// along a row first).  Prints GB/s per active CU and in total.
// Build: hipcc -O3 --offload-arch=gfx950 store_path.hip -o store_path
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
typedef int v4i __attribute__((ext_vector_type(4)));
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1); } } while (0)

__global__ __launch_bounds__(512, 1) void store_kernel(uint8_t* buf, int xcds, int cus_per_xcd, int reps, int waves, int mib = 4) {
  if ((int)(blockIdx.x & 7) >= xcds || (int)(blockIdx.x >> 3) >= cus_per_xcd) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave >= waves) return;
  uint8_t* base = buf + (size_t)blockIdx.x * ((size_t)mib << 20);
  const uint32_t pitch = 4096;  // 256 * mib rows x 4096 bytes per workgroup
  const v4i val = v4i{lane, wave, 3, 4};
  const int rg_bits = 31 - __builtin_clz(32 * mib);  // mib is a power of two
  for (int r = 0; r < reps; ++r)
    for (int q = wave; q < (32 << rg_bits); q += waves) {  // row groups of 8 rows x 32 column chunks of 128 bytes
      const int rg = q & ((1 << rg_bits) - 1), c = q >> rg_bits;
      *(v4i*)(base + (size_t)(rg * 8 + (lane >> 3)) * pitch + c * 128 + (lane & 7) * 16) = val;
    }
}

// Wave-stores of `rows` rows x (1024 / rows) bytes; along_row != 0 walks the chunks of a row group
// before the next row group, so the eight waves of a workgroup write neighbouring chunks.
__global__ __launch_bounds__(512, 1) void store_shape_kernel(uint8_t* buf, int reps, int rows, int along_row, int skew) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // skew: workgroup regions start 4 MiB + skew bytes apart instead of exactly 4 MiB
  uint8_t* base = buf + (size_t)blockIdx.x * ((4u << 20) + (uint32_t)skew);
  const uint32_t pitch = 4096;
  const int width = 1024 / rows;           // bytes of a row that one wave-store covers
  const int lanes_per_row = width / 16;
  const int row_groups = 1024 / rows, chunks = 4096 / width;
  const v4i val = v4i{lane, wave, 3, 4};
  for (int r = 0; r < reps; ++r)
    for (int q = wave; q < row_groups * chunks; q += 8) {
      const int rg = along_row ? q / chunks : q % row_groups;
      const int c = along_row ? q % chunks : q / row_groups;
      *(v4i*)(base + (size_t)(rg * rows + lane / lanes_per_row) * pitch + c * width + (lane % lanes_per_row) * 16) = val;
    }
}

int main() {
  uint8_t* buf; CHECK(hipMalloc(&buf, (size_t)3 << 29));
  hipEvent_t a, b; CHECK(hipEventCreate(&a)); CHECK(hipEventCreate(&b));
  for (int xcds : {1, 2, 4, 8})
    for (int cus : {1, 4, 8, 16, 32}) {
      const int reps = 4;
      store_kernel<<<256, 512>>>(buf, xcds, cus, 1, 8);
      CHECK(hipEventRecord(a));
      store_kernel<<<256, 512>>>(buf, xcds, cus, reps, 8);
      CHECK(hipEventRecord(b)); CHECK(hipEventSynchronize(b));
      float ms; CHECK(hipEventElapsedTime(&ms, a, b));
      const double bytes = (double)xcds * cus * reps * (4u << 20);
      printf("XCDs %d x CUs %2d: %6.1f GB/s per CU, %5.2f TB/s in total\n", xcds, cus, bytes / (ms * 1e-3) / 1e9 / (xcds * cus), bytes / (ms * 1e-3) / 1e12);
      fflush(stdout);
    }
  // all 256 CUs, fewer waves of each writing (the same bytes per CU)
  for (int waves : {1, 2, 4, 8}) {
    const int reps = 4;
    store_kernel<<<256, 512>>>(buf, 8, 32, 1, waves);
    CHECK(hipEventRecord(a));
    store_kernel<<<256, 512>>>(buf, 8, 32, reps, waves);
    CHECK(hipEventRecord(b)); CHECK(hipEventSynchronize(b));
    float ms; CHECK(hipEventElapsedTime(&ms, a, b));
    const double bytes = 256.0 * reps * (4u << 20);
    printf("256 CUs, %d writing wave(s) each: %6.1f GB/s per CU, %5.2f TB/s in total\n", waves, bytes / (ms * 1e-3) / 1e9 / 256, bytes / (ms * 1e-3) / 1e12);
  }
  // 64 CUs again, with 16 MiB each: 1 GiB written per pass, more than the memory-side cache holds
  {
    const int reps = 2;
    store_kernel<<<256, 512>>>(buf, 8, 8, 1, 8, 16);
    CHECK(hipEventRecord(a));
    store_kernel<<<256, 512>>>(buf, 8, 8, reps, 8, 16);
    CHECK(hipEventRecord(b)); CHECK(hipEventSynchronize(b));
    float ms; CHECK(hipEventElapsedTime(&ms, a, b));
    const double bytes = 64.0 * reps * (16u << 20);
    printf("XCDs 8 x CUs  8, 16 MiB each: %6.1f GB/s per CU, %5.2f TB/s in total\n", bytes / (ms * 1e-3) / 1e9 / 64, bytes / (ms * 1e-3) / 1e12);
  }
  for (int skew : {0, 4096, 37 * 256, 1 << 20})
   for (int along : {0, 1})
    for (int rows : {8, 4, 2, 1}) {
      if (skew && (rows == 4 || rows == 2)) continue;
      const int reps = 4;
      store_shape_kernel<<<256, 512>>>(buf, 1, rows, along, skew);
      CHECK(hipEventRecord(a));
      store_shape_kernel<<<256, 512>>>(buf, reps, rows, along, skew);
      CHECK(hipEventRecord(b)); CHECK(hipEventSynchronize(b));
      float ms; CHECK(hipEventElapsedTime(&ms, a, b));
      const double bytes = 256.0 * reps * (4u << 20);
      printf("256 CUs, regions 4 MiB + %7d bytes apart, wave-stores of %d rows x %4d bytes, %s: %6.1f GB/s per CU, %5.2f TB/s in total\n", skew, rows, 1024 / rows,
             along ? "along a row first  " : "down the rows first", bytes / (ms * 1e-3) / 1e9 / 256, bytes / (ms * 1e-3) / 1e12);
    }
  return 0;
}
