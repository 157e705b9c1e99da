// Persistent FP8 GEMM for gfx950: one workgroup per CU walks a list of BM x BN output tiles.
//
//  * 256 x 256 tiles: every byte fetched from L2 feeds twice as many MFMAs as with 128 x 128
//    tiles, which is what the ~64 B/clk/CU L2 port can sustain at the FP8 rate.
//  * the group -> tile table of the m-grouped mode is built once per workgroup in LDS (ragged
//    groups: a group of n 128-row blocks gives ceil(n/2) row tiles, the last one half filled);
//    no host-side tile count and no device-to-host sync.
//  * operand tiles and their scales go global -> LDS with direct-to-LDS *buffer* loads issued from
//    inline assembly and waited for with explicit s_waitcnt, so the loads of step i+1 are in
//    flight during all MFMAs of step i.  (Issued through the compiler builtin, every later ds_read
//    of the other buffer would be made to wait for them.)  Buffer descriptors bound-check in
//    hardware: rows past a tile edge and reduction tails read as zero, and addresses are one
//    32-bit per-lane offset plus a scalar offset instead of a 64-bit pointer per load.
//  * results leave through buffer stores whose descriptor ends at the tile's last valid row, so
//    ragged rows are dropped by the hardware and the store address is again lane offset + scalar.
//  * consecutive logical tiles stay on one XCD (workgroup ids are dealt round-robin over the 8
//    XCDs, each with its own L2) and tiles that share a b-tile are adjacent.
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
static constexpr uint32_t kOob = 0x80000000u;  // per-lane offset that is out of range for every descriptor used here
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
__device__ __forceinline__ void dma16(v4i rsrc, uint32_t voff, uint32_t soff, uint32_t lds_off) {
  soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);  // uniform by construction; pin them to SGPRs
  lds_off = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_off);
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voff), "s"(rsrc), "s"(soff),
               "s"(lds_off)
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
// bf16 through a per-wave LDS staging tile (32 rows x 64 B): the accumulator layout (a lane owns
// one column) is turned into rows, so that every lane stores 16 contiguous bytes and one store
// instruction covers 16 rows x 64 B.  The memory pipeline spends the same time on a 4-byte and a
// 16-byte store instruction, so this is a quarter of the store issue time of store_pairs_bf16.
// Only this wave touches its staging tile, so a counter wait between the phases is enough.
// voff: lane's byte offset (row lane/4, 16-byte chunk lane%4) or kOob; soff: tile row 0, column 0.
__device__ __forceinline__ void store_staged_bf16(const v16f& a, __amdgpu_buffer_rsrc_t out, uint8_t* stg, uint32_t voff,
                                                  uint32_t soff, uint32_t pitch, bool accumulate, int lane) {
  const bool odd = lane & 1;
  uint8_t* wr = stg + (4 * (lane >> 5) + (odd ? 1 : 0)) * 64 + ((lane & 31) >> 1) * 4;
  // p = (row r | row r+1) of the lane's column; the even lane of a pair takes both low halves (row r,
  // columns c and c+1), the odd lane both high halves (row r+1): one byte permute of own and neighbour
  const uint32_t sel = odd ? 0x03020706u : 0x05040100u;
#pragma unroll
  for (int v = 0; v < 16; v += 2) {
    const uint32_t pk = pack2_bf16(a[v], a[v + 1]);
    const uint32_t nb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)pk, 0xB1, 0xF, 0xF, false);
    *(uint32_t*)(wr + (8 * (v >> 2) + (v & 3)) * 64) = __builtin_amdgcn_perm(nb, pk, sel);
  }
  // the reads below alias the writes above: keep the compiler from reordering them (the LDS
  // executes one wave's operations in order, so no counter wait is needed)
  asm volatile("" ::: "memory");
  const uint8_t* rd = stg + (lane >> 2) * 64 + (lane & 3) * 16;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    v4i w = *(const v4i*)(rd + h * 1024);
    const uint32_t s = soff + h * 16 * pitch;
    if (accumulate) {
      const v4i old = __builtin_amdgcn_raw_buffer_load_b128(out, voff, s, 0);
#pragma unroll
      for (int q = 0; q < 4; ++q)
        w[q] = (int)pack2_bf16(bf16_lo((uint32_t)old[q]) + bf16_lo((uint32_t)w[q]), bf16_hi((uint32_t)old[q]) + bf16_hi((uint32_t)w[q]));
    }
    __builtin_amdgcn_raw_buffer_store_b128(w, out, voff, s, 0);
    // A 16-byte store reads its data registers for a few cycles after it issues; the compiler
    // only guards that window for stores without a scalar offset, so hold the registers here.
    asm volatile("s_nop 4" ::"v"(w) : "memory");
  }
}
// As store_staged_bf16 with an arbitrary output row per lane: voff0 / voff1 are the lane's byte
// offsets (row start + 16-byte chunk, or kOob) for tile rows lane/4 and 16 + lane/4; soff the
// column offset in bytes.
__device__ __forceinline__ void store_staged_bf16_rows(const v16f& a, __amdgpu_buffer_rsrc_t out, uint8_t* stg, uint32_t voff0,
                                                       uint32_t voff1, uint32_t soff, int lane) {
  const bool odd = lane & 1;
  uint8_t* wr = stg + (4 * (lane >> 5) + (odd ? 1 : 0)) * 64 + ((lane & 31) >> 1) * 4;
  // p = (row r | row r+1) of the lane's column; the even lane of a pair takes both low halves (row r,
  // columns c and c+1), the odd lane both high halves (row r+1): one byte permute of own and neighbour
  const uint32_t sel = odd ? 0x03020706u : 0x05040100u;
#pragma unroll
  for (int v = 0; v < 16; v += 2) {
    const uint32_t pk = pack2_bf16(a[v], a[v + 1]);
    const uint32_t nb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)pk, 0xB1, 0xF, 0xF, false);
    *(uint32_t*)(wr + (8 * (v >> 2) + (v & 3)) * 64) = __builtin_amdgcn_perm(nb, pk, sel);
  }
  asm volatile("" ::: "memory");  // compiler fence only: same-wave LDS operations execute in order
  const uint8_t* rd = stg + (lane >> 2) * 64 + (lane & 3) * 16;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const v4i w = *(const v4i*)(rd + h * 1024);
    __builtin_amdgcn_raw_buffer_store_b128(w, out, h ? voff1 : voff0, soff, 0);
    asm volatile("s_nop 4" ::"v"(w) : "memory");  // see store_staged_bf16
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

template <int MODE, int BM, int BN, int WGM, int WGN, bool ACC>
__global__ __launch_bounds__(WGM * WGN * 64, 1) void fp8_gemm_nt_persistent_kernel(GemmArgs p) {
  constexpr int NW = WGM * WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int BK = 128;                      // reduction depth of one stage = one scale block = two MFMA steps
  constexpr int NS = 2;                        // stages in the LDS ring
  constexpr int STAGE = (BM + BN) * BK;
  constexpr int LA = BM / 8, LB = BN / 8;      // 1 KiB wave-loads (8 rows x 128 B: full cache lines) per operand stage
  constexpr int SLA = BM / 64, SLB = BN / 64;  // 256 B wave-loads per scale vector
  constexpr int DPW = (LA + LB) / NW;          // data loads per wave per stage
  constexpr int SPW = (SLA + SLB) / NW;        // scale loads per wave per stage
  static_assert(BM % 128 == 0 && BN % 128 == 0 && LA % NW == 0 && LB % NW == 0 && (SLA + SLB) % NW == 0 && SLA % SPW == 0,
                "every wave must issue the same number of loads per stage");
  constexpr int SC_RING = NS;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // [NS][STAGE] operand stages | [SC_RING][BM+BN] fp32 scales
  __shared__ int s_pref[MODE == GEMM_M_GROUPED ? kMaxGroupsGemm + 1 : 1];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
  const uint32_t sc_base = lds_base + NS * STAGE;
  const float* sc_lds = (const float*)(lds + NS * STAGE);

  // ---- tile list ----
  int total_tiles;
  if (MODE == GEMM_M_GROUPED) {
    // s_pref[g] = number of row tiles of groups < g
    if (tid < 64) {
      const int per = (p.G + 63) / 64;
      const int g0 = tid * per;
      int sum = 0;
      for (int q = 0; q < per; ++q) {
        const int g = g0 + q;
        if (g < p.G) sum += (p.offs[g] - (g ? p.offs[g - 1] : 0) + BM - 1) / BM;
      }
      int incl = sum;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int y = __shfl_up(incl, d);
        if (lane >= d) incl += y;
      }
      int run = incl - sum;
      for (int q = 0; q < per; ++q) {
        const int g = g0 + q;
        if (g < p.G) {
          s_pref[g] = run;
          run += (p.offs[g] - (g ? p.offs[g - 1] : 0) + BM - 1) / BM;
        }
      }
      if (tid == 63) s_pref[p.G] = incl;
    }
    __syncthreads();
    total_tiles = __builtin_amdgcn_readfirstlane(s_pref[p.G]) * p.tiles_b;
  } else {
    total_tiles = (int)p.total_tiles;
  }
  const int per_xcd = (total_tiles + 7) / 8;
  const int xcd = blockIdx.x & 7;
  int t_end = (xcd + 1) * per_xcd;
  if (t_end > total_tiles) t_end = total_tiles;
  const int t_step = gridDim.x >> 3;
  const int t_first = xcd * per_xcd + (blockIdx.x >> 3);

  // geometry of logical tile t; plain per-lane arithmetic (used by every lane for a different t
  // when the tile table is built, and uniformly beyond the table)
  auto decode_any = [&](int t, Tile& T) {
    if (MODE == GEMM_DENSE) {
      T.g = 0;
      // The 32 CUs of an XCD work on 32 consecutive logical tiles at a time; laying those out as
      // a 4 x 8 block of the output makes them share 4 a-tiles and 8 b-tiles in that XCD's L2
      // instead of 32 a-tiles and 1 b-tile.
      int ta, tb;
      const int full_a = p.tiles_a & ~3, full_b = p.tiles_b & ~7;
      const int nblk = (full_a >> 2) * (full_b >> 3);
      if (t < nblk * 32) {
        const int blk = t >> 5, in = t & 31;
        ta = (blk % (full_a >> 2)) * 4 + (in & 3);
        tb = (blk / (full_a >> 2)) * 8 + (in >> 2);
      } else {  // ragged fringe: remaining columns of tiles, then remaining rows
        const int r = t - nblk * 32;
        const int fringe_b = p.tiles_b - full_b;  // extra b-tiles, all a-tiles
        if (r < fringe_b * p.tiles_a) { ta = r % p.tiles_a; tb = full_b + r / p.tiles_a; }
        else { const int r2 = r - fringe_b * p.tiles_a; ta = full_a + r2 % (p.tiles_a - full_a); tb = r2 / (p.tiles_a - full_a); }
      }
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
      T.a_row0 = (idx % p.tiles_a) * BM; T.b_row0 = (idx / p.tiles_a) * BN;
      T.a_lim = (int)p.rows_a; T.b_lim = (int)p.rows_b;
      T.k_begin = g ? p.offs[g - 1] : 0; T.k_len = p.offs[g] - T.k_begin; T.kb0 = T.k_begin >> 7;
    }
  };

  // ---- tile table: the first kTileTable tiles of this workgroup, decoded once by as many lanes
  // in parallel; the two cursors (loader, MFMAs) then fetch a tile with one LDS read each instead
  // of redoing the group search and the integer divisions at every tile switch ----
  constexpr int kTileTable = 48;
  __shared__ __attribute__((aligned(16))) int s_tiles[kTileTable][8];
  if (tid < kTileTable) {
    const int t = t_first + tid * t_step;
    if (t < t_end) {
      Tile T;
      decode_any(t, T);
      *(int4*)&s_tiles[tid][0] = make_int4(T.a_row0, T.b_row0, T.a_lim, T.b_lim);
      *(int4*)&s_tiles[tid][4] = make_int4(T.k_begin, T.k_len, T.kb0, T.g);
    }
  }
  __syncthreads();
  // n = ordinal of the tile in this workgroup's list (t = t_first + n * t_step)
  auto decode = [&](int n, int t, Tile& T) {
    if (n < kTileTable) {
      const int4 a = *(const int4*)&s_tiles[n][0];
      const int4 b = *(const int4*)&s_tiles[n][4];
      T.a_row0 = __builtin_amdgcn_readfirstlane(a.x); T.b_row0 = __builtin_amdgcn_readfirstlane(a.y);
      T.a_lim = __builtin_amdgcn_readfirstlane(a.z); T.b_lim = __builtin_amdgcn_readfirstlane(a.w);
      T.k_begin = __builtin_amdgcn_readfirstlane(b.x); T.k_len = __builtin_amdgcn_readfirstlane(b.y);
      T.kb0 = __builtin_amdgcn_readfirstlane(b.z); T.g = __builtin_amdgcn_readfirstlane(b.w);
    } else {
      Tile U;
      decode_any(t, U);
      T.a_row0 = __builtin_amdgcn_readfirstlane(U.a_row0); T.b_row0 = __builtin_amdgcn_readfirstlane(U.b_row0);
      T.a_lim = __builtin_amdgcn_readfirstlane(U.a_lim); T.b_lim = __builtin_amdgcn_readfirstlane(U.b_lim);
      T.k_begin = __builtin_amdgcn_readfirstlane(U.k_begin); T.k_len = __builtin_amdgcn_readfirstlane(U.k_len);
      T.kb0 = __builtin_amdgcn_readfirstlane(U.kb0); T.g = __builtin_amdgcn_readfirstlane(U.g);
    }
  };

  // ---- LDS addressing ----
  // A stage holds rows of 128 bytes (8 chunks of 16).  Row r keeps logical chunk c at position
  // c ^ fs(r), fs(r) = (r&7) ^ ((r>>3)&1), which spreads the ds_read_b128 of 8 or 16 consecutive
  // rows over all banks.  Direct-to-LDS wave-load q covers rows 8q..8q+7 (1 KiB, eight full
  // 128-byte lines): lane -> row 8q + lane/8, position lane%8, i.e. logical chunk
  // (lane%8) ^ (lane/8) ^ (q&1).  A wave's loads q = w, w+NW, ... all have the parity of w, so one
  // per-lane offset serves them all and the rest of the address is uniform (scalar offset).
  const int chunk = (lane & 7) ^ (lane >> 3) ^ (wave & 1);
  const uint32_t va = (uint32_t)(lane >> 3) * (uint32_t)p.lda + chunk * 16;
  const uint32_t vb = (uint32_t)(lane >> 3) * (uint32_t)p.ldb + chunk * 16;
  const int fs_rd = (lane & 7) ^ ((lane >> 3) & 1);
  const int roff = (lane & 31) * 128;
  int coff[2][2];  // [MFMA step][half]: the lane's two chunks of a row for that step
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int h = 0; h < 2; ++h) coff[ks][h] = roff + (((ks * 4 + (lane >> 5) * 2 + h) ^ fs_rd) << 4);

  const v4i rs_a = make_rsrc(p.a, (uint32_t)p.a_bytes);
  const v4i rs_sa = make_rsrc(p.sa, (uint32_t)p.sa_bytes);
  const uint32_t esz = p.out_dtype == PT_F32 ? 4 : 2;
  const uint32_t pitch = (uint32_t)p.ldo * esz;
  const bool pair_ok = p.out_dtype != PT_F32 && (p.ldo & 1) == 0 && (((uintptr_t)p.out) & 3) == 0;
  const bool wide_ok = p.out_dtype != PT_F32 && (p.ldo & 7) == 0 && (((uintptr_t)p.out) & 15) == 0 &&
                       (MODE != GEMM_K_GROUPED || (p.out_stride_g & 7) == 0);

  // ---- loader: walks (tile, 128-block) pairs ahead of the MFMAs and keeps the LDS ring full ----
  Tile L;
  int lt = t_first - t_step, l_it = 0, l_nk = 0, n_issued = 0;
  int l_n = -1, p_n = -1, c_n = -1;  // per-cursor ordinal of the current tile in this workgroup's list
  v4i rs_b = rs_a, rs_sb = rs_sa;
  uint32_t vs[SPW];  // this wave's per-lane scale offsets (bytes) at step 0 of the loader's tile
  auto issue_stage = [&]() {
    while (l_it >= l_nk) {
      lt += t_step;
      if (lt >= t_end) return;
      decode(++l_n, lt, L);
      l_it = 0;
      l_nk = (L.k_len + 127) >> 7;
      rs_b = make_rsrc(p.b + (MODE == GEMM_M_GROUPED ? (int64_t)L.g * p.b_stride_g : 0), (uint32_t)p.b_bytes);
      rs_sb = make_rsrc(p.sb + (MODE == GEMM_M_GROUPED ? (int64_t)L.g * p.sb_stride_g : 0), (uint32_t)p.sb_bytes);
#pragma unroll
      for (int u = 0; u < SPW; ++u) {
        const int q = wave * SPW + u;  // scale wave-load index: a for q < SLA, b after
        if (q < SLA) {
          const int r = L.a_row0 + 64 * q + lane;
          vs[u] = (uint32_t)(((int64_t)(r >> p.sa_shift) * p.sa_rs + (int64_t)L.kb0 * p.sa_ks) * 4);
        } else {
          const int r = L.b_row0 + 64 * (q - SLA) + lane;
          vs[u] = (uint32_t)(((int64_t)(r >> p.sb_shift) * p.sb_rs + (int64_t)L.kb0 * p.sb_ks) * 4);
        }
      }
    }
    const int st = n_issued % NS;
    const uint32_t koff = (uint32_t)l_it * BK;
    const bool in = (int)(koff + chunk * 16) < L.k_len;  // false only in a ragged last 128-block
    const uint32_t sA = lds_base + st * STAGE, sB = sA + BM * BK;
    const int a_rows = L.a_lim - L.a_row0;  // rows past the end of a ragged group are not fetched
    const uint32_t soA = (uint32_t)L.a_row0 * (uint32_t)p.lda + L.k_begin + koff;
    const uint32_t soB = (uint32_t)L.b_row0 * (uint32_t)p.ldb + L.k_begin + koff;
#pragma unroll
    for (int q0 = 0; q0 < LA; q0 += NW) {
      const int q = q0 + wave;
      dma16(rs_a, (in && 8 * q < a_rows) ? va : kOob, soA + (uint32_t)(8 * q) * (uint32_t)p.lda, sA + q * 1024);
    }
#pragma unroll
    for (int q0 = 0; q0 < LB; q0 += NW) {
      const int q = q0 + wave;
      dma16(rs_b, in ? vb : kOob, soB + (uint32_t)(8 * q) * (uint32_t)p.ldb, sB + q * 1024);
    }
    {
      const uint32_t sc = sc_base + st * (BM + BN) * 4;
#pragma unroll
      for (int u = 0; u < SPW; ++u) {
        const int q = wave * SPW + u;
        if (q < SLA) dma4(rs_sa, vs[u], (uint32_t)(l_it * p.sa_ks * 4), sc + q * 256);
        else         dma4(rs_sb, vs[u], (uint32_t)(l_it * p.sb_ks * 4), sc + q * 256);
      }
    }
    ++l_it;
    ++n_issued;
  };
  // ---- L2 prefetcher: a third cursor, p.pf_dist 128-blocks ahead of the loader.  HBM latency is
  // longer than the 1.5 stages of lookahead the LDS ring can hold, so the lines of a stage are
  // pulled into L2 early by touching one dword of each 128-byte line (direct-to-LDS loads into a
  // sink area: no VGPR is written behind the compiler's back).  Each wave touches the lines its
  // own later stage loads will fetch: lane x -> load x/8 of the wave, row x%8. ----
  Tile Pf;
  int pt = t_first - t_step, p_it = 0, p_nk = 0;
  v4i rs_b_pf = rs_a;
  const uint32_t pf_sink = sc_base + NS * (BM + BN) * 4;
  const bool pfa_ok = (lane >> 3) < LA / NW, pfb_ok = (lane >> 3) < LB / NW;
  const uint32_t vpa = (uint32_t)(8 * (wave + NW * (lane >> 3)) + (lane & 7)) * (uint32_t)p.lda;
  const uint32_t vpb = (uint32_t)(8 * (wave + NW * (lane >> 3)) + (lane & 7)) * (uint32_t)p.ldb;
  auto prefetch_stage = [&]() {
    while (p_it >= p_nk) {
      pt += t_step;
      if (pt >= t_end) return;
      decode(++p_n, pt, Pf);
      p_it = 0;
      p_nk = (Pf.k_len + 127) >> 7;
      rs_b_pf = make_rsrc(p.b + (MODE == GEMM_M_GROUPED ? (int64_t)Pf.g * p.b_stride_g : 0), (uint32_t)p.b_bytes);
    }
    const uint32_t koff = (uint32_t)p_it * BK;
    const int a_rows = Pf.a_lim - Pf.a_row0;
    const bool a_in = pfa_ok && 8 * (wave + NW * (lane >> 3)) < a_rows;
    dma4(rs_a, a_in ? vpa : kOob, (uint32_t)Pf.a_row0 * (uint32_t)p.lda + Pf.k_begin + koff, pf_sink);
    dma4(rs_b_pf, pfb_ok ? vpb : kOob, (uint32_t)Pf.b_row0 * (uint32_t)p.ldb + Pf.k_begin + koff, pf_sink + 256);
    ++p_it;
  };

  // Wait until stage `s` has landed for this wave.  Loads return in order, so it is enough that
  // at most the operand and scale loads of the one stage issued after it are outstanding (its
  // prefetch touches were issued before them and are older).  Stores of an earlier epilogue can
  // only make the wait longer, never too short.
  auto wait_stage = [&](int s) {
    if (n_issued - s - 1 >= 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DPW + SPW) : "memory");
    else wait_all_vmem();
  };

  auto read_frags = [&](int s, int ks, v8i* af, v8i* bf) {
    const uint8_t* sA = lds + (s % NS) * STAGE + wm0 * BK;
    const uint8_t* sB = lds + (s % NS) * STAGE + BM * BK + wn0 * BK;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const uint4 lo = *(const uint4*)(sA + i * 32 * BK + coff[ks][0]);
      const uint4 hi = *(const uint4*)(sA + i * 32 * BK + coff[ks][1]);
      af[i] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint4 lo = *(const uint4*)(sB + j * 32 * BK + coff[ks][0]);
      const uint4 hi = *(const uint4*)(sB + j * 32 * BK + coff[ks][1]);
      bf[j] = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    }
  };

#pragma unroll 1
  for (int s = 0; s < NS + p.pf_dist; ++s) prefetch_stage();
#pragma unroll 1
  for (int s = 0; s < NS; ++s) issue_stage();

  int gb = 0;  // global 128-block counter: the stage the MFMAs consume next
  Tile C;
#pragma unroll 1
  for (int t = t_first; t < t_end; t += t_step) {
    decode(++c_n, t, C);
    const int nk = (C.k_len + 127) >> 7;
    // Waves whose whole row range lies past the end of a ragged group skip the MFMAs (they still
    // take part in the loads and barriers).
    const bool wave_active = C.a_row0 + wm0 < C.a_lim;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

#pragma unroll 1
    for (int it = 0; it < nk; ++it, ++gb) {
      wait_stage(gb);
      __syncthreads();  // everybody's share of stage gb has landed
      v8i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
      int sca[TM], scb[TN];
      if (wave_active) {
        const float* scA = sc_lds + (gb % NS) * (BM + BN);
        const float* scB = scA + BM;
#pragma unroll
        for (int i = 0; i < TM; ++i) sca[i] = (int)(__float_as_uint(scA[wm0 + i * 32 + (lane & 31)]) >> 23);
#pragma unroll
        for (int j = 0; j < TN; ++j) scb[j] = (int)(__float_as_uint(scB[wn0 + j * 32 + (lane & 31)]) >> 23);
        read_frags(gb, 0, fa0, fb0);
        read_frags(gb, 1, fa1, fb1);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa0[i], fb0[j], acc[i][j], 0, 0, 0, sca[i], 0, scb[j]);
      }
      // Every wave has pulled both steps' fragments of stage gb into registers: its ring slot can
      // be refilled now, half a stage before the next barrier (the loads get 1.5 stages to land).
      __syncthreads();
      if (p.pf_dist > 0) prefetch_stage();
      issue_stage();
      if (wave_active) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa1[i], fb1[j], acc[i][j], 0, 0, 0, sca[i], 0, scb[j]);
      }
    }

    // ---- epilogue ----
    if (!wave_active) continue;
    if (MODE == GEMM_K_GROUPED && nk == 0 && ACC) continue;
    // The descriptor ends after the tile's last valid row: stores to ragged rows are dropped.
    char* outp = (char*)p.out + (MODE == GEMM_K_GROUPED ? (int64_t)C.g * p.out_stride_g * esz : 0);
    const __amdgpu_buffer_rsrc_t rs_out = __builtin_amdgcn_make_buffer_rsrc(outp, 0, (int)((uint32_t)C.a_lim * pitch), kRsrcFlags);
    const uint32_t s_tile = (uint32_t)(C.a_row0 + wm0) * pitch + (uint32_t)(C.b_row0 + wn0) * esz;
    const int colw = C.b_row0 + wn0 + (lane & 31);
    if (MODE == GEMM_M_GROUPED && p.out_row_index) {
      // Result row r goes to output row out_row_index[r] (the un-permute folded into the store);
      // rows of the group's padding map to a negative index and are dropped.
      uint8_t* stg = lds + NS * STAGE + SC_RING * (BM + BN) * 4 + 512 + wave * 2048;
      const __amdgpu_buffer_rsrc_t rs_sc = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, (int)((uint32_t)p.out_rows * pitch), kRsrcFlags);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        uint32_t vrow[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int r = C.a_row0 + wm0 + i * 32 + h * 16 + (lane >> 2);
          const int dst = r < C.a_lim ? p.out_row_index[r] : -1;
          vrow[h] = dst >= 0 ? (uint32_t)dst * pitch + (uint32_t)(lane & 3) * 16 : kOob;
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int colc = C.b_row0 + wn0 + j * 32 + (lane & 3) * 8;
          const bool col_ok = colc < C.b_lim;
          store_staged_bf16_rows(acc[i][j], rs_sc, stg, col_ok ? vrow[0] : kOob, col_ok ? vrow[1] : kOob,
                                 (uint32_t)(C.b_row0 + wn0 + j * 32) * 2, lane);
        }
      }
    } else if (p.out_dtype != PT_F32 && wide_ok && (C.b_lim & 7) == 0) {
      uint8_t* stg = lds + NS * STAGE + SC_RING * (BM + BN) * 4 + 512 + wave * 2048;
      // rows first, then the column blocks of a row band back to back: adjacent 64-byte halves of
      // a cache line are written by consecutive instructions
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int colc = C.b_row0 + wn0 + j * 32 + (lane & 3) * 8;
          const uint32_t voff = colc < C.b_lim ? (uint32_t)(lane >> 2) * pitch + (uint32_t)(lane & 3) * 16 : kOob;
          store_staged_bf16(acc[i][j], rs_out, stg, voff, s_tile + i * 32 * pitch + j * 64, pitch, ACC, lane);
        }
    } else if (p.out_dtype != PT_F32 && pair_ok && (C.b_lim & 1) == 0) {
      const bool odd = lane & 1;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint32_t voff = colw + j * 32 < C.b_lim ? (uint32_t)(4 * (lane >> 5) + odd) * pitch + (uint32_t)(((lane & 31) & ~1) + j * 32) * 2 : kOob;
#pragma unroll
        for (int i = 0; i < TM; ++i) store_pairs_bf16(acc[i][j], rs_out, voff, s_tile + i * 32 * pitch, pitch, ACC, odd);
      }
    } else if (p.out_dtype == PT_F32) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint32_t voff = colw + j * 32 < C.b_lim ? (uint32_t)(4 * (lane >> 5)) * pitch + (uint32_t)((lane & 31) + j * 32) * 4 : kOob;
#pragma unroll
        for (int i = 0; i < TM; ++i) store_f32(acc[i][j], rs_out, voff, s_tile + i * 32 * pitch, pitch, ACC);
      }
    } else {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint32_t voff = colw + j * 32 < C.b_lim ? (uint32_t)(4 * (lane >> 5)) * pitch + (uint32_t)((lane & 31) + j * 32) * 2 : kOob;
#pragma unroll
        for (int i = 0; i < TM; ++i) store_single_bf16(acc[i][j], rs_out, voff, s_tile + i * 32 * pitch, pitch, ACC);
      }
    }
  }
  wait_all_vmem();  // nothing may still be writing into this workgroup's LDS when it retires
}

static int g_num_cus = 0;

template <int MODE, int BM, int BN, int WGM, int WGN, bool ACC>
static int launch_one(GemmArgs a, hipStream_t stream) {
  constexpr int threads = WGM * WGN * 64;
  constexpr size_t lds = (size_t)2 * (BM + BN) * 128 + 2 * (BM + BN) * 4 + 512 + (size_t)WGM * WGN * 2048;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)fp8_gemm_nt_persistent_kernel<MODE, BM, BN, WGM, WGN, ACC>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_error("gemm: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return PT_ERR_LAUNCH; }
    attr_set = true;
  }
  if (g_num_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    g_num_cus = n;
  }
  { const char* e = getenv("PT_GEMM_PF"); a.pf_dist = e ? atoi(e) : 0; if (a.pf_dist < 0) a.pf_dist = 0; }
  a.tiles_a = (int)cdiv(a.rows_a, BM);
  a.tiles_b = (int)cdiv(a.rows_b, BN);
  int64_t upper;
  if (MODE == GEMM_DENSE) upper = a.total_tiles = (int64_t)a.tiles_a * a.tiles_b;
  else if (MODE == GEMM_K_GROUPED) upper = a.total_tiles = (int64_t)a.tiles_a * a.tiles_b * a.G;
  else upper = ((a.rows_a / 128 + a.G) / 2 + 1) * a.tiles_b;  // the kernel counts the exact number
  if (upper == 0) return PT_OK;
  PT_REQUIRE(upper < (1ll << 30), "gemm: too many tiles");
  int64_t blocks = (g_num_cus + 7) / 8 * 8;
  if (upper < blocks) blocks = (upper + 7) / 8 * 8;
  hipLaunchKernelGGL((fp8_gemm_nt_persistent_kernel<MODE, BM, BN, WGM, WGN, ACC>), dim3((unsigned)blocks), dim3(threads), lds, stream, a);
  return check_launch("fp8_gemm_nt_persistent_kernel");
}

template <int BM, int BN, int WGM, int WGN>
static int launch_mode(const GemmArgs& a, hipStream_t stream) {
  switch (a.mode) {
    case GEMM_DENSE: return launch_one<GEMM_DENSE, BM, BN, WGM, WGN, false>(a, stream);
    case GEMM_M_GROUPED: return launch_one<GEMM_M_GROUPED, BM, BN, WGM, WGN, false>(a, stream);
    default:
      return a.accumulate ? launch_one<GEMM_K_GROUPED, BM, BN, WGM, WGN, true>(a, stream)
                          : launch_one<GEMM_K_GROUPED, BM, BN, WGM, WGN, false>(a, stream);
  }
}

int launch_gemm_persistent(const GemmArgs& a, int variant, hipStream_t stream) {
  PT_REQUIRE(a.mode != GEMM_M_GROUPED || a.G <= kMaxGroupsGemm, "gemm: at most %d groups", kMaxGroupsGemm);
  switch (variant) {
    case 0: return launch_mode<256, 256, 2, 4>(a, stream);  // 8 waves, 128 x 64 per wave
    case 1: return launch_mode<256, 256, 2, 2>(a, stream);  // 4 waves, 128 x 128 per wave
  }
  PT_REQUIRE(false, "gemm: unknown variant %d", variant);
}

}  // namespace pt
