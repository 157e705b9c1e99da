// Persistent FP8 GEMM for gfx950 with a software-pipelined main loop.  Work list, loads, LDS
// layout and result stores are those of the two-phase kernel in gemm_persistent.hip; the
// difference is how one wave orders its own instructions inside a tile:
//
//  * the fragments of MFMA step 0 of a 128-block are read from LDS while step 1 of the block
//    before runs, and those of step 1 while step 0 runs: each wave overlaps its own LDS reads
//    with its own MFMAs instead of relying on the other wave of its SIMD to fill the gap;
//  * the refill of a ring slot is cut into its single wave-loads, issued one per MFMA slot, so
//    the address arithmetic and the M0 writes hide under the matrix pipe as well;
//  * one workgroup barrier per 128-block instead of two;
//  * the MFMAs are volatile inline assembly with a memory clobber, which pins this interleaving
//    (the compiler's scheduler would otherwise regroup reads and MFMAs); the accumulators of the
//    8-wave shape stay in ordinary registers, where the epilogue reads them without a copy, those
//    of the 4-wave shape (256 values per lane) in the accumulation registers;
//  * the E8M0 exponent bytes of a block's scales are packed four to a register and selected by
//    the MFMA's op_sel bits.
//
// The pipeline has a fill/drain of one block per tile and a slower tile switch: it wins when a
// tile's reduction is long (dense GEMMs, grouped GEMMs with K >= 1536), and the two-phase kernel
// wins for short ones; the dispatcher in gemm.hip chooses.
#include "gemm_persistent_parts.h"
#include <type_traits>

namespace pt {

template <int MODE, int BM, int BN, int WGM, int WGN, bool ACC>
__global__ __launch_bounds__(WGM * WGN * 64, 1) void fp8_gemm_nt_pipelined_kernel(GemmArgs p) {
  constexpr int NW = WGM * WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  // 128 accumulator values per lane fit next to everything else in the 256 ordinary registers a
  // wave has at two waves per SIMD; 256 need the accumulation registers.
  constexpr bool kAccInAgpr = TM * TN * 16 > 128;
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
  __shared__ int s_pref[MODE != GEMM_DENSE ? kMaxGroupsGemm + 2 : 2];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
  const uint32_t sc_base = lds_base + NS * STAGE;
  const float* sc_lds = (const float*)(lds + NS * STAGE);

  // ---- tile list ----
  int total_tiles;
  if (MODE == GEMM_M_GROUPED) {
    scan_group_tiles<BM>(p, s_pref, tid, lane);
    total_tiles = __builtin_amdgcn_readfirstlane(s_pref[p.G]) * p.tiles_b;
  } else {
    total_tiles = (int)p.total_tiles;
    if (MODE == GEMM_K_GROUPED) scan_group_costs(p, s_pref, tid, lane);
  }
  const int xcd = blockIdx.x & 7;
  // lanes 0 and 1 find the two ends of this XCD's share of the list side by side
  const int t_step = gridDim.x >> 3;
  const int t_cut = xcd_first_tile<MODE>(p, s_pref, total_tiles, xcd + (lane & 1), t_step);
  const int t_end = __builtin_amdgcn_readlane(t_cut, 1);
  const int t_first = __builtin_amdgcn_readlane(t_cut, 0) + (blockIdx.x >> 3);

  auto decode_any = [&](int t, Tile& T) { decode_tile<MODE, BM, BN>(p, s_pref, t, T); };

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

  // ---- loader: walks (tile, 128-block) pairs ahead of the MFMAs and keeps the LDS ring full ----
  Tile L;
  int lt = t_first - t_step, l_it = 0, l_nk = 0, n_issued = 0;
  int l_n = -1, c_n = -1;  // per-cursor ordinal of the current tile in this workgroup's list
  v4i rs_b = rs_a, rs_sb = rs_sa;
  uint32_t vs[SPW];  // this wave's per-lane scale offsets (bytes) at step 0 of the loader's tile
  bool l_ok = false, l_in = false;
  uint32_t l_sA = 0, l_soA = 0, l_soB = 0, l_sc = 0, l_sa_off = 0, l_sb_off = 0;
  int l_a_rows = 0;
  // After the work list is exhausted the pieces still execute (no branches between the MFMAs)
  // but every lane's offset is out of range, so nothing is fetched.
  int n_slots = 0;  // issue_begin calls so far (real or not): picks the ring slot
  auto issue_begin = [&]() {
    l_ok = false;
    l_in = false;
    {  // the slot this call owns; an exhausted call still (zero-)fills it, and it is free by then
      const int st0 = n_slots % NS;
      ++n_slots;
      l_sA = lds_base + st0 * STAGE;
      l_sc = sc_base + st0 * (BM + BN) * 4;
    }
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
    const uint32_t koff = (uint32_t)l_it * BK;
    l_in = (int)(koff + chunk * 16) < L.k_len;  // false only in a ragged last 128-block
    l_a_rows = L.a_lim - L.a_row0;  // rows past the end of a ragged group are not fetched
    l_soA = (uint32_t)L.a_row0 * (uint32_t)p.lda + L.k_begin + koff;
    l_soB = (uint32_t)L.b_row0 * (uint32_t)p.ldb + L.k_begin + koff;
    l_sa_off = (uint32_t)(l_it * p.sa_ks * 4);
    l_sb_off = (uint32_t)(l_it * p.sb_ks * 4);
    l_ok = true;
    ++l_it;
    ++n_issued;
  };
  // Load number k (0 <= k < DPW + SPW) of the stage set up by issue_begin: this wave's k-th 1 KiB
  // operand load, then its scale loads.  Kept as separate pieces so that the main loop can slot
  // them between MFMAs.
  auto issue_piece = [&](int k) {
    if (k < LA / NW) {
      const int q = k * NW + wave;
      dma16(rs_a, (l_in && 8 * q < l_a_rows) ? va : kOob, l_soA + (uint32_t)(8 * q) * (uint32_t)p.lda, l_sA + q * 1024);
    } else if (k < DPW) {
      const int q = (k - LA / NW) * NW + wave;
      dma16(rs_b, l_in ? vb : kOob, l_soB + (uint32_t)(8 * q) * (uint32_t)p.ldb, l_sA + BM * BK + q * 1024);
    } else {
      const int u = k - DPW;
      const int q = wave * SPW + u;
      if (q < SLA) dma4(rs_sa, l_ok ? vs[u] : kOob, l_sa_off, l_sc + q * 256);
      else         dma4(rs_sb, l_ok ? vs[u] : kOob, l_sb_off, l_sc + q * 256);
    }
  };
  auto issue_stage = [&]() {
    issue_begin();
#pragma unroll
    for (int k = 0; k < DPW + SPW; ++k) issue_piece(k);
  };

  // Wait until stage `s` has landed for this wave.  Loads return in order, so it is enough that
  // at most the operand and scale loads of the one stage issued after it are outstanding.  Stores of an earlier epilogue can
  // only make the wait longer, never too short.
  auto wait_stage = [&](int s) {
    if (n_issued - s - 1 >= 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DPW + SPW) : "memory");
    else wait_all_vmem();
  };

  // fragment r of a step: a-block r for r < TM, b-block r - TM after
  auto read_frag_piece = [&](int s, int ks, int r, v8i* af, v8i* bf) {
    const uint8_t* base = lds + (s % NS) * STAGE + (r < TM ? (wm0 + r * 32) * BK : BM * BK + (wn0 + (r - TM) * 32) * BK);
    const uint4 lo = *(const uint4*)(base + coff[ks][0]);
    const uint4 hi = *(const uint4*)(base + coff[ks][1]);
    const v8i f = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    if (r < TM) af[r] = f; else bf[r - TM] = f;
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
  for (int s = 0; s < NS; ++s) issue_stage();

  // Software pipeline over 128-blocks ("stages", numbered globally across this workgroup's tiles):
  // the fragments of MFMA step 0 of a stage are pulled from LDS while step 1 of the stage before
  // runs, and those of step 1 while step 0 runs, so ds_reads and MFMAs of one wave overlap.
  //   top of stage g:   regs hold step-0 fragments + scales of stage g
  //                     issue ds_reads of step 1 (stage g) | MFMAs of step 0
  //   barrier:          every wave holds all of stage g in registers and its share of stage g+1
  //                     has landed -> slot g%2 is refilled with stage g+2
  //                     issue ds_reads of step 0 (stage g+1) | MFMAs of step 1
  // The E8M0 exponent bytes of a stage's scales, packed one byte per 32-row block: the MFMA picks
  // its byte with the opsel immediates, so a whole stage costs two registers.
  static_assert(TM <= 4 && TN <= 4, "one packed register per operand");
  auto read_scales = [&](int s, int& pa, int& pb) {
    const float* scA = sc_lds + (s % NS) * (BM + BN);
    const float* scB = scA + BM;
    uint32_t a = 0, b = 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) a |= ((__float_as_uint(scA[wm0 + i * 32 + (lane & 31)]) >> 23) & 0xFFu) << (8 * i);
#pragma unroll
    for (int j = 0; j < TN; ++j) b |= ((__float_as_uint(scB[wn0 + j * 32 + (lane & 31)]) >> 23) & 0xFFu) << (8 * j);
    pa = (int)a; pb = (int)b;
  };
  v8i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
  int sca = 0, scb = 0, sca_n = 0, scb_n = 0;
  wait_stage(0);
  __syncthreads();
  read_scales(0, sca, scb);
  read_frags(0, 0, fa0, fb0);

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
      // MFMAs are issued in a fixed order with the LDS reads and the direct-to-LDS loads slotted
      // between them (scheduling barriers pin the order): one wavefront keeps its SIMD's matrix
      // pipe fed while it does its own data movement.
      constexpr int NM = TM * TN, NR = TM + TN, NP = DPW + SPW;
      constexpr int DMA_SLOTS = NM;  // the direct-to-LDS loads are spread over all MFMA slots of the second half
      auto half_a = [&](auto act) {
#pragma unroll
        for (int m = 0; m < NM; ++m) {
          mfma_sel<kAccInAgpr>(fa0[m / TN], fb0[m % TN], acc[m / TN][m % TN], m / TN, sca, m % TN, scb);
#pragma unroll
          for (int r = m * NR / NM; r < (m + 1) * NR / NM; ++r) read_frag_piece(gb, 1, r, fa1, fb1);
          __builtin_amdgcn_sched_barrier(0);
        }
      };
      auto half_b = [&](auto act) {
#pragma unroll
        for (int m = 0; m < NM; ++m) {
          mfma_sel<kAccInAgpr>(fa1[m / TN], fb1[m % TN], acc[m / TN][m % TN], m / TN, sca, m % TN, scb);
          // the direct-to-LDS loads go out in the first DMA_SLOTS MFMA slots: the earlier they start,
          // the longer they have before the next stage's barrier
          if (m < DMA_SLOTS) {
#pragma unroll
            for (int k = m * NP / DMA_SLOTS; k < (m + 1) * NP / DMA_SLOTS; ++k) issue_piece(k);
          }
          if (m == 0) read_scales(gb + 1, sca_n, scb_n);
#pragma unroll
          for (int r = m * NR / NM; r < (m + 1) * NR / NM; ++r) read_frag_piece(gb + 1, 0, r, fa0, fb0);
          __builtin_amdgcn_sched_barrier(0);
        }
      };
      half_a(std::true_type{});
      // This wave's reads of stage gb are complete and its share of stage gb+1 (the only loads in
      // flight) has landed; after the barrier that holds for every wave.
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();
      issue_begin();
      half_b(std::true_type{});
      sca = sca_n; scb = scb_n;
    }
    // the compiler does not see the MFMAs inside the assembly statements: cover the result latency
    // of the last one before the epilogue reads the accumulators
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue ----
    if (!wave_active) continue;
    if (MODE == GEMM_K_GROUPED && nk == 0 && ACC) continue;
    store_tile<MODE, TM, TN, ACC, kAccInAgpr ? 1 : 2>(acc, p, C, wm0, wn0, lane, lds + NS * STAGE + SC_RING * (BM + BN) * 4 + 512 + wave * 2048);
  }
  wait_all_vmem();  // nothing may still be writing into this workgroup's LDS when it retires
}

template <int MODE, int BM, int BN, int WGM, int WGN, bool ACC>
static int launch_one(GemmArgs a, hipStream_t stream) {
  // LDS: two operand stages, two stages of scales, a sink line, 2 KiB of result staging per wave
  constexpr size_t lds = (size_t)2 * (BM + BN) * 128 + 2 * (BM + BN) * 4 + 512 + (size_t)WGM * WGN * 2048;
  static bool attr_set = false;
  const int64_t upper = plan_tiles(a, BM, BN);
  return launch_persistent_grid(fp8_gemm_nt_pipelined_kernel<MODE, BM, BN, WGM, WGN, ACC>, "fp8_gemm_nt_pipelined_kernel", a, upper, WGM * WGN * 64, lds, attr_set, stream);
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

int launch_gemm_pipelined(const GemmArgs& a, int variant, hipStream_t stream) {
  PT_REQUIRE(a.mode == GEMM_DENSE || a.G <= kMaxGroupsGemm, "gemm: at most %d groups", kMaxGroupsGemm);
  switch (variant) {
    case 0: return launch_mode<256, 256, 2, 4>(a, stream);  // 8 waves, 128 x 64 per wave
    case 1: return launch_mode<256, 256, 2, 2>(a, stream);  // 4 waves, 128 x 128 per wave
  }
  PT_REQUIRE(false, "gemm: unknown variant %d", variant);
}

}  // namespace pt
