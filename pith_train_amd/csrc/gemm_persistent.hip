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
#include "gemm_persistent_parts.h"

namespace pt {

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
  // Wait until stage `s` has landed for this wave.  Loads return in order, so it is enough that
  // at most the operand and scale loads of the one stage issued after it are outstanding.  Stores of an earlier epilogue can
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

    // The two waves of a SIMD (w and w + NW/2) run half a block apart: the later one keeps the
    // second MFMA step of a block until after the next block's barrier, so its MFMAs run while the
    // earlier wave reads its fragments and its own reads run under the earlier wave's MFMAs.  (It
    // holds the step's fragments over the barrier, which it did anyway; the ring slot is free
    // once they are in registers.)  The step still pending when the tile ends runs before the
    // epilogue.
    const bool late = wave >= NW / 2;
    v8i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    int sca[TM], scb[TN];
    auto mfma_step = [&](const v8i* af, const v8i* bf) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf[j], acc[i][j], 0, 0, 0, sca[i], 0, scb[j]);
    };
#pragma unroll 1
    for (int it = 0; it < nk; ++it, ++gb) {
      wait_stage(gb);
      __syncthreads();  // everybody's share of stage gb has landed
      if (wave_active) {
        if (late && it > 0) mfma_step(fa1, fb1);  // second step of the block before
        const float* scA = sc_lds + (gb % NS) * (BM + BN);
        const float* scB = scA + BM;
#pragma unroll
        for (int i = 0; i < TM; ++i) sca[i] = (int)(__float_as_uint(scA[wm0 + i * 32 + (lane & 31)]) >> 23);
#pragma unroll
        for (int j = 0; j < TN; ++j) scb[j] = (int)(__float_as_uint(scB[wn0 + j * 32 + (lane & 31)]) >> 23);
        read_frags(gb, 0, fa0, fb0);
        read_frags(gb, 1, fa1, fb1);
        mfma_step(fa0, fb0);
      }
      // Every wave has pulled both steps' fragments of stage gb into registers: its ring slot can
      // be refilled now, half a stage before the next barrier (the loads get 1.5 stages to land).
      __syncthreads();
      issue_stage();
      if (wave_active && !late) mfma_step(fa1, fb1);
    }
    if (wave_active && late && nk > 0) mfma_step(fa1, fb1);

    // ---- epilogue ----
    if (!wave_active) continue;
    if (MODE == GEMM_K_GROUPED && nk == 0 && ACC) continue;
    store_tile<MODE, TM, TN, ACC, 0>(acc, p, C, wm0, wn0, lane, lds + NS * STAGE + SC_RING * (BM + BN) * 4 + 512 + wave * 2048);
  }
  wait_all_vmem();  // nothing may still be writing into this workgroup's LDS when it retires
}

template <int MODE, int BM, int BN, int WGM, int WGN, bool ACC>
static int launch_one(GemmArgs a, hipStream_t stream) {
  // LDS: two operand stages, two stages of scales, a sink line, 2 KiB of result staging per wave
  constexpr size_t lds = (size_t)2 * (BM + BN) * 128 + 2 * (BM + BN) * 4 + 512 + (size_t)WGM * WGN * 2048;
  static bool attr_set = false;
  const int64_t upper = plan_tiles(a, BM, BN);
  return launch_persistent_grid(fp8_gemm_nt_persistent_kernel<MODE, BM, BN, WGM, WGN, ACC>, "fp8_gemm_nt_persistent_kernel", a, upper, WGM * WGN * 64, lds, attr_set, stream);
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
  PT_REQUIRE(a.mode == GEMM_DENSE || a.G <= kMaxGroupsGemm, "gemm: at most %d groups", kMaxGroupsGemm);
  switch (variant) {
    case 0: return launch_mode<256, 256, 2, 4>(a, stream);  // 8 waves, 128 x 64 per wave
  }
  PT_REQUIRE(false, "gemm: unknown variant %d", variant);
}

}  // namespace pt
