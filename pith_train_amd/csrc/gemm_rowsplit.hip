// Persistent FP8 GEMM for gfx950 whose direct-to-LDS loads are in progress all the time.
//
// The loads of a CU move at most ~70 GB/s out of L2: a 64 KiB stage of a 256 x 256 x 128 tile needs
// about as long to arrive as its MFMAs need to run, so the load path must never idle.  In the
// two-slot ring of the other persistent kernels a slot can be refilled only after every wave has
// read all of its fragments, i.e. during one half of the loop body.  Here the two MFMA steps of a
// 128-block are cut by rows instead of by reduction depth:
//
//   step X:  A blocks 0,1 (rows 0-63 of the wave's 128) x B blocks 0,1, both 64-deep halves
//   step Y:  A blocks 2,3 (rows 64-127)                 x B blocks 0,1, both halves
//
// and a ring slot is cut the same way: its half E holds the a rows of block rows 0,1 and one half
// of the b part (plus the block's scales), its half O the a rows of block rows 2,3 and the other
// half of the b part.  Inside a step the first 64-deep half comes before the second, which makes
// the a fragments short-lived: four 8-register buffers hold the step's two block rows x two
// halves, and each buffer takes a fragment of the next step as soon as the last MFMA on its old
// content has issued.  With the four b fragments of the block that is 64 fragment registers (the
// first version of this loop held every fragment of a step before the step began, 96 registers,
// and spilled), which leaves the compiler a few registers in hand in all variants.  E of block g
// has been read completely when X(g) ends, O(g) when Y(g) ends; either step refills the half it
// finds free with block g + 2's data, 32 KiB per step, requested two steps before the barrier
// behind which it is first read.  One workgroup barrier per step.
//
// Work list, tile table, LDS layout, scale handling and result stores are those of the
// software-pipelined kernel (gemm_pipelined.hip, gemm_persistent_parts.h).
#include "gemm_persistent_parts.h"
#include <type_traits>

// Measurement builds only (never defined by the Makefile's default target): parts of the main loop
// compiled out to see what the rest costs.  PT_GEMM_ABLATE_MFMA: no MFMAs (the fragment reads go
// with them, nothing consumes their results).  PT_GEMM_ABLATE_LOADS: 1 = every operand and scale
// load is issued out of range (the instruction runs, nothing is fetched), 2 = not issued at all.
// The results of such builds are garbage; only their timing means something.
#ifndef PT_GEMM_ABLATE_MFMA
#define PT_GEMM_ABLATE_MFMA 0
#endif
#ifndef PT_GEMM_ABLATE_LOADS
#define PT_GEMM_ABLATE_LOADS 0
#endif

namespace pt {

// BT: the b operand is given reduction-major, [red][rows_b] with row pitch ldb (the forward layout of
// a weight, read by its input-gradient GEMM), instead of [rows_b][red].
template <int MODE, int BM, int BN, int WGM, int WGN, bool ACC, bool BT = false>
__global__ __launch_bounds__(WGM * WGN * 64, 1) void fp8_gemm_nt_rowsplit_kernel(GemmArgs p) {
  constexpr int NW = WGM * WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int TM = WM / 32, TN = WN / 32;
  // 128 accumulator values per lane fit next to everything else in the 256 ordinary registers a
  // wave has at two waves per SIMD; 256 need the accumulation registers.
  constexpr bool kAccInAgpr = TM * TN * 16 > 128;
  constexpr int BK = 128;                      // reduction depth of one stage = one scale block = two MFMA steps
  constexpr int NS = 2;                        // stages in the LDS ring
  constexpr int STAGE = (BM + BN) * BK;
  constexpr int SLA = BM / 64, SLB = BN / 64;  // 256 B wave-loads per scale vector
  static_assert(BM == 256 && BN == 256 && WGM == 2 && WGN == 4, "the row split is written for 8 waves of 128 x 64");
  constexpr int NP = 5;  // loads a wave issues per step: two 1 KiB loads of a rows, two of b rows, one of scales
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

  // Reduction-major b operand: its part of a stage holds 128 reduction rows of 256 bytes (the
  // tile's 256 b rows), logical 16-byte chunk c of row k at position c ^ 2 (k & 7): the eight rows
  // that one transposing read touches put a chunk at eight different positions, and the chunks
  // c and c + 1 (c even) of the two halves of a 32-row b block never share one, so such a read
  // spreads over all banks.  A direct-to-LDS
  // wave-load covers four such rows (lane -> row lane / 16, position lane % 16); a wave's loads are
  // row quads Q = w, w + 8, ... of a half, so (k & 7) = 4 (w & 1) + lane / 16 for all of them.
  // Fragments come out of it through the transposing LDS read: in every group of 16 lanes, source
  // lane s supplies the address of 8 bytes and lane l receives byte (l & 7) of source lanes
  // (l >> 3), 2 + (l >> 3), ..., 14 + (l >> 3).  With source lane s pointing at reduction row
  // s / 2 and b rows 8 (s & 1) .. + 7 of the group's 16, lane l gets 8 consecutive reduction
  // elements of b row l % 16: four such reads are the lane's 32 bytes of an MFMA operand.
  const int bt_chunk = (lane & 15) ^ (2 * (4 * (wave & 1) + (lane >> 4)));
  const uint32_t vbt = (uint32_t)(lane >> 4) * (uint32_t)p.ldb + bt_chunk * 16;
  uint32_t bt_rd[2];  // per b block j: the lane's byte offset inside the b part of a stage, for reduction rows 0-7
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int s16 = lane & 15, g16 = lane >> 4;
    const int c = (wn0 >> 4) + 2 * j + (g16 & 1);
    bt_rd[j] = (uint32_t)((32 * (g16 >> 1) + (s16 >> 1)) * 256 + ((c ^ (2 * (s16 >> 1))) << 4) + 8 * (s16 & 1));
  }

  const v4i rs_a = make_rsrc(p.a, (uint32_t)p.a_bytes);
  const v4i rs_sa = make_rsrc(p.sa, (uint32_t)p.sa_bytes);

  // ---- loader: walks (tile, 128-block, half) triples ahead of the MFMAs ----
  // Half 0 of a block: a rows 128r + 0..63 and b rows 64c + 0..31 (the A0,A1 and B0 fragments of
  // every wave) plus the block's scales; half 1: the other rows.  Wave-load q covers rows 8q..8q+7.
  Tile L;
  int lt = t_first - t_step, l_u = 0, l_nu = 0;  // l_u: next step of the loader's tile, l_nu: its number of steps
  int l_n = -1, c_n = -1;  // per-cursor ordinal of the current tile in this workgroup's list
  v4i rs_b = rs_a, rs_sb = rs_sa;
  uint32_t vs = 0;  // this wave's per-lane scale offset (bytes) at block 0 of the loader's tile
  bool l_ok = false, l_in = false;
  int l_half = 0;
  uint32_t l_sA = 0, l_soA = 0, l_soB = 0, l_sc = 0, l_sa_off = 0, l_sb_off = 0;
  int l_a_rows = 0;
  // After the work list is exhausted the pieces still execute (no branches between the MFMAs)
  // but every lane's offset is out of range, so nothing is fetched; the wave still issues NP
  // loads per step, which is what the counted waits rely on.
  int n_steps = 0;  // issue_begin calls so far (real or not): block = n_steps / 2 picks the slot, n_steps % 2 the half
  auto issue_begin = [&]() {
    l_ok = false;
    l_in = false;
    {
      const int blk = n_steps >> 1;
      l_half = n_steps & 1;
      l_sA = lds_base + (blk % NS) * STAGE;
      l_sc = sc_base + (blk % NS) * (BM + BN) * 4;
      ++n_steps;
    }
    while (l_u >= l_nu) {
      lt += t_step;
      if (lt >= t_end) return;
      decode(++l_n, lt, L);
      l_u = 0;
      l_nu = ((L.k_len + 127) >> 7) * 2;
      rs_b = make_rsrc(p.b + (MODE == GEMM_M_GROUPED ? (int64_t)L.g * p.b_stride_g : 0), (uint32_t)p.b_bytes);
      rs_sb = make_rsrc(p.sb + (MODE == GEMM_M_GROUPED ? (int64_t)L.g * p.sb_stride_g : 0), (uint32_t)p.sb_bytes);
      if (wave < SLA) {
        const int r = L.a_row0 + 64 * wave + lane;
        vs = (uint32_t)(((int64_t)(r >> p.sa_shift) * p.sa_rs + (int64_t)L.kb0 * p.sa_ks) * 4);
      } else {
        const int r = L.b_row0 + 64 * (wave - SLA) + lane;
        vs = (uint32_t)(((int64_t)(r >> p.sb_shift) * p.sb_rs + (int64_t)L.kb0 * p.sb_ks) * 4);
      }
    }
    const int l_it = l_u >> 1;
    const uint32_t koff = (uint32_t)l_it * BK;
    l_in = (int)(koff + chunk * 16) < L.k_len;  // false only in a ragged last 128-block
    l_a_rows = L.a_lim - L.a_row0;  // rows past the end of a ragged group are not fetched
    l_soA = (uint32_t)L.a_row0 * (uint32_t)p.lda + L.k_begin + koff;
    l_soB = BT ? (uint32_t)(L.k_begin + koff) * (uint32_t)p.ldb + (uint32_t)L.b_row0
               : (uint32_t)L.b_row0 * (uint32_t)p.ldb + L.k_begin + koff;

    l_sa_off = (uint32_t)(l_it * p.sa_ks * 4);
    l_sb_off = (uint32_t)(l_it * p.sb_ks * 4);
    l_ok = true;
    ++l_u;
  };
  // Load number k (0 <= k < NP) of the step set up by issue_begin.  The wave-load numbers keep the
  // parity of the wave (the LDS swizzle of a load depends on it, see above).
  auto issue_piece = [&](int k) {
    if (PT_GEMM_ABLATE_LOADS == 2) return;
    if (PT_GEMM_ABLATE_LOADS == 1) { l_in = false; l_ok = false; }
    if (k < 2) {
      const int q = 16 * k + 8 * l_half + wave;
      dma16_op<0>(rs_a, (l_in && 8 * q < l_a_rows) ? va : kOob, l_soA + (uint32_t)(8 * q) * (uint32_t)p.lda, l_sA + q * 1024);
    } else if (k < 4) {
      if constexpr (BT) {
        // reduction rows 64 half + 0..63: row quad Q covers rows 4Q..4Q+3.  Rows past the end of a
        // ragged reduction lie past the end of the group's b matrix, whose extent is the
        // descriptor's: the hardware returns zeros for them (its range check includes the scalar
        // offset), so no lane needs a check of its own.
        const int Q = 16 * l_half + 8 * (k - 2) + wave;
        dma16_op<1>(rs_b, l_ok ? vbt : kOob, l_soB + (uint32_t)(4 * Q) * (uint32_t)p.ldb, l_sA + BM * BK + Q * 1024);
      } else {
        const int q = 8 * (2 * (k - 2) + (wave >> 2)) + 4 * l_half + (wave & 3);
        dma16_op<1>(rs_b, l_in ? vb : kOob, l_soB + (uint32_t)(8 * q) * (uint32_t)p.ldb, l_sA + BM * BK + q * 1024);
      }
    } else {
      // scales go with the first half of a block; with the second the same instruction is issued
      // out of range into a sink, so that every step counts the same number of loads
      const uint32_t sink = sc_base + SC_RING * (BM + BN) * 4;
      const bool real = l_ok && l_half == 0;
      if (wave < SLA) dma4(rs_sa, real ? vs : kOob, l_sa_off, real ? l_sc + wave * 256 : sink);
      else            dma4(rs_sb, real ? vs : kOob, l_sb_off, real ? l_sc + wave * 256 : sink);
    }
  };
  auto issue_step = [&]() {
    issue_begin();
#pragma unroll
    for (int k = 0; k < NP; ++k) issue_piece(k);
  };

  // one 32-row block of fragments, 64 deep: rows blk_row.. of block `blk` (a: wm0 + 32 i, b: BM + wn0 + 32 j), half ks
  auto read_frag = [&](int stage, int row0, int ks) -> v8i {
    const uint8_t* base = lds + (stage % NS) * STAGE + row0 * BK;
    const uint4 lo = *(const uint4*)(base + coff[ks][0]);
    const uint4 hi = *(const uint4*)(base + coff[ks][1]);
    return v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };
  auto a_row = [&](int i) { return wm0 + 32 * i; };
  auto b_row = [&](int j) { return BM + wn0 + 32 * j; };
  // The b fragments are kept as fb[late][early]: the half of the b part of a slot that is read
  // during step X of its block ("late") against the one read ahead during step Y of the block
  // before.  Row-major b: late = b block j (rows 64c + 32..63), early = 64-deep half.
  // Reduction-major b: late = the 64-deep half (reduction rows 64..127), early = b block j.
  auto read_b = [&](int stage, int late, int early) -> v8i {
    if constexpr (BT) {
      typedef int v2i_t __attribute__((ext_vector_type(2)));
      const uint8_t* base = lds + (stage % NS) * STAGE + BM * BK + bt_rd[early] + late * (64 * 256);
      v8i r;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v2i_t t = __builtin_amdgcn_ds_read_tr8_b64_v2i32((v2i_t __attribute__((address_space(3)))*)(base + q * 8 * 256));
        r[2 * q] = t[0];
        r[2 * q + 1] = t[1];
      }
      return r;
    } else {
      return read_frag(stage, b_row(late), early);
    }
  };

#pragma unroll 1
  for (int s = 0; s < 2 * NS - 1; ++s) issue_step();

  // The E8M0 exponent bytes of a block's scales, packed one byte per 32-row block: the MFMA picks
  // its byte with the opsel immediates, so a whole block costs two registers.
  auto read_scales = [&](int stage, int& pa, int& pb) {
    const float* scA = sc_lds + (stage % NS) * (BM + BN);
    const float* scB = scA + BM;
    uint32_t a = 0, b = 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) a |= ((__float_as_uint(scA[wm0 + i * 32 + (lane & 31)]) >> 23) & 0xFFu) << (8 * i);
#pragma unroll
    for (int j = 0; j < TN; ++j) b |= ((__float_as_uint(scB[wn0 + j * 32 + (lane & 31)]) >> 23) & 0xFFu) << (8 * j);
    pa = (int)a; pb = (int)b;
  };
  // Fragments.  A: four buffers; the step in progress owns all four (two block rows x two 64-deep
  // halves) and hands each to the next step's fragment as soon as its last MFMA has issued.  B:
  // fb[late][early], both block columns and both halves of the current 128-block.
  v8i fa[4], fb[2][2];
  int sca = 0, scb = 0, sca_n = 0, scb_n = 0;
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NP) : "memory");  // both halves of block 0 have landed
  __syncthreads();
  read_scales(0, sca, scb);
  fa[0] = read_frag(0, a_row(0), 0);
  fa[1] = read_frag(0, a_row(1), 0);
  fb[0][0] = read_b(0, 0, 0);
  fb[0][1] = read_b(0, 0, 1);

  int gs = 0;  // global 128-block counter: the block the MFMAs consume next
  Tile C;
#pragma unroll 1
  for (int t = t_first; t < t_end; t += t_step) {
    decode(++c_n, t, C);
    const int nk = (C.k_len + 127) >> 7;
    // Waves whose whole row range lies past the end of a ragged group skip the MFMAs, which leaves
    // the matrix pipe to the other wave of their SIMD, and have nothing to store; they still take
    // part in the loads, the fragment reads and the barriers.
    const bool wave_active = C.a_row0 + wm0 < C.a_lim;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

#pragma unroll 1
    for (int it = 0; it < nk; ++it, ++gs) {
      // Slot m of a step: MFMA (block row i, block column j, half ks), the first 64-deep half
      // before the second:
      //   m:   0        1        2        3        4        5        6        7
      //   X: (0,0,0)  (1,0,0)  (0,1,0)  (1,1,0)  (0,0,1)  (1,0,1)  (0,1,1)  (1,1,1)
      //   Y: (2,0,0)  (3,0,0)  (2,1,0)  (3,1,0)  (2,0,1)  (3,0,1)  (2,1,1)  (3,1,1)
      // The same accumulator comes back four slots later.  A fragment (i, ks) of the step lives in
      // fa[2 ks + (i & 1)] and is used in slots 4 ks + (i & 1) and 4 ks + 2 + (i & 1): the first
      // half's buffers are free from slot 4 on and take the next step's first-half fragments
      // (slots 5, 6); the second half's are free when the step ends and take the next step's
      // second-half fragments in its slots 1, 2.  B fragments fb[late][early] (row-major b: late =
      // block column, early = half; reduction-major b: the other way round): the "early" part of a
      // block's slot is read during step Y of the block before (fb[0][.], each after its last MFMA),
      // the "late" part in slots 0, 1 of step X (fb[1][.]).
      // The two halves of a ring slot: E = a rows of block rows 0,1 + the early b part (+ scales),
      // O = a rows of block rows 2,3 + the late b part.  E of block g has been read when X(g) ends
      // and is refilled during Y(g) with block g + 2; O(g) has been read when Y(g) ends and is
      // refilled during X(g + 1).  Every refill is requested two steps before the barrier behind
      // which it is first read, so a step waits until only the previous step's loads are outstanding.
      // ---- step X ----
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NP) : "memory");
      __syncthreads();
      issue_begin();
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        const int i = m & 1, j = (m >> 1) & 1, ks = m >> 2;
        const int late = BT ? ks : j, early = BT ? j : ks;
        if (wave_active && !PT_GEMM_ABLATE_MFMA) mfma_sel<false>(fa[2 * ks + i], fb[late][early], acc[i][j], i, sca, j, scb);
#pragma unroll
        for (int k = m * NP / 8; k < (m + 1) * NP / 8; ++k) issue_piece(k);
        if (m == 0) fb[1][0] = read_b(gs, 1, 0);
        if (m == 1) { fb[1][1] = read_b(gs, 1, 1); fa[2] = read_frag(gs, a_row(0), 1); }
        if (m == 2) fa[3] = read_frag(gs, a_row(1), 1);
        if (m == 5) fa[0] = read_frag(gs, a_row(2), 0);
        if (m == 6) fa[1] = read_frag(gs, a_row(3), 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      // ---- step Y ----
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NP) : "memory");
      __syncthreads();
      issue_begin();
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        const int i = m & 1, j = (m >> 1) & 1, ks = m >> 2;
        const int late = BT ? ks : j, early = BT ? j : ks;
        if (wave_active && !PT_GEMM_ABLATE_MFMA) mfma_sel<false>(fa[2 * ks + i], fb[late][early], acc[2 + i][j], 2 + i, sca, j, scb);
#pragma unroll
        for (int k = m * NP / 8; k < (m + 1) * NP / 8; ++k) issue_piece(k);
        if (m == 0) read_scales(gs + 1, sca_n, scb_n);
        if (m == 1) fa[2] = read_frag(gs, a_row(2), 1);
        if (m == 2) fa[3] = read_frag(gs, a_row(3), 1);
        if (m == 3) fb[0][0] = read_b(gs + 1, 0, 0);
        if (m == (BT ? 5 : 6)) fb[0][1] = read_b(gs + 1, 0, 1);
        if (m == 5) fa[0] = read_frag(gs + 1, a_row(0), 0);
        if (m == 6) fa[1] = read_frag(gs + 1, a_row(1), 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      sca = sca_n; scb = scb_n;
    }
    // the compiler does not see the MFMAs inside the assembly statements: cover the result latency
    // of the last one before the epilogue reads the accumulators
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue ----
    if (!wave_active) continue;
    if (MODE == GEMM_K_GROUPED && nk == 0 && ACC) continue;
    store_tile<MODE, TM, TN, ACC, 2>(acc, p, C, wm0, wn0, lane, lds + NS * STAGE + SC_RING * (BM + BN) * 4 + 512 + wave * 2048);
  }
  wait_all_vmem();  // nothing may still be writing into this workgroup's LDS when it retires
}

template <int MODE, int BM, int BN, int WGM, int WGN, bool ACC, bool BT = false>
static int launch_one(GemmArgs a, hipStream_t stream) {
  // LDS: two operand stages, two stages of scales, a sink line, 2 KiB of result staging per wave
  constexpr size_t lds = (size_t)2 * (BM + BN) * 128 + 2 * (BM + BN) * 4 + 512 + (size_t)WGM * WGN * 2048;
  static bool attr_set = false;
  const int64_t upper = plan_tiles(a, BM, BN);
  return launch_persistent_grid(fp8_gemm_nt_rowsplit_kernel<MODE, BM, BN, WGM, WGN, ACC, BT>, "fp8_gemm_nt_rowsplit_kernel", a, upper, WGM * WGN * 64, lds, attr_set, stream);
}

template <int BM, int BN, int WGM, int WGN>
static int launch_mode(const GemmArgs& a, hipStream_t stream) {
  switch (a.mode) {
    case GEMM_DENSE: return launch_one<GEMM_DENSE, BM, BN, WGM, WGN, false>(a, stream);
    case GEMM_M_GROUPED:
      return a.b_kmajor ? launch_one<GEMM_M_GROUPED, BM, BN, WGM, WGN, false, true>(a, stream)
                        : launch_one<GEMM_M_GROUPED, BM, BN, WGM, WGN, false>(a, stream);
    default:
      return a.accumulate ? launch_one<GEMM_K_GROUPED, BM, BN, WGM, WGN, true>(a, stream)
                          : launch_one<GEMM_K_GROUPED, BM, BN, WGM, WGN, false>(a, stream);
  }
}

int launch_gemm_rowsplit(const GemmArgs& a, int variant, hipStream_t stream) {
  PT_REQUIRE(a.mode == GEMM_DENSE || a.G <= kMaxGroupsGemm, "gemm: at most %d groups", kMaxGroupsGemm);
  PT_REQUIRE(!a.b_kmajor || a.mode == GEMM_M_GROUPED, "gemm: a reduction-major b operand is built for the m-grouped mode only");
  switch (variant) {
    case 0: return launch_mode<256, 256, 2, 4>(a, stream);  // 8 waves, 128 x 64 per wave
  }
  PT_REQUIRE(false, "gemm: unknown variant %d", variant);
}

}  // namespace pt
