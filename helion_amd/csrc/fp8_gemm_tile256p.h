// hx_fp8_gemm_tile256p: the 256x256x128 FP8 tile kernel as a persistent workgroup (opt-in, HX_FEATURE_FP8_GEMM_PERSISTENT;
// not yet run on the hardware).  Same tile, LDS layout, fragment scheme and k-tile schedule as hx_fp8_gemm_tile256 (full
// tiles, K-contiguous B, 16-bit output); what changes is what happens between two tiles of one workgroup:
//
//   * the k-tile pipeline does not stop at a tile's end.  The DMA of "k-tile kt+2" simply goes on into the next tile's
//     k-tiles 0 and 1 during the last two k-tiles of the current one (the number of k-tiles is even, so the stages keep
//     their parity), and the fragment refills of the last k-tile fetch the next tile's first fragments;
//   * the epilogue of tile T runs INSIDE the first k-tile of tile T+1.  That k-tile touches every accumulator block exactly
//     once (one 16x16x128 MFMA per block per k-tile) and may do so in any order, with a zero C operand instead of the
//     old accumulator.  So the accumulators are handed over in four groups of 32 rows: group g is scaled, converted and
//     written to a staging block in the LDS, then the 16 MFMAs of the new tile that overwrite exactly those blocks are
//     issued, then the staged rows are read back as whole 256-byte row pieces and stored - while the matrix pipe works
//     through those MFMAs the wave converts the next group.  The matrix pipe therefore never drains between tiles, the
//     prologue (two k-tiles of DMA latency) is paid once per workgroup instead of once per tile, and there is no launch gap;
//   * the staging blocks live in 32 KB of LDS next to the two stages (160 KB in all), 8 KB per wave = one 32-row group
//     of a 16-bit output, rows of 256 bytes with the 16-byte chunk c of row r at position c ^ (r & 15) instead of padding
//     (conflict-free for the 8-byte writes down a column as for the 16-byte reads along a row);
//   * waits: the stores of a hand-over are newer than the DMA instructions the next counted wait is for and older than
//     the ones issued after them, so the two waits that follow a hand-over allow 32 instructions in flight instead of 16
//     (16 DMA + 16 stores); all other waits are the plain kernel's.
// Every MFMA is written as an instruction with its accumulator an explicit operand (hx_common.h: hx_mfma_..._acc /
// _overwrite, hx_acc_read), so that all 256 accumulators keep their registers around the tile loop and nothing is spilled:
// a reload from scratch memory would make the compiler wait for every DMA in flight.
// Tiles are dealt to the workgroups so that the 32 workgroups of an XCD work on 32 consecutive tiles of that XCD's range
// of the grouped raster at any time, as the plain kernel's launch order does.
#pragma once
#include "hx_common.h"

#define T256P_STG_BYTES (32 * 256)  // one wave's staging block: 32 rows x 128 columns of a 16-bit type

template <int OUT>
__global__ __launch_bounds__(256) void hx_fp8_gemm_tile256p(const uint8_t* __restrict__ A, const uint8_t* __restrict__ Bt,
                                                           typename OutT<OUT>::T* __restrict__ C, int M, int N, int K, long lda,
                                                           long ldb, long ldc, const float* __restrict__ scale_a,
                                                           const float* __restrict__ scale_b, int tiles_m, int tiles_n) {
  typedef typename OutT<OUT>::T out_t;
  static_assert(sizeof(out_t) == 2, "the staging blocks are sized for 16-bit outputs");
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2][2][T256_TILE_BYTES];  // [stage][A|B][256 rows x 128 B]
  __shared__ __attribute__((aligned(1024))) uint8_t stg[4][T256P_STG_BYTES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;
  const int nk = K / T256_BK;  // even, >= 4 (the host checks)

  // ---- this workgroup's tiles: XCD x (= blockIdx % 8) owns a contiguous range of the raster, its workgroups take that
  // range's tiles in turn
  const int ntiles = tiles_m * tiles_n;
  const int xcd = (int)blockIdx.x & 7, loc = (int)blockIdx.x >> 3, cpx = (int)gridDim.x >> 3;  // gridDim.x is a multiple of 8
  const int per = ntiles >> 3, rem = ntiles & 7;
  const int lo = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per, cnt = xcd < rem ? per + 1 : per;
  const int nt = loc < cnt ? (cnt - loc + cpx - 1) / cpx : 0;  // tiles lo + loc, + cpx, ...
  if (nt == 0) return;  // (whole workgroup)
  auto tile_origin = [&](int ti, long& m0, long& n0) {  // ti-th tile of this workgroup -> grouped raster, 8 tile rows tall
    const int tile = lo + loc + ti * cpx;
    const int GM = 8, group_size = GM * tiles_n, gid = tile / group_size, first_m = gid * GM;
    const int gm = min(tiles_m - first_m, GM);
    m0 = (long)(first_m + (tile % group_size) % gm) * T256_BM;
    n0 = (long)((tile % group_size) / gm) * T256_BN;
  };

  // ---- DMA addressing (as in hx_fp8_gemm_tile256): wave w owns tile rows [64w, 64w+64); instruction j covers rows 64w+8j..
  const int lrow = lane >> 3, lpos = lane & 7;
  const uint32_t a_vo0 = (uint32_t)(lrow * lda + (lpos ^ ((lrow >> 1) & 7)) * 16);
  const uint32_t a_vo1 = (uint32_t)(lrow * lda + (lpos ^ ((4 + (lrow >> 1)) & 7)) * 16);
  const uint32_t b_vo0 = (uint32_t)(lrow * ldb + (lpos ^ ((lrow >> 1) & 7)) * 16);
  const uint32_t b_vo1 = (uint32_t)(lrow * ldb + (lpos ^ ((4 + (lrow >> 1)) & 7)) * 16);
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]) + (uint32_t)w * 64 * 128;
  // DMA instruction i (0..15) of the k-tile at byte column kb of the tile whose wave rows start at pa / pb
  auto issue_one = [&](const uint8_t* pa, const uint8_t* pb, long kb, int stage, int i) {
    const uint32_t la = lds0 + (uint32_t)stage * 2 * T256_TILE_BYTES, lb = la + T256_TILE_BYTES;
    if (i < 8) hx_g2l16_s(pa + (long)i * 8 * lda + kb, (i & 1) ? a_vo1 : a_vo0, la + i * 1024);
    else hx_g2l16_s(pb + (long)(i - 8) * 8 * ldb + kb, (i & 1) ? b_vo1 : b_vo0, lb + (i - 8) * 1024);
  };

  // ---- MFMA operand addressing (as in hx_fp8_gemm_tile256)
  const int r16 = lane & 15, gq = lane >> 4;
  const int kq = (gq >> 1) ^ ((gq & 1) * 3);
  const int x16 = ((2 * kq) ^ ((r16 >> 1) & 7)) * 16;
  const int a_base = (wm * 128 + r16) * 128, b_base = (wn * 128 + r16) * 128;
  auto load_a = [&](v8i& f, int stage, int bi) {
    const uint8_t* base = &smem[stage][0][0] + a_base + bi * 2048;
    v4i lo4 = *(const v4i*)(base + x16), hi4 = *(const v4i*)(base + (x16 ^ 16));
    f = (v8i){lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
  };
  auto load_b = [&](v8i& f, int stage, int bj) {
    const uint8_t* base = &smem[stage][1][0] + b_base + bj * 2048;
    v4i lo4 = *(const v4i*)(base + x16), hi4 = *(const v4i*)(base + (x16 ^ 16));
    f = (v8i){lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
  };

  // acc[bj][bi][r] is C[m0 + wm*128 + 16 bi + lane%16][n0 + wn*128 + 16 bj + 4*(lane/16) + r]
  v4f acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  v8i fa[8], fb[8];

  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;

  // ---- one ordinary k-tile (hx_fp8_gemm_tile256's EARLY schedule): 32 MFMAs and the 16 DMA instructions of the k-tile
  // two ahead (at pa / pb / kb, which may belong to the next tile), the counted wait for the k-tile one ahead, a barrier, 32
  // MFMAs and the refill of all 16 fragments from the other stage, a barrier.  KEEP: instructions that may stay in
  // flight at the wait (16 = the DMA just issued; 32 after a hand-over, whose second half's stores are newer than the DMA
  // waited for).
  auto ktile = [&](int stage, const uint8_t* pa, const uint8_t* pb, long kb, auto keep_c) {
    constexpr int KEEP = decltype(keep_c)::value;
    HX_OPAQUE_S(stage);  // (every k-tile computes its fragment addresses from the stage it is given, at run time)
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int bi = i >> 2, bj = i & 3;
      hx_mfma_16x16x128_e4m3_acc(acc[bj][bi], fb[bj], fa[bi]);
      if (i & 1) issue_one(pa, pb, kb, stage, i >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(KEEP));
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int bi = i >> 2, bj = 4 + (i & 3);
      hx_mfma_16x16x128_e4m3_acc(acc[bj][bi], fb[bj], fa[bi]);
      if ((i & 3) == 3) load_a(fa[bi], stage ^ 1, bi);
      if ((i & 7) == 1) load_b(fb[i >> 3], stage ^ 1, i >> 3);
      if (i >= 28) load_b(fb[4 + (i - 28)], stage ^ 1, 4 + (i - 28));
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };

  // ---- the epilogue's two halves for one group of 32 rows (accumulator blocks bi = 2 g32, 2 g32 + 1, all bj)
  uint8_t* st = &stg[0][0] + w * T256P_STG_BYTES;
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
  auto stage_rows = [&](int g32) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int bj = 0; bj < 8; ++bj) {
        ov4 o;
#pragma unroll
        for (int b = 0; b < 4; ++b) o[b] = (out_t)(hx_acc_read(acc[bj][2 * g32 + h][b]) * alpha);
        const int row = h * 16 + r16;  // row of the group; columns 16 bj + 4 gq .. + 3 = bytes 32 bj + 8 gq .. + 7
        *(ov4*)(st + row * 256 + (((2 * bj + (gq >> 1)) ^ (row & 15)) * 16) + (gq & 1) * 8) = o;
        // one block at a time: with all 256 accumulators and 128 fragment registers live there is no room for the
        // scheduler to convert several blocks ahead
        __builtin_amdgcn_sched_barrier(0);
      }
  };
  auto drain = [&](int g32, long m0, long n0) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int row = p * 4 + (lane >> 4), ch = lane & 15;
      const v4i v = *(const v4i*)(st + row * 256 + ((ch ^ (row & 15)) * 16));
      *(v4i*)(C + (m0 + wm * 128 + g32 * 32 + row) * ldc + n0 + wn * 128 + ch * 8) = v;
      if (p & 1) __builtin_amdgcn_sched_barrier(0);  // two row pieces in flight at a time
    }
  };

  // ---- prologue, once per workgroup: the first tile's k-tiles 0 and 1, the fragments of k-tile 0
  long m0, n0;
  tile_origin(0, m0, n0);
  const uint8_t* pa = A + (m0 + w * 64) * lda;
  const uint8_t* pb = Bt + (n0 + w * 64) * ldb;
#pragma unroll
  for (int i = 0; i < 16; ++i) issue_one(pa, pb, 0, 0, i);
#pragma unroll
  for (int i = 0; i < 16; ++i) issue_one(pa, pb, T256_BK, 1, i);
  __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(16));
  __syncthreads();
#pragma unroll
  for (int f = 0; f < 8; ++f) load_a(fa[f], 0, f);
#pragma unroll
  for (int f = 0; f < 8; ++f) load_b(fb[f], 0, f);
  __syncthreads();

  // Every tile runs the same code, so that the accumulators keep their registers from one tile to the next (a branch
  // around part of a tile makes the compiler move them where the paths meet): k-tile 0 as a hand-over - of the previous
  // tile's accumulators, or, for the workgroup's first tile, of the zeros the accumulators start with, which go to the
  // tile's own (not yet written) part of C and are overwritten by its real values later - then k-tiles 1 .. nk-1.
  long mp = m0, np = n0;  // the tile whose accumulators the next hand-over stores
  for (int ti = 0; ti < nt; ++ti) {
    // where the DMA goes on once this tile's own k-tiles are all issued: the next tile, or (last tile) this tile's last
    // k-tile again, into a stage nobody reads any more - every k-tile issues its 16 DMA instructions, the waits stay constant
    const bool has_next = ti + 1 < nt;
    long m1 = m0, n1 = n0;
    if (has_next) tile_origin(ti + 1, m1, n1);
    const uint8_t* na = A + (m1 + w * 64) * lda;
    const uint8_t* nb = Bt + (n1 + w * 64) * ldb;
    const long nkb0 = has_next ? 0 : (long)(nk - 1) * T256_BK, nkb1 = has_next ? T256_BK : (long)(nk - 1) * T256_BK;

    // ---- hand-over = k-tile 0: stage 0 holds it (its fragments are in registers), stage 1 holds k-tile 1; k-tile 2 goes
    // into stage 0 by DMA under the first half, exactly as in an ordinary k-tile.  The accumulators of tile (mp, np) leave
    // in four groups of 32 rows, each just before the 16 MFMAs that overwrite its blocks.
    auto group_mfma = [&](int g32, auto with_dma, auto second_half) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int bi = 2 * g32 + (i & 1), bj = i >> 1;
        hx_mfma_16x16x128_e4m3_overwrite(acc[bj][bi], fb[bj], fa[bi]);
        if (decltype(with_dma)::value && (i & 1)) issue_one(pa, pb, 2L * T256_BK, 0, 8 * (g32 & 1) + (i >> 1));
        if (decltype(second_half)::value) {
          // fragments die in this order: the A blocks of the first half are dead already, this group's after their last
          // MFMA; B fragments only in the last group, two MFMAs apart
          if (g32 == 2 && i < 4) load_a(fa[i], 1, i);
          if (i == 14 || i == 15) load_a(fa[2 * g32 + (i & 1)], 1, 2 * g32 + (i & 1));
          if (g32 == 3 && (i & 1)) load_b(fb[bj], 1, bj);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    stage_rows(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    group_mfma(0, std::true_type{}, std::false_type{});
    drain(0, mp, np);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    stage_rows(1);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    group_mfma(1, std::true_type{}, std::false_type{});
    drain(1, mp, np);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // k-tile 1 (issued two k-tiles ago) has landed; the 16 DMA instructions of k-tile 2 and the 16 stores above may fly
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(32));
    __syncthreads();
    stage_rows(2);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    group_mfma(2, std::false_type{}, std::true_type{});
    drain(2, mp, np);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    stage_rows(3);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    group_mfma(3, std::false_type{}, std::true_type{});
    drain(3, mp, np);
    __syncthreads();  // every wave has read k-tile 1's fragments out of stage 1: it is free

    // ---- k-tiles 1 .. nk-1.  The wait of k-tile 1 has the second half's 16 stores in flight besides the DMA it issues.
    ktile(1, pa, pb, 3L * T256_BK, std::integral_constant<int, 32>{});
    for (int kt = 2; kt + 2 < nk; ++kt) ktile(kt & 1, pa, pb, (long)(kt + 2) * T256_BK, std::integral_constant<int, 16>{});
    ktile(0, na, nb, nkb0, std::integral_constant<int, 16>{});  // kt = nk - 2
    ktile(1, na, nb, nkb1, std::integral_constant<int, 16>{});  // kt = nk - 1: its refills fetch the next tile's first fragments
    mp = m0, np = n0;
    m0 = m1, n0 = n1, pa = na, pb = nb;
  }

  // ---- the workgroup's last tile: nothing left to overlap the epilogue with
  HX_WAIT_VM0();  // the trailing re-fetches
#pragma unroll
  for (int g32 = 0; g32 < 4; ++g32) {
    stage_rows(g32);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    drain(g32, mp, np);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}
