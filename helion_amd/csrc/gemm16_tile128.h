// 128x128x64 tile kernel for 16-bit GEMMs: the small-problem companion of gemm16_tile256.h, same modes and arguments.
// A 256x256 tile needs 64 KB of operands per 2048 matrix-pipe cycles, this one 32 KB per 512, which is right at what a
// CU can pull out of its L2 — so it is slower per flop, but it cuts a problem into four times as many tiles.  The
// entry points use it while 256x256 tiles would leave most of the chip idle (a 2048^3 product has only 64 of them) and
// for grouped GEMMs whose experts hold few rows (less padding in the last row tile of every expert).
//
// 4 waves (2x2) of 64x64, 32x32x16 MFMAs, NS LDS stages of (A 16 KB + W 16 KB): NS = 2 (64 KB, two workgroups per CU)
// for compute-heavy problems, NS = 4 (128 KB, three k-tiles in flight per CU) when there is at most one workgroup per
// CU anyway and the kernel is a weight-streaming loop (a decode batch against a wide weight matrix).
//   A tile [128 rows][128 B]   : as in the 256 kernel (rows gathered by the DMA in the grouped mode).
//   W tile [64 k][256 B]       : row = k, 16 chunks of 8 columns, chunk stored at pos = chunk ^ ((k & 3) << 2): one
//                                transposing read has 32 lanes fetch 4 consecutive k rows x 64 contiguous bytes, and
//                                the xor puts the four rows into different 64-byte quarters of the bank window.
//   W tile, column-major W     : [128 columns][128 B], exactly like the A tile.
// The fragments of a whole k-tile (4 k-steps) live in registers and are refilled in place with the next tile's, k-step
// by k-step, right behind the MFMAs that used them, so the LDS stage of a tile is free for the DMA of tile kt+NS as soon
// as every wave has passed the barrier of tile kt.  Past the last k-tile the DMA fetches the last tile again, so every
// step issues the same number of instructions and the counted waits stay exact.
#pragma once
#include "gemm16_tile256.h"

#define G128_BM 128
#define G128_BN 128
#define G128_TILE_BYTES (128 * 128)

// KTAIL: K is any multiple of 8 (16-byte rows): the last k-tile may be partial.  Its DMA re-reads valid chunks / k rows
// instead of running off the operands, and the part past K is zeroed in LDS once it has landed.
// A4 (with KTAIL, row-major W): K is any even number, so the rows of A are only 4-byte aligned: A comes in through the
// 4-byte DMA, four lanes per 16-byte chunk (the same LDS image from four times the instructions).
template <bool BF, int MODE, bool BCOL = false, int NS = 2, bool KTAIL = false, bool A4 = false>
__global__ __launch_bounds__(256, 2) void hx_gemm16_tile128(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                                                           void* __restrict__ Cv, const int* __restrict__ num_tiles,
                                                           const MoeTile* __restrict__ table, const int32_t* __restrict__ idx, int T,
                                                           int K, int N, int max_tiles, int tiles_n, int a_div, G16Dense d) {
  typedef typename Mfma16<BF>::T out_t;
  typedef typename Mfma16<BF>::V8 V8;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NS][2][G128_TILE_BYTES];  // [stage][A | W]

  // the raster of the 256 kernel: 8 row tiles tall, every 256 consecutive tiles spread over the XCDs in blocks of 32
  int tile;
  {
    const int nwg = gridDim.x, wg = blockIdx.x, chunk = wg >> 8;
    // (the last, partial run of R tiles likewise in 8 blocks of R / 8 when R is a multiple of 8)
    const int rem = nwg & 255, l = wg & 255;
    tile = chunk < (nwg >> 8) ? (chunk << 8) + ((wg & 7) << 5) + ((wg >> 3) & 31)
           : (rem & 7) == 0   ? (chunk << 8) + (l & 7) * (rem >> 3) + (l >> 3)
                              : wg;
  }
  const int GM = 8;
  const int group_size = GM * tiles_n;
  const int gid = tile / group_size;
  const int first_m = gid * GM;
  const int gm = min(max_tiles - first_m, GM);
  const int tm = first_m + (tile % group_size) % gm;
  const int tn = (tile % group_size) / gm;
  MoeTile mt;
  if (MODE == 0) {
    if (tm >= *num_tiles) return;
    mt = table[tm];
  } else {
    mt.expert = 0;
    mt.row_start = tm * G128_BM;
    mt.rows = min(G128_BM, T - tm * G128_BM);
  }
  auto row_of = [&](int lr) {  // matrix row of tile row lr (< mt.rows)
    if (MODE != 0) return mt.row_start + lr;
    const int r = idx[mt.row_start + lr];
    return (r >= 0 && r < T) ? r : -1;
  };
  const int kt0 = MODE == 2 ? (int)blockIdx.y * d.kt_per_split : 0;
  static_assert(!KTAIL || MODE != 2, "a partial last k-tile is not combined with split-K");
  static_assert(!A4 || (KTAIL && !BCOL), "the 4-byte A path exists for the partial-k-tile kernel with a row-major W");
  constexpr int DPI = A4 ? 20 : 8;  // DMA instructions per wave and k-tile
  const int nk = MODE == 2 ? min(d.kt_per_split, K / MOE_BK - kt0) : KTAIL ? (K + MOE_BK - 1) / MOE_BK : K / MOE_BK;
  const int ktail = K - (nk - 1) * MOE_BK;  // valid k of the last tile: 64 unless KTAIL
  const bool has_tail = KTAIL && ktail != MOE_BK;
  A += (long)kt0 * (MOE_BK * 2);
  const long n0 = (long)tn * G128_BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;

  // ---- A DMA: wave w owns tile rows [32w, 32w+32), 4 instructions of 8 rows
  const int lrow = lane >> 3, lpos = lane & 7;
  uint32_t a_vo[4], a_vo_t[KTAIL ? 4 : 1];
  // A4: 16 instructions of 2 rows; lane = (row2, chunk position, 4-byte piece); the swizzle (row >> 1) & 7 of tile row
  // 32w + 2jj + row2 is jj & 7, the same for the whole instruction
  const int row2 = lane >> 5, lpos4 = (lane >> 2) & 7, piece = lane & 3;
  uint32_t a_row4[A4 ? 16 : 1];
  if (A4) {
#pragma unroll
    for (int jj = 0; jj < 16; ++jj) {
      int lr = w * 32 + jj * 2 + row2;
      lr = lr < mt.rows ? lr : 0;
      int r = row_of(lr);
      r = r < 0 ? 0 : r;
      a_row4[jj] = (uint32_t)(r / a_div) * (uint32_t)(d.lda * 2);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int lr = w * 32 + j * 8 + lrow;
    lr = lr < mt.rows ? lr : 0;  // padded rows re-read row 0 of the tile; never stored
    int r = row_of(lr);
    r = r < 0 ? 0 : r;
    const int swz = ((j & 1) ? 4 + (lrow >> 1) : (lrow >> 1)) & 7;
    a_vo[j] = (uint32_t)(r / a_div) * (uint32_t)(d.lda * 2) + (uint32_t)((lpos ^ swz) * 16);
    // last, partial k-tile: chunks past K re-read the last valid one
    if (KTAIL) a_vo_t[j] = (uint32_t)(r / a_div) * (uint32_t)(d.lda * 2) + (uint32_t)(min(lpos ^ swz, ktail / 8 - 1) * 16);
  }
  // ---- W DMA, row-major W: wave w owns k rows [16w, 16w+16), 4 instructions of 4 rows x 256 B; row k = 16w + 4j +
  // (lane>>4), so k & 3 and with it the swizzle do not depend on j.  Chunks past a ragged N re-read the last valid one.
  const uint8_t* We = W + (long)mt.expert * K * N * 2 + n0 * 2 + ((long)kt0 * MOE_BK + w * 16) * d.ldb * 2;  // wave-uniform
  const int wk_l = lane >> 4, wpos = lane & 15;
  const int cmax = (int)((min((long)N - n0, (long)G128_BN) >> 3) - 1);
  const uint32_t w_ch = (uint32_t)(min(wpos ^ (wk_l << 2), cmax) * 16);
  const uint32_t w_vo = (uint32_t)(wk_l * d.ldb * 2) + w_ch;
  // column-major W: wave w owns tile columns [32w, 32w+32) = rows of W^T, 4 instructions of 8 rows, like A
  uint32_t wc_vo[BCOL ? 4 : 1], wc_vo_t[BCOL && KTAIL ? 4 : 1];
  if (BCOL) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = (int)min(n0 + w * 32 + j * 8 + lrow, (long)N - 1);
      const int swz = ((j & 1) ? 4 + (lrow >> 1) : (lrow >> 1)) & 7;
      wc_vo[j] = (uint32_t)col * (uint32_t)(d.ldb * 2) + (uint32_t)((lpos ^ swz) * 16);
      if (KTAIL) wc_vo_t[j] = (uint32_t)col * (uint32_t)(d.ldb * 2) + (uint32_t)(min(lpos ^ swz, ktail / 8 - 1) * 16);
    }
  }
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]);
  auto issue = [&](int kt_unclamped) {  // this wave's 8 DMA instructions of k-tile kt into stage kt % NS
    const int kt = min(kt_unclamped, nk - 1), stage = kt_unclamped % NS;
    const uint32_t la = lds0 + (uint32_t)stage * 2 * G128_TILE_BYTES + (uint32_t)w * 32 * 128;
    const uint32_t lw = lds0 + (uint32_t)stage * 2 * G128_TILE_BYTES + G128_TILE_BYTES;
    const bool tail = has_tail && kt == nk - 1;  // (uniform)
    if (A4) {
      const int emax = tail ? ktail - 2 : MOE_BK - 2;  // last valid pair of elements of this k-tile (K is even)
#pragma unroll
      for (int jj = 0; jj < 16; ++jj) {
        const int e = min((lpos4 ^ (jj & 7)) * 8 + piece * 2, emax);
        hx_g2l4_s(A + (long)kt * 128, a_row4[A4 ? jj : 0] + (uint32_t)(e * 2), la + jj * 256);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) hx_g2l16_s(A + (long)kt * 128, KTAIL && tail ? a_vo_t[KTAIL ? j : 0] : a_vo[j], la + j * 1024);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (BCOL) {
        const uint32_t vo = KTAIL && tail ? wc_vo_t[BCOL && KTAIL ? j : 0] : wc_vo[BCOL ? j : 0];
        if (MODE != 0 && d.w_once) hx_g2l16_s_nt(W + ((long)kt0 + kt) * 128, vo, lw + (uint32_t)w * 32 * 128 + j * 1024);
        else hx_g2l16_s(W + ((long)kt0 + kt) * 128, vo, lw + (uint32_t)w * 32 * 128 + j * 1024);
      } else if (KTAIL && tail) {  // k rows past K re-read row K-1 (offsets from the tile's first k row)
        const int kr = min(w * 16 + 4 * j + wk_l, ktail - 1);
        hx_g2l16_s(We + ((long)kt * MOE_BK - w * 16) * d.ldb * 2, (uint32_t)(kr * d.ldb * 2) + w_ch, lw + (uint32_t)w * 16 * 256 + j * 1024);
      } else if (MODE != 0 && d.w_once) {
        hx_g2l16_s_nt(We + ((long)kt * MOE_BK + 4 * j) * d.ldb * 2, w_vo, lw + (uint32_t)w * 16 * 256 + j * 1024);
      } else {
        hx_g2l16_s(We + ((long)kt * MOE_BK + 4 * j) * d.ldb * 2, w_vo, lw + (uint32_t)w * 16 * 256 + j * 1024);
      }
    }
  };
  // Zero the part of the last k-tile past K, each wave in what it fetched itself (so its own vmcnt wait covers it):
  // A rows (and the rows of a column-major W) 32w .. 32w+31, chunks ktail/8 .. 7; row-major W: whole k rows >= ktail.
  auto zero_tail = [&](int stage) {
    const v4i z = {0, 0, 0, 0};
    const int row = w * 32 + (lane & 31);
    if (A4) {  // 4-byte pieces ktail/2 .. 31 of the row (K even)
      for (int dw = ktail / 2 + (lane >> 5); dw < 32; dw += 2)
        *(int*)(&smem[stage][0][0] + row * 128 + (((dw >> 2) ^ ((row >> 1) & 7)) * 16) + (dw & 3) * 4) = 0;
    } else {
      for (int c = ktail / 8 + (lane >> 5); c < 8; c += 2) {
        const int off = row * 128 + ((c ^ ((row >> 1) & 7)) * 16);
        *(v4i*)(&smem[stage][0][0] + off) = z;
        if (BCOL) *(v4i*)(&smem[stage][1][0] + off) = z;
      }
    }
    if (!BCOL) {
      const int k = w * 16 + (lane >> 2);
      if (k >= ktail)
#pragma unroll
        for (int q = 0; q < 4; ++q) *(v4i*)(&smem[stage][1][0] + k * 256 + ((lane & 3) * 4 + q) * 16) = z;
    }
  };

  // ---- operand addressing
  const int r31 = lane & 31, g = lane >> 5;
  const int ax = (g ^ ((r31 >> 1) & 7)) * 16;  // chunk (2*ks + g) ^ swz -> ax ^ (ks*32)
  const int a_base = (wm * 64 + r31) * 128;
  // transposing read: lane -> (block tb = lane>>4, te = (lane>>2)&3, tq = lane&3) supplies 8 bytes of row
  //   k = 16*ks + 8*(tb>>1) + 4*half + te, columns wn*64 + 32*bj + 16*(tb&1) + 4*tq .. +3, and receives column
  //   32*bj + lane%32 with k = 8*(lane>>5) + 4*half .. +3 of the k-step.  Column block bj sets bit 2 of the chunk index,
  //   which the swizzle only xors: an xor with 64 on the byte offset; k-step ks adds 16 rows = 4096 bytes.
  const int tb = lane >> 4, te = (lane >> 2) & 3, tq = lane & 3;
  int w_off[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int k = 8 * (tb >> 1) + 4 * half + te;
    const int chunk = 8 * wn + 2 * (tb & 1) + (tq >> 1);
    w_off[half] = k * 256 + ((chunk ^ ((k & 3) << 2)) * 16) + (tq & 1) * 8;
  }

  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // One set of fragments per wave (4 k-steps x (2 A + 2 W)), refilled in place: the four fragments of k-step ks take
  // tile kt+1's as soon as the four MFMAs of k-step ks of tile kt have been issued, twelve MFMAs before their next use.
  V8 af[4][2], wf[4][2];
  auto load_ks = [&](int ks, int stage) {
    const uint8_t* sa = &smem[stage][0][0];
    const uint8_t* sw = &smem[stage][1][0];
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) af[ks][bi] = *(const V8*)(sa + a_base + bi * 4096 + (ax ^ (ks * 32)));
#pragma unroll
    for (int bj = 0; bj < 2; ++bj) {
      if (BCOL) {
        wf[ks][bj] = *(const V8*)(sw + (wn * 64 + r31) * 128 + bj * 4096 + (ax ^ (ks * 32)));
      } else {
        v4s part[2];
#pragma unroll
        for (int half = 0; half < 2; ++half)
          part[half] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (v4s __attribute__((address_space(3)))*)(sw + ((w_off[half] ^ (bj * 64)) + ks * 4096)));
        v8s both = (v8s){part[0][0], part[0][1], part[0][2], part[0][3], part[1][0], part[1][1], part[1][2], part[1][3]};
        wf[ks][bj] = __builtin_bit_cast(V8, both);
      }
    }
  };
  // one k-tile: the fragments hold tile kt; tile kt+1 has landed (the refills read it), later ones are in flight.  Every
  // step is the same code (a second register set, alternating, had the compiler shuffle the accumulators between
  // the two copies of the loop body).  Past the last k-tile the refills read the ring's copy of the last tile again.
  auto ktile = [&](int kt) {
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((NS - 2) * DPI));  // this wave's part of tile kt+1 has landed
    if (has_tail && kt + 1 == nk - 1) zero_tail((kt + 1) % NS);
    __syncthreads();  // ... everybody's has, and every wave has read tile kt out of its stage: that stage is free
    issue(kt + NS);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) acc[bj][bi] = Mfma16<BF>::run(wf[ks][bj], af[ks][bi], acc[bj][bi]);
      load_ks(ks, (kt + 1) % NS);
    }
  };
  for (int t = 0; t < NS; ++t) issue(t);
  __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((NS - 1) * DPI));
  if (has_tail && nk == 1) zero_tail(0);
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) load_ks(ks, 0);
  for (int kt = 0; kt < nk; ++kt) ktile(kt);
  HX_WAIT_VM0();  // no DMA may still be writing this workgroup's LDS when it ends

  // ---- epilogue: acc[bj][bi][4a+b] is C[row_of(wm*64 + bi*32 + lane%32)][n0 + wn*64 + bj*32 + 8a + 4g + b].
  // N % 8 == 0 and a piece starts at a multiple of 4: it is either wholly inside the row or wholly outside.
  const long ncol = n0 + wn * 64 + 4 * g;
  if (MODE == 2) {
    float* Cp = (float*)Cv + (long)blockIdx.y * T * d.ldc;
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
      const int lr = wm * 64 + bi * 32 + r31;
      if (lr >= mt.rows) continue;
      float* crow = Cp + (long)(mt.row_start + lr) * d.ldc + ncol;
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int a = 0; a < 4; ++a)
          if (ncol + bj * 32 + 8 * a < N)
            *(v4f*)(crow + bj * 32 + 8 * a) = (v4f){acc[bj][bi][4 * a], acc[bj][bi][4 * a + 1], acc[bj][bi][4 * a + 2], acc[bj][bi][4 * a + 3]};
    }
    return;
  }
  out_t* C = (out_t*)Cv;
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
  int rr[2];  // matrix row of each of this lane's two tile rows, -1: not stored
#pragma unroll
  for (int bi = 0; bi < 2; ++bi) {
    const int lr = wm * 64 + bi * 32 + r31;
    rr[bi] = lr < mt.rows ? row_of(lr) : -1;
  }
#pragma unroll
  for (int bj = 0; bj < 2; ++bj) {
    v4f bv[4];
    if (MODE == 1) {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        bv[a] = (v4f){0.f, 0.f, 0.f, 0.f};
        const long n = ncol + bj * 32 + 8 * a;
        if (d.bias && n < N) {
          if (d.bias_f32) {
            bv[a] = *(const v4f*)((const float*)d.bias + n);
          } else {
            const ov4 b16 = *(const ov4*)((const out_t*)d.bias + n);
            bv[a] = (v4f){(float)b16[0], (float)b16[1], (float)b16[2], (float)b16[3]};
          }
        }
      }
    }
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
      if (rr[bi] < 0) continue;
      out_t* crow = C + (long)rr[bi] * d.ldc + ncol + bj * 32;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        ov4 o;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          float v = acc[bj][bi][4 * a + b];
          if (MODE == 1) {
            v += bv[a][b];
            if (d.relu) v = fmaxf(v, 0.f);
          }
          o[b] = (out_t)v;
        }
        if (ncol + bj * 32 + 8 * a < N) *(ov4*)(crow + 8 * a) = o;
      }
    }
  }
}
