// 256x256x64 tile kernel for 16-bit (bf16 / fp16) GEMMs with fp32 accumulation on gfx950, shared by the grouped (MoE)
// GEMM and the dense matmul entry points.
#pragma once
#include "hx_common.h"

struct MoeTile {
  int expert;
  int row_start;  // position in the sorted order (index into idx)
  int rows;       // valid rows in this tile (1..BM)
  int pad;
};


// ------------------------------------------------------------------------------------------
// tile256: 256 gathered rows x 256 columns x 64 k per step; 4 waves (2x2) of 128x128; 16x16x32 MFMA (under the power
//   limit a stream of them sustains about a fifth more than one of 32x32x16: a quarter of the accumulator registers
//   move per instruction).
//   A tile  [256 rows][128 B]  : same chunk-swizzled layout as the fp8 GEMM; the DMA gathers rows
//                                through idx, so the gather costs nothing extra.
//   W tile  [64 k][512 B]      : row = k, 32 chunks of 8 columns; chunk stored at pos = chunk ^ (moe_wswz(k)<<1).
//                                The MFMA wants 8 consecutive k per lane for one column, W has the
//                                columns contiguous: ds_read_b64_tr_b16 transposes 4(k) x 16(n) blocks
//                                on the way out of LDS (two reads per operand).
//   One MFMA multiplies 32 k; lane (r = lane%16, g = lane/16) supplies k = 8g .. 8g+7 of row / column r: chunk
//   4*ks + g of an A row, k rows 32*ks + 8g .. +7 of a W column.
// ------------------------------------------------------------------------------------------
// Swizzle of a W-tile row, in units of 32 bytes (a pair of chunks).  One transposing read has the 32 lanes
// that the LDS serves together (two groups of 16) fetch 4 consecutive k rows each, 8 rows apart, of the same 32-byte
// column group; rows are 512 B apart (the same banks), so the 8 rows must land in 8 different 32-byte bank groups:
// k&3 goes to bits 2:1 and bit 3 of k to bit 0.
__device__ __forceinline__ int moe_wswz(int k) { return ((k & 3) << 1) | ((k >> 3) & 1); }

#define MOE_BM 256
#define MOE_BN 256
#define MOE_BK 64
#define MOE_TILE_BYTES (256 * 128)

// MODE 0: grouped (MoE) GEMM: rows gathered through the tile table and idx, W of the tile's expert, 16-bit output.
// MODE 1: dense C = act(A @ W + bias): row tile t covers rows 256t ..; 16-bit output.
// BCOL (dense modes): W is given column-major, i.e. as W^T [N][K] with row stride ldb (an nn.Linear weight used as
//         w.T): its tile sits in LDS like the A tile, rows = columns of W, and feeds the MFMA through plain 16-byte reads.
// MODE 2: dense, raw fp32 accumulators of k-tiles [y*kt_per_split, ...) to the fp32 matrix number blockIdx.y at C
//         (split-K partial sums, or the input of an epilogue applied elsewhere).
struct G16Dense {
  long lda, ldb, ldc;   // row strides in elements (grouped GEMM: K, N, N)
  const void* bias;     // [N] or null (MODE 1)
  int bias_f32;         // bias is fp32 rather than the operand type
  int relu;
  int kt_per_split;     // MODE 2: k-tiles per blockIdx.y
  int w_once;           // dense modes, 128-tile kernel: the launch has one row tile, so every byte of W is read once
                        // (its DMA then carries the non-temporal hint)
};

template <bool BF, int MODE, bool BCOL = false>
__global__ __launch_bounds__(256) void hx_gemm16_tile256(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                                                        void* __restrict__ Cv, const int* __restrict__ num_tiles,
                                                        const MoeTile* __restrict__ table, const int32_t* __restrict__ idx, int T, int K,
                                                        int N, int max_tiles, int tiles_n, int a_div, G16Dense d) {
  typedef typename Mfma16<BF>::T out_t;
  typedef typename Mfma16<BF>::V8 V8;
  // [stage][A|W][32 KB]
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2][2][MOE_TILE_BYTES];

  // Grouped raster over (row tile, column tile), 4 row tiles tall (measured against 2, 6, 8 and 16).  Workgroup i runs on
  // XCD i % 8; each run of 256 workgroups covers 256 consecutive tiles of that order, 32 consecutive ones (4 row tiles x
  // 8 column tiles) per XCD,
  // so one XCD's resident tiles share operand panels in its L2 and all eight XCDs work side by side on the same row
  // tiles and on neighbouring column panels of the same expert — the set of panels in flight then fits the memory-side
  // cache, which a contiguous range of the tile order per XCD (eight different experts at once) does not (C5: -6 %).
  int tile;
  {
    const int nwg = gridDim.x, wg = blockIdx.x, chunk = wg >> 8;
    // (the last, partial run of R tiles likewise in 8 blocks of R / 8 when R is a multiple of 8)
    const int rem = nwg & 255, l = wg & 255;
    tile = chunk < (nwg >> 8) ? (chunk << 8) + ((wg & 7) << 5) + ((wg >> 3) & 31)
           : (rem & 7) == 0   ? (chunk << 8) + (l & 7) * (rem >> 3) + (l >> 3)
                              : wg;
  }
  const int GM = 4;
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
    mt.row_start = tm * MOE_BM;
    mt.rows = min(MOE_BM, T - tm * MOE_BM);
  }
  auto row_of = [&](int lr) {  // matrix row of tile row lr (< mt.rows)
    if (MODE != 0) return mt.row_start + lr;
    const int r = idx[mt.row_start + lr];
    return (r >= 0 && r < T) ? r : -1;
  };
  // k-tiles of this workgroup: all of them, or one split's share
  const int kt0 = MODE == 2 ? (int)blockIdx.y * d.kt_per_split : 0;
  const int nk = MODE == 2 ? min(d.kt_per_split, K / MOE_BK - kt0) : K / MOE_BK;
  A += (long)kt0 * (MOE_BK * 2);
  const long n0 = (long)tn * MOE_BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;

  // ---- A DMA: wave w owns tile rows [64w, 64w+64), 8 instructions of 8 rows; rows are gathered, so the
  // per-lane byte offset carries the row (A is below 4 GB, checked by the host).
  const int lrow = lane >> 3, lpos = lane & 7;
  uint32_t a_vo[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    int lr = w * 64 + j * 8 + lrow;
    lr = lr < mt.rows ? lr : 0;  // padded rows re-read row 0 of the tile; never stored
    int r = row_of(lr);
    r = r < 0 ? 0 : r;
    const int swz = ((j & 1) ? 4 + (lrow >> 1) : (lrow >> 1)) & 7;
    // a_div > 1: C row r is the product of A row r / a_div (top-k routing without a replicated A)
    a_vo[j] = (uint32_t)(r / a_div) * (uint32_t)(d.lda * 2) + (uint32_t)((lpos ^ swz) * 16);
  }
  // ---- W DMA: wave w owns k rows [16w, 16w+16), 8 instructions of 2 rows x 512 B.
  // row k = 16w + 2j + (lane>>5); chunk = (lane&31) ^ (moe_wswz(k)<<1); k&15 = 2j + (lane>>5)
  const uint8_t* We = W + (long)mt.expert * K * N * 2 + n0 * 2 + ((long)kt0 * MOE_BK + w * 16) * d.ldb * 2;  // wave-uniform
  const int wk_l = lane >> 5, wpos = lane & 31;
  uint32_t w_vo[8];
  // The last column tile may be ragged (N % 256 != 0, N % 8 == 0): chunks past the end re-read the last valid chunk of
  // the row; the columns they feed are never stored.
  const int cmax = (int)((min((long)N - n0, (long)MOE_BN) >> 3) - 1);
#pragma unroll
  for (int j = 0; j < 8; ++j) w_vo[j] = (uint32_t)(wk_l * d.ldb * 2 + min(wpos ^ (moe_wswz(2 * j + wk_l) << 1), cmax) * 16);
  // column-major W: wave w owns tile columns [64w, 64w+64) = rows of W^T, 8 instructions of 8 rows, exactly like A;
  // columns past N re-read column N-1 and are never stored (W^T is below 4 GB, checked by the host)
  uint32_t wc_vo[BCOL ? 8 : 1];
  if (BCOL) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int col = (int)min(n0 + w * 64 + j * 8 + lrow, (long)N - 1);
      const int swz = ((j & 1) ? 4 + (lrow >> 1) : (lrow >> 1)) & 7;
      wc_vo[j] = (uint32_t)col * (uint32_t)(d.ldb * 2) + (uint32_t)((lpos ^ swz) * 16);
    }
  }
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]);

  // DMA instruction i (0..15) of a k-tile: i < 8 -> gathered A rows 64w + 8i .., else W k-rows 16w + 2(i-8), +1
  auto issue_one = [&](int kt, int stage, int i) {
    const uint32_t la = lds0 + (uint32_t)stage * 2 * MOE_TILE_BYTES + (uint32_t)w * 64 * 128;
    const uint32_t lw = lds0 + (uint32_t)stage * 2 * MOE_TILE_BYTES + MOE_TILE_BYTES + (uint32_t)w * 16 * 512;
    if (i < 8) hx_g2l16_s(A + (long)kt * 128, a_vo[i], la + i * 1024);
    else if (BCOL) hx_g2l16_s(W + ((long)kt0 + kt) * 128, wc_vo[BCOL ? i - 8 : 0], lds0 + (uint32_t)stage * 2 * MOE_TILE_BYTES + MOE_TILE_BYTES + (uint32_t)w * 64 * 128 + (i - 8) * 1024);
    else hx_g2l16_s(We + ((long)kt * MOE_BK + 2 * (i - 8)) * d.ldb * 2, w_vo[i - 8], lw + (i - 8) * 1024);
  };
  auto issue = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < 16; ++i) issue_one(kt, stage, i);
  };

  // ---- operand addressing
  const int r16 = lane & 15, g = lane >> 4;
  const int ax = (g ^ ((r16 >> 1) & 7)) * 16;  // chunk (4*ks + g) ^ swz -> ax ^ (ks*64)
  const int a_base = (wm * 128 + r16) * 128;
  // transposing read: lane -> (group g = lane>>4, e = (lane>>2)&3, q = lane&3) supplies 8 bytes of
  //   k = 32*ks + 8*g + 4*half + e ; n = wn*128 + 16*bj + 4q   and receives column lane%16 of block bj, 4 k
  const int te = (lane >> 2) & 3, tq = lane & 3;
  const int tn_ = wn * 128 + 4 * tq;  // + 16*bj
  // byte offset of (k = 8g + e + 4*half, n = tn_) in the W tile.  Column block bj adds 2 to the chunk index in bits
  // the swizzle mask covers and tn_>>3 leaves alone, so it is an xor with 32*bj; k-step ks adds 32 rows = 16384 bytes.
  int w_off[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int k = 8 * g + te + 4 * half;
    w_off[half] = k * 512 + (((tn_ >> 3) ^ (moe_wswz(k) << 1)) * 16) + (tn_ & 7) * 2;
  }

  // acc[bj][bi][r] is C[row_of(wm*128 + 16 bi + lane%16)][n0 + wn*128 + 16 bj + 4*(lane/16) + r]
  v4f acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  // fragment f (0..15) of k-step ks (32 k) of a stage: f < 8 -> A rows 16f.. (one b128), else W columns 16(f-8)..
  // (two transposing b64 reads, or one b128 of a column-major W)
  auto load_frag = [&](V8(&af)[8], V8(&wf)[8], int stage, int ks, int f) {
    if (f < 8) {
      af[f] = *(const V8*)(&smem[stage][0][0] + a_base + f * 2048 + (ax ^ (ks * 64)));
    } else if (BCOL) {
      wf[f - 8] = *(const V8*)(&smem[stage][1][0] + (wn * 128 + r16) * 128 + (f - 8) * 2048 + (ax ^ (ks * 64)));
    } else {
      const uint8_t* sw = &smem[stage][1][0];
      v4s part[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int off = (w_off[half] ^ ((f - 8) * 32)) + ks * 16384;
        part[half] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3)))*)(sw + off));
      }
      v8s both = (v8s){part[0][0], part[0][1], part[0][2], part[0][3], part[1][0], part[1][1], part[1][2], part[1][3]};
      wf[f - 8] = __builtin_bit_cast(V8, both);
    }
  };
  // The fragments of a whole k-tile live in registers (2 k-steps x (8 A + 8 W) = 128 VGPRs) and are refilled in place
  // with the next tile's as they die, always a good part of a tile before their next use, so that an LDS read slowed
  // down by the DMA writing the same LDS never holds up an MFMA.  One k-tile:
  //   first half  (k-step 0): 64 MFMAs and nothing else;
  //   barrier: tile kt+1 has landed in the other stage, and the last reads of this stage (issued at the end of the
  //            previous tile) are complete: it is free;
  //   second half (k-step 1): 64 MFMAs, behind them the refills - k-step 0's fragments under the first 32, k-step 1's
  //            own each behind its last MFMA - and the 16 DMA instructions of tile kt+2 into the free stage, one every
  //            fourth MFMA.  Past the last tile the last one is fetched again and the refills read whatever the other
  //            stage holds: every tile runs the same code.
  V8 fa[2][8], fw[2][8];  // [k-step][row block], [k-step][column block]
  auto mfma_ks = [&](int ks, auto after) {
#pragma unroll
    for (int i = 0; i < 64; ++i) {
      acc[i >> 3][i & 7] = Mfma16<BF>::run16(fw[ks][i >> 3], fa[ks][i & 7], acc[i >> 3][i & 7]);
      after(i);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  issue(0, 0);
  if (nk > 1) issue(1, 1);
  if (nk > 1) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(16)); else HX_WAIT_VM0();
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int f = 0; f < 16; ++f) load_frag(fa[ks], fw[ks], 0, ks, f);
  constexpr bool EARLY = MODE == 0;
  if (EARLY) __syncthreads();  // ... of stage 0
  for (int kt = 0; kt < nk; ++kt) {
    const int stage = kt & 1, dkt = min(kt + 2, nk - 1);
    // EARLY (grouped mode): a second barrier at the end of the tile frees the stage a half tile sooner, so the DMA of
    // tile kt+2 goes out under the first half and has a whole tile to land (C5 -1 %; the dense instantiations
    // measured 1-2 % slower with it, and those with an epilogue then compile with accumulator copies inside the loop).
    mfma_ks(0, [&](int i) {
      if (EARLY && (i & 3) == 3) issue_one(dkt, stage, i >> 2);
    });
    if (EARLY) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(16));  // tile kt+1, issued a tile ago, has landed; tile kt+2 stays in flight
    else HX_WAIT_VM0();
    __syncthreads();
    mfma_ks(1, [&](int i) {
      if (i < 32 && !(i & 1)) load_frag(fa[0], fw[0], stage ^ 1, 0, i >> 1);
      if (!EARLY && (i & 3) == 3) issue_one(dkt, stage, i >> 2);
      if ((i & 7) == 7) load_frag(fa[1], fw[1], stage ^ 1, 1, 8 + (i >> 3));  // W fragment i>>3: its eight MFMAs are out
      if (i >= 56) load_frag(fa[1], fw[1], stage ^ 1, 1, i - 56);              // A fragment i-56: last used by MFMA i
    });
    if (EARLY) __syncthreads();  // every wave has read tile kt+1's fragments out of the other stage: it is free
  }
  HX_WAIT_VM0();  // trailing re-fetches must land before the workgroup's LDS is released

  // ---- epilogue: acc[bj][bi][r] is C[row_of(wm*128 + 16 bi + lane%16)][n0 + wn*128 + 16 bj + 4g + r].
  const long ncol = n0 + wn * 128 + 4 * g;
  // A lane holds 4 consecutive columns of a row, so direct stores would hit every 128-byte line of C with sixteen
  // separate 8-byte writes, and the write burst at the end of a round of tiles becomes L2-transaction-bound.  Each wave
  // instead passes 32 rows x 128 columns at a time through its own quarter of the (now idle) LDS and writes whole
  // 256-byte row pieces: 16 bytes per lane, consecutive lanes on consecutive bytes.  The matrix rows of the wave's
  // 128 tile rows (gathered in the grouped mode) go through the LDS as well.
  out_t* C = (out_t*)Cv;
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
  __syncthreads();  // every wave is past its last fragment read: the LDS can be reused
  constexpr int RSTR = 256 + 16;   // padded row stride of a staging block
  constexpr int BLK = 32 * RSTR;
  uint8_t* st = &smem[0][0][0] + w * MOE_TILE_BYTES;  // this wave's 32 KB: two staging blocks, then the row table
  int* srow = (int*)(st + 2 * BLK);
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int lr = wm * 128 + p * 64 + lane;
    srow[p * 64 + lane] = lr < mt.rows ? row_of(lr) : -1;  // -1: not stored
  }
  if (MODE == 2) {  // fp32 accumulators as they are: 16 rows x 128 columns per staging block, two rows per store instruction
    float* Cp = (float*)Cv + (long)blockIdx.y * T * d.ldc;
    constexpr int RS2 = 512 + 16, BLK2 = 16 * RS2;
    const int q_row = lane >> 5, q_ch = lane & 31;
    const long ncol4 = n0 + wn * 128 + q_ch * 4;
#pragma unroll
    for (int bb = 0; bb < 9; ++bb) {
      if (bb < 8) {
        uint8_t* sb = st + (bb & 1) * BLK2 + r16 * RS2 + 16 * g;
#pragma unroll
        for (int bj = 0; bj < 8; ++bj) {
          v4f t = acc[bj][bb];
          asm volatile("" : "+v"(t));  // a copy the compiler cannot fold into the accumulator's own register
          *(v4f*)(sb + bj * 64) = t;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      if (bb >= 1) {
        const uint8_t* sb = st + ((bb - 1) & 1) * BLK2;
#pragma unroll
        for (int p = 0; p < 8; ++p) {
          const int row = p * 2 + q_row;
          const int r = srow[(bb - 1) * 16 + row];
          const v4i v = *(const v4i*)(sb + row * RS2 + q_ch * 16);
          if (r >= 0 && ncol4 < N) *(v4i*)(Cp + (long)r * d.ldc + ncol4) = v;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    return;
  }
  v4f bv[8];  // MODE 1: bias of this lane's columns n0 + wn*128 + 16 bj + 4 g ..+3
  if (MODE == 1) {
#pragma unroll
    for (int bj = 0; bj < 8; ++bj) {
      bv[bj] = (v4f){0.f, 0.f, 0.f, 0.f};
      const long n = ncol + bj * 16;
      if (d.bias && n < N) {
        if (d.bias_f32) {
          bv[bj] = *(const v4f*)((const float*)d.bias + n);
        } else {
          const ov4 b16 = *(const ov4*)((const out_t*)d.bias + n);
          bv[bj] = (v4f){(float)b16[0], (float)b16[1], (float)b16[2], (float)b16[3]};
        }
      }
    }
  }
  auto stage_rows = [&](int bb) {  // accumulators of tile rows 32 bb .. +31 of this wave -> staging block bb % 2
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint8_t* sb = st + (bb & 1) * BLK + (16 * h + r16) * RSTR + 8 * g;
#pragma unroll
      for (int bj = 0; bj < 8; ++bj) {
        ov4 o;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          float v = acc[bj][2 * bb + h][b];
          if (MODE == 1) {
            v += bv[bj][b];
            if (d.relu) v = fmaxf(v, 0.f);
          }
          o[b] = (out_t)v;
        }
        *(ov4*)(sb + bj * 32) = o;
      }
    }
  };
  const int rb_row = lane >> 4, rb_ch = lane & 15;  // on the way out: 16 lanes per row, 4 rows per store instruction
  const long ncol8 = n0 + wn * 128 + rb_ch * 8;    // N % 8 == 0: an 8-column piece is wholly inside the row or outside
  auto drain = [&](int bb) {
    const uint8_t* sb = st + (bb & 1) * BLK;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int row = p * 4 + rb_row;
      const int r = srow[bb * 32 + row];
      const v4i v = *(const v4i*)(sb + row * RSTR + rb_ch * 16);
      // (non-temporal: the output is written once and not read here, and lines of it lingering in the L2s displace operand
      // panels: dense 8192^3 -4 %, grouped +-0)
      if (r >= 0 && ncol8 < N) __builtin_nontemporal_store(v, (v4i*)(C + (long)r * d.ldc + ncol8));
    }
  };
  // The LDS executes one wave's operations in order, so a block may be refilled as soon as the reads that drain it
  // have been issued; the fences only pin that program order.  With two blocks the conversion of the next row block
  // runs under the LDS and store latency of the previous one.
#pragma unroll
  for (int bb = 0; bb < 5; ++bb) {
    if (bb < 4) stage_rows(bb);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    if (bb >= 1) drain(bb - 1);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}
