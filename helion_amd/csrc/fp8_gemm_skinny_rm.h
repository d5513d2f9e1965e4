// hx_fp8_gemm_skinny_rm: the decode-shape FP8 GEMM (M <= 32) for a ROW-major B ([K][N], N contiguous - the layout the
// reference's own check feeds, examples/fp8_gemm.py:105-108), read in place.  HBM-bound: every byte of B is fetched once,
// in whole 128-byte lines.
//
// A workgroup (4 waves) owns column groups of 128 columns; the waves split the workgroup's k range in four.  A wave streams
// its part of the strip as slices of 32 k-rows x 128 bytes (4 KB = four DMA instructions of 8 rows each) through a
// private ring of 8 slices in the LDS: seven slices (28 KB per wave, 112 KB per CU) are in flight while one is consumed,
// and since nobody else touches a wave's ring the loop needs no barrier - a slice is refilled one step after the wave's
// own reads of it.  Within a slice the 16-byte chunk c of row r sits at position c ^ (r & 7) (the DMA's source address
// does the permutation), so the eight rows a transposing read touches come from eight different bank groups.
// One ds_read_b64_tr_b8 hands lane (i = lane % 16, g = lane / 16) the 8 bytes B[8g .. 8g+7][16 cb + i] of a slice, which
// is exactly this lane's operand of v_mfma_f32_16x16x32_fp8_fp8; the A operand (row lane % 16 of A, the same 8 k) stays
// in registers for the whole kernel (K / 4 / 32 steps x 2 registers per 16-row block).  B is the first MFMA operand, so a
// lane ends up with 4 consecutive columns of one row of C.
// At the end of a column group the four partial sums meet in the LDS (32 KB next to the rings), are added in a fixed
// order, scaled, cast and stored as whole 16-byte pieces; the next group's first seven slices are already in flight.
// When the column groups alone would leave most CUs idle the k range is also split over gridDim.y: each split writes an
// unscaled fp32 slab and hx_fp8_gemm_split_reduce adds them up.
#pragma once
#include "hx_common.h"

#define SKR_WAVES 4
#define SKR_RS 8                   // ring slots per wave
#define SKR_SLICE (32 * 128)       // bytes per slice
#define SKR_COLS 128               // columns per group

// NSTEP: slices (32 k) per wave, a multiple of SKR_RS; the workgroup covers 128 * NSTEP k.
// BNT: B is larger than the memory-side cache can keep between calls: its DMA carries the non-temporal hint.
template <int OUT, int MB, int NSTEP, bool BNT>
__global__ __launch_bounds__(256) void hx_fp8_gemm_skinny_rm(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                            typename OutT<OUT>::T* __restrict__ C, int M, int N, long lda, long ldb,
                                                            long ldc, const float* __restrict__ scale_a,
                                                            const float* __restrict__ scale_b, int ngroups, long split_stride) {
  typedef typename OutT<OUT>::T out_t;
  static_assert(NSTEP % SKR_RS == 0, "ring slots are compile-time constants");
  __shared__ __attribute__((aligned(1024))) uint8_t ring[SKR_WAVES][SKR_RS][SKR_SLICE];
  __shared__ __attribute__((aligned(16))) float part[SKR_WAVES][16][SKR_COLS];

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const long kw0 = (long)blockIdx.y * (128L * NSTEP) + (long)w * (32L * NSTEP);  // first k of this wave
  C += (long)blockIdx.y * split_stride;

  // ---- A operands: row min(16 mb + i16, M - 1), k = kw0 + 32 s + 8 g .. + 7
  long af[MB][NSTEP];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const uint8_t* ap = A + (long)min(mb * 16 + i16, M - 1) * lda + kw0 + 8 * g;
#pragma unroll
    for (int s = 0; s < NSTEP; ++s) af[mb][s] = *(const long*)(ap + 32 * s);
  }
  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;
  HX_WAIT_VM0();  // from here on the only memory operations in flight are this wave's DMA instructions (and C's stores)

  // ---- this workgroup's column groups: blockIdx.x, + gridDim.x, ...
  const int gstride = (int)gridDim.x;
  const int ngm = (ngroups - (int)blockIdx.x + gstride - 1) / gstride;  // >= 1: the grid has at most `ngroups` columns of workgroups
  // DMA source of a slice: instruction j fetches rows 8j + lane/8; LDS position lane%8 of row r takes chunk (lane%8) ^ (r&7);
  // chunks past the end of a ragged last group re-read its last valid chunk (those columns are never stored)
  const int drow = lane >> 3, dchunk = (lane & 7) ^ drow;
  auto voff_of = [&](int grp) {
    const int nch = min(8, (N - grp * SKR_COLS) >> 4);
    return (uint32_t)(drow * ldb + min(dchunk, nch - 1) * 16);
  };
  const uint8_t* Bw = B + kw0 * ldb;  // this wave's first k-row
  const uint32_t ring0 = hx_lds_addr(&ring[0][0][0]) + (uint32_t)w * (SKR_RS * SKR_SLICE);
  auto issue = [&](const uint8_t* colbase, uint32_t voff, int s, int slot) {  // slice s of the group at colbase -> ring slot
    const uint8_t* base = colbase + (long)(32 * s) * ldb;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (BNT) hx_g2l16_s_nt(base + (long)(8 * j) * ldb, voff, ring0 + slot * SKR_SLICE + j * 1024);
      else hx_g2l16_s(base + (long)(8 * j) * ldb, voff, ring0 + slot * SKR_SLICE + j * 1024);
    }
  };
  // transposing read of column block cb out of a slice: row 8g + i16/2, position cb ^ (row & 7), half i16 & 1
  const int tr_off = (8 * g + (i16 >> 1)) * 128 + ((i16 >> 1) * 16) + (i16 & 1) * 8;
  const uint8_t* myring = &ring[0][0][0] + w * (SKR_RS * SKR_SLICE);

  int grp = (int)blockIdx.x;
  const uint8_t* cur = Bw + (long)grp * SKR_COLS;
  uint32_t vcur = voff_of(grp);
#pragma unroll
  for (int s = 0; s < SKR_RS - 1; ++s) issue(cur, vcur, s, s);

  for (int gi = 0; gi < ngm; ++gi) {
    // the group after this one (the last group: itself again - its first slices are then re-fetched into slots nobody
    // reads any more, so that every step issues the same number of DMA instructions and the waits are constants)
    const int ngrp = gi + 1 < ngm ? grp + gstride : grp;
    const uint8_t* nxt = Bw + (long)ngrp * SKR_COLS;
    const uint32_t vnxt = voff_of(ngrp);
    v4f acc[MB][8];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int cb = 0; cb < 8; ++cb) acc[mb][cb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NSTEP; ++s) {
      constexpr int RS = SKR_RS;
      // slices s+1 .. s+RS-2 (of this group or the next) may still be in flight; slice s has landed
      __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(4 * (RS - 2)));
      const uint8_t* sl = myring + (s % RS) * SKR_SLICE;
      long bf[8];
#pragma unroll
      for (int cb = 0; cb < 8; ++cb) {
        const v2i t = __builtin_amdgcn_ds_read_tr8_b64_v2i32((v2i __attribute__((address_space(3)))*)(sl + (tr_off ^ (cb * 16))));
        bf[cb] = ((long)(unsigned)t[1] << 32) | (unsigned)t[0];
      }
#pragma unroll
      for (int cb = 0; cb < 8; ++cb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb][cb] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(bf[cb], af[mb][s], acc[mb][cb], 0, 0, 0);
      // refill the slot consumed one step ago (slot (s - 1) % RS == (s + RS - 1) % RS) with slice s + RS - 1
      if (s + RS - 1 < NSTEP) issue(cur, vcur, s + RS - 1, (s + RS - 1) % RS);
      else issue(nxt, vnxt, s + RS - 1 - NSTEP, (s + RS - 1) % RS);
    }
    // ---- the four waves' partial sums meet in the LDS, one 16-row block at a time:
    // acc[mb][cb][r] is C[16 mb + i16][128 grp + 16 cb + 4 g + r] summed over this wave's k
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int cb = 0; cb < 8; ++cb) *(v4f*)&part[w][i16][cb * 16 + 4 * g] = acc[mb][cb];
      __syncthreads();
      {
        const int row = tid >> 4, c8 = (tid & 15) * 8;
        v4f lo = *(const v4f*)&part[0][row][c8], hi = *(const v4f*)&part[0][row][c8 + 4];
#pragma unroll
        for (int ww = 1; ww < SKR_WAVES; ++ww) {
          lo += *(const v4f*)&part[ww][row][c8];
          hi += *(const v4f*)&part[ww][row][c8 + 4];
        }
        const int m = mb * 16 + row;
        const long n = (long)grp * SKR_COLS + c8;
        if (m < M && n < N) {  // N % 16 == 0: the eight columns are valid together
          out_t o[8];
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            o[b] = (out_t)(lo[b] * alpha);
            o[4 + b] = (out_t)(hi[b] * alpha);
          }
          out_t* dst = C + (long)m * ldc + n;
          if (((uintptr_t)dst & 15) == 0) {
#pragma unroll
            for (int q = 0; q < (int)(8 * sizeof(out_t)) / 16; ++q) ((v4i*)dst)[q] = ((const v4i*)o)[q];
          } else {
#pragma unroll
            for (int b = 0; b < 8; ++b) dst[b] = o[b];
          }
        }
      }
      __syncthreads();  // the partial-sum area is free again
    }
    grp = ngrp;
    cur = nxt;
    vcur = vnxt;
  }
}
