// 32x128x64 tile kernel for grouped 16-bit GEMMs whose row tiles hold only a few rows: experts with a decode batch's
// worth of rows each.  Such a launch streams every weight once and does almost no arithmetic, so what
// counts is how many weight bytes a CU keeps in flight against the memory latency; a 128-row A tile would spend half
// of the LDS on padding rows.  Here a stage is A 4 KB + W 16 KB, and NS - 1 stages are in flight per workgroup
// (NS = 3: 60 KB, two workgroups per CU).
//   A tile [32 rows][128 B], W tile [64 k][256 B]: the layouts and swizzles of the 128-row kernel.
// 4 waves, wave w owns columns [32w, 32w+32) of the tile: one 32x32x16 MFMA per k-step, fragments read straight
// before use.  Past the last k-tile the DMA fetches the last tile again so that the counted waits stay exact.
#pragma once
#include "gemm16_tile256.h"

#define R32_BM 32
#define R32_BN 128
#define R32_A_BYTES (32 * 128)
#define R32_STAGE_BYTES (R32_A_BYTES + 64 * 256)

template <bool BF, int NS>
__global__ __launch_bounds__(256, NS <= 3 ? 2 : 1) void hx_gemm16_rows32(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                                                                        void* __restrict__ Cv, const int* __restrict__ num_tiles,
                                                                        const MoeTile* __restrict__ table,
                                                                        const int32_t* __restrict__ idx, int T, int K, int N,
                                                                        int max_tiles, int tiles_n, int a_div, G16Dense d) {
  typedef typename Mfma16<BF>::T out_t;
  typedef typename Mfma16<BF>::V8 V8;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NS][R32_STAGE_BYTES];  // [stage][A | W]

  // neighbouring workgroups take neighbouring column tiles of one row tile: together they read whole rows of W
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
  if (tm >= *num_tiles) return;
  const MoeTile mt = table[tm];
  auto row_of = [&](int lr) {  // matrix row of tile row lr (< mt.rows)
    const int r = idx[mt.row_start + lr];
    return (r >= 0 && r < T) ? r : -1;
  };
  const int nk = K / MOE_BK;
  const long n0 = (long)tn * R32_BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- A DMA: wave w owns tile rows [8w, 8w+8), one instruction
  const int lrow = lane >> 3, lpos = lane & 7;
  uint32_t a_vo;
  {
    const int pos_row = w * 8 + lrow;
    int r = row_of(pos_row < mt.rows ? pos_row : 0);  // padded rows re-read row 0 of the tile; never stored
    r = r < 0 ? 0 : r;
    a_vo = (uint32_t)(r / a_div) * (uint32_t)(d.lda * 2) + (uint32_t)((lpos ^ ((pos_row >> 1) & 7)) * 16);
  }
  // ---- W DMA: wave w owns k rows [16w, 16w+16), 4 instructions of 4 rows x 256 B; row k = 16w + 4j + (lane>>4), so
  // k & 3 and with it the swizzle do not depend on j.  Chunks past a ragged N re-read the last valid one.
  const uint8_t* We = W + (long)mt.expert * K * N * 2 + n0 * 2 + (long)(w * 16) * d.ldb * 2;  // wave-uniform
  const int wk_l = lane >> 4, wpos = lane & 15;
  const int cmax = (int)((min((long)N - n0, (long)R32_BN) >> 3) - 1);
  const uint32_t w_vo = (uint32_t)(wk_l * d.ldb * 2 + min(wpos ^ (wk_l << 2), cmax) * 16);
  const uint32_t lds0 = hx_lds_addr(&smem[0][0]);
  auto issue = [&](int kt_unclamped) {  // this wave's 5 DMA instructions of k-tile kt into stage kt % NS
    const int kt = min(kt_unclamped, nk - 1), stage = kt_unclamped % NS;
    const uint32_t la = lds0 + (uint32_t)stage * R32_STAGE_BYTES + (uint32_t)w * 1024;
    const uint32_t lw = lds0 + (uint32_t)stage * R32_STAGE_BYTES + R32_A_BYTES + (uint32_t)w * 16 * 256;
    hx_g2l16_s(A + (long)kt * 128, a_vo, la);
#pragma unroll
    for (int j = 0; j < 4; ++j) hx_g2l16_s_nt(We + ((long)kt * MOE_BK + 4 * j) * d.ldb * 2, w_vo, lw + j * 1024);  // W: read once
  };

  // ---- operand addressing (see the 128-row kernel): A fragment of k-step ks at a_base + (ax ^ (ks * 32)); the two
  // transposing reads of W at w_off[half] + ks * 4096
  const int r31 = lane & 31, g = lane >> 5;
  const int ax = (g ^ ((r31 >> 1) & 7)) * 16;
  const int a_base = r31 * 128;
  const int tb = lane >> 4, te = (lane >> 2) & 3, tq = lane & 3;
  int w_off[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int k = 8 * (tb >> 1) + 4 * half + te;
    const int chunk = 4 * w + 2 * (tb & 1) + (tq >> 1);
    w_off[half] = k * 256 + ((chunk ^ ((k & 3) << 2)) * 16) + (tq & 1) * 8;
  }

  v16f acc[2];  // even and odd k-steps, summed at the end: two independent MFMA chains
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;

  for (int t = 0; t < NS - 1; ++t) issue(t);
  for (int kt = 0; kt < nk; ++kt) {
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((NS - 2) * 5));  // this wave's part of tile kt has landed
    __syncthreads();  // ... everybody's has, and every wave is done reading tile kt-1: its stage is free
    issue(kt + NS - 1);
    const uint8_t* sa = &smem[kt % NS][0];
    const uint8_t* sw = sa + R32_A_BYTES;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const V8 af = *(const V8*)(sa + a_base + (ax ^ (ks * 32)));
      v4s part[2];
#pragma unroll
      for (int half = 0; half < 2; ++half)
        part[half] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3)))*)(sw + w_off[half] + ks * 4096));
      const v8s both = (v8s){part[0][0], part[0][1], part[0][2], part[0][3], part[1][0], part[1][1], part[1][2], part[1][3]};
      acc[ks & 1] = Mfma16<BF>::run(__builtin_bit_cast(V8, both), af, acc[ks & 1]);
    }
  }
  HX_WAIT_VM0();  // no DMA may still be writing this workgroup's LDS when it ends

  // ---- epilogue: acc[4a+b] is C[row_of(lane%32)][n0 + 32w + 8a + 4g + b].  N % 8 == 0 and a piece starts at a
  // multiple of 4: it is either wholly inside the row or wholly outside.
  const int rr = r31 < mt.rows ? row_of(r31) : -1;
  if (rr < 0) return;
  const long ncol = n0 + 32 * w + 4 * g;
  out_t* crow = (out_t*)Cv + (long)rr * d.ldc + ncol;
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const long n = ncol + 8 * a;
    if (n >= N) continue;
    ov4 o;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      o[b] = (out_t)(acc[0][4 * a + b] + acc[1][4 * a + b]);
    }
    *(ov4*)(crow + 8 * a) = o;
  }
}
