// MoE grouped GEMM for gfx950 — device side of examples/moe_matmul_ogs.py:25-80 of the reference
// (semantics: moe_matmul_ogs_reference, :125-148):
//   for expert e, i < counts[e]:  r = idx[offsets[e] + i];   C[r, :] = cast(A[r, :] @ W[e])
//   rows of C that no expert covers are zero.
// A [T,K], W [E,K,N] (N contiguous), C [T,N]; bf16 or fp16; fp32 accumulation.
//
// Launch sequence (all on the caller's stream, no host synchronisation):
//   1. hx_moe_prep       : builds the tile table (tile -> expert, first sorted row, row count) from
//                          counts/offsets on the device and clears the row-covered flags;
//   2. hx_moe_mark       : flags every row some expert covers;
//   3. hx_moe_tile256 / hx_moe_general : the grouped GEMM over (row tile, column tile) pairs;
//   4. hx_moe_zero_rows  : zero-fills rows whose flag is still clear.
// Padded rows of a tile are never stored, so there is no read-modify-write and no write race.
#include "hx_common.h"

struct MoeTile {
  int expert;
  int row_start;  // position in the sorted order (index into idx)
  int rows;       // valid rows in this tile (1..BM)
  int pad;
};

// workspace layout: [0] int num_tiles | [16 ..) MoeTile table[max_tiles] | flags[T] bytes
static inline size_t moe_table_bytes(int64_t max_tiles) { return 16 + (size_t)max_tiles * sizeof(MoeTile); }
static inline int64_t moe_max_tiles(int64_t T, int64_t E, int bm) { return (T + bm - 1) / bm + E; }

__global__ void hx_moe_prep(const int32_t* __restrict__ counts, const int32_t* __restrict__ offsets, int E, int T, int bm,
                            int max_tiles, int* __restrict__ num_tiles, MoeTile* __restrict__ table, uint8_t* __restrict__ flags) {
  const int tid = blockIdx.x * blockDim.x + threadIdx.x, nth = gridDim.x * blockDim.x;
  for (int i = tid; i < T; i += nth) flags[i] = 0;
  if (blockIdx.x != 0) return;
  // block 0: each thread walks the experts whose index is congruent to it, after a serial prefix
  // of tile counts (E is small: tens to a few thousand)
  __shared__ int s_total;
  if (threadIdx.x == 0) {
    int t = 0;
    for (int e = 0; e < E; ++e) {
      int c = counts[e];
      c = c < 0 ? 0 : c;
      const int start = offsets[e];
      // clamp malformed tables so the GEMM never indexes outside idx[0..T)
      if (start < 0 || start > T) c = 0;
      if (c > T - start) c = T - start;
      const int nt = (c + bm - 1) / bm;
      for (int i = 0; i < nt && t < max_tiles; ++i, ++t) {
        table[t].expert = e;
        table[t].row_start = start + i * bm;
        table[t].rows = min(bm, c - i * bm);
        table[t].pad = 0;
      }
    }
    s_total = t;
    *num_tiles = t;
  }
}

__global__ void hx_moe_mark(const int* __restrict__ num_tiles, const MoeTile* __restrict__ table, const int32_t* __restrict__ idx,
                            int T, uint8_t* __restrict__ flags) {
  const int nt = *num_tiles;
  for (int t = blockIdx.x; t < nt; t += gridDim.x) {
    const MoeTile mt = table[t];
    for (int i = threadIdx.x; i < mt.rows; i += blockDim.x) {
      const int r = idx[mt.row_start + i];
      if (r >= 0 && r < T) flags[r] = 1;
    }
  }
}

template <typename T16>
__global__ void hx_moe_zero_rows(T16* __restrict__ C, long ldc, int T, int N, const uint8_t* __restrict__ flags) {
  const int row = blockIdx.x;
  if (row >= T || flags[row]) return;
  T16* c = C + (long)row * ldc;
  for (int n = threadIdx.x; n < N; n += blockDim.x) c[n] = (T16)0.f;
}

// ------------------------------------------------------------------------------------------
// tile256: 256 gathered rows x 256 columns x 64 k per step; 4 waves (2x2) of 128x128; 32x32x16 MFMA.
//   A tile  [256 rows][128 B]  : same chunk-swizzled layout as the fp8 GEMM; the DMA gathers rows
//                                through idx, so the gather costs nothing extra.
//   W tile  [64 k][512 B]      : row = k, 32 chunks of 8 columns; chunk stored at pos = chunk ^ (moe_wswz(k)<<1).
//                                The MFMA wants 8 consecutive k per lane for one column, W has the
//                                columns contiguous: ds_read_b64_tr_b16 transposes 4(k) x 16(n) blocks
//                                on the way out of LDS (two reads per operand).
// ------------------------------------------------------------------------------------------
// Swizzle of a W-tile row, in units of 32 bytes (a pair of chunks).  One transposing read has the 32 lanes
// that the LDS serves together fetch 4 consecutive k rows x two adjacent 32-byte column groups; rows are 512 B
// apart (the same banks), so the 8 (row, group) combinations must land in 8 different 32-byte bank groups:
// k&3 goes to bits 2:1 and bit 2 of k to bit 0, which the column-group bit then flips.
__device__ __forceinline__ int moe_wswz(int k) { return ((k & 3) << 1) | ((k >> 2) & 1); }

template <bool BF>
struct Mfma16;
template <>
struct Mfma16<true> {
  typedef __bf16 T;
  typedef v8bf V8;
  static __device__ __forceinline__ v16f run(v8bf a, v8bf b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <>
struct Mfma16<false> {
  typedef _Float16 T;
  typedef v8h V8;
  static __device__ __forceinline__ v16f run(v8h a, v8h b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

#define MOE_BM 256
#define MOE_BN 256
#define MOE_BK 64
#define MOE_TILE_BYTES (256 * 128)

template <bool BF>
__global__ __launch_bounds__(256) void hx_moe_tile256(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                                                     typename Mfma16<BF>::T* __restrict__ C, const int* __restrict__ num_tiles,
                                                     const MoeTile* __restrict__ table, const int32_t* __restrict__ idx, int T, int K,
                                                     int N, int max_tiles, int tiles_n, int a_div) {
  typedef typename Mfma16<BF>::T out_t;
  typedef typename Mfma16<BF>::V8 V8;
  // [stage][A|W][32 KB]
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2][2][MOE_TILE_BYTES];

  // XCD-contiguous grouped raster over (row tile, column tile), as in the fp8 GEMM
  int tile;
  {
    const int nwg = gridDim.x, wg = blockIdx.x;
    const int per = nwg >> 3, rem = nwg & 7, xcd = wg & 7, loc = wg >> 3;
    tile = (xcd < rem) ? xcd * (per + 1) + loc : rem * (per + 1) + (xcd - rem) * per + loc;
  }
  const int GM = 8;
  const int group_size = GM * tiles_n;
  const int gid = tile / group_size;
  const int first_m = gid * GM;
  const int gm = min(max_tiles - first_m, GM);
  const int tm = first_m + (tile % group_size) % gm;
  const int tn = (tile % group_size) / gm;
  if (tm >= *num_tiles) return;
  const MoeTile mt = table[tm];
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
    int r = idx[mt.row_start + lr];
    r = (r >= 0 && r < T) ? r : 0;
    const int swz = ((j & 1) ? 4 + (lrow >> 1) : (lrow >> 1)) & 7;
    // a_div > 1: C row r is the product of A row r / a_div (top-k routing without a replicated A)
    a_vo[j] = (uint32_t)(r / a_div) * (uint32_t)(K * 2) + (uint32_t)((lpos ^ swz) * 16);
  }
  // ---- W DMA: wave w owns k rows [16w, 16w+16), 8 instructions of 2 rows x 512 B.
  // row k = 16w + 2j + (lane>>5); chunk = (lane&31) ^ (moe_wswz(k)<<1); k&7 = (2j + (lane>>5)) & 7
  const uint8_t* We = W + (long)mt.expert * K * N * 2 + n0 * 2 + (long)(w * 16) * N * 2;  // wave-uniform
  const int wk_l = lane >> 5, wpos = lane & 31;
  uint32_t w_vo[4];
  // The last column tile may be ragged (N % 256 != 0, N % 8 == 0): chunks past the end re-read the last valid chunk of
  // the row; the columns they feed are never stored.
  const int cmax = (int)((min((long)N - n0, (long)MOE_BN) >> 3) - 1);
#pragma unroll
  for (int j = 0; j < 4; ++j) w_vo[j] = (uint32_t)(wk_l * N * 2 + min(wpos ^ (moe_wswz(2 * j + wk_l) << 1), cmax) * 16);
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]);

  // DMA instruction i (0..15) of a k-tile: i < 8 -> gathered A rows 64w + 8i .., else W k-rows 16w + 2(i-8), +1
  auto issue_one = [&](int kt, int stage, int i) {
    const uint32_t la = lds0 + (uint32_t)stage * 2 * MOE_TILE_BYTES + (uint32_t)w * 64 * 128;
    const uint32_t lw = lds0 + (uint32_t)stage * 2 * MOE_TILE_BYTES + MOE_TILE_BYTES + (uint32_t)w * 16 * 512;
    if (i < 8) hx_g2l16_s(A + (long)kt * 128, a_vo[i], la + i * 1024);
    else hx_g2l16_s(We + (long)kt * MOE_BK * N * 2 + (long)(2 * (i - 8)) * N * 2, w_vo[(i - 8) & 3], lw + (i - 8) * 1024);
  };
  auto issue = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < 16; ++i) issue_one(kt, stage, i);
  };

  // ---- operand addressing
  const int r31 = lane & 31, g = lane >> 5;
  const int ax = (g ^ ((r31 >> 1) & 7)) * 16;  // chunk (2*ks + g) ^ swz -> ax ^ (ks*32)
  const int a_base = (wm * 128 + r31) * 128;
  // transposing read: lane -> (block b = lane>>4, e = (lane>>2)&3, q = lane&3)
  //   k = 16*ks + 8*(b>>1) + 4*half + e ; n = wn*128 + 32*bj + 16*(b&1) + 4q
  const int tb = lane >> 4, te = (lane >> 2) & 3, tq = lane & 3;
  const int tk = 8 * (tb >> 1) + te;                  // + 16*ks + 4*half
  const int tn_ = wn * 128 + 16 * (tb & 1) + 4 * tq;  // + 32*bj
  // byte offset of (k = tk + 4*half, n = tn_) in the W tile.  Column block bj adds 4 to the chunk index in bits
  // the swizzle mask and tn_>>3 leave alone, so it is an xor with 64*bj; k-step ks adds 16 rows = 8192 bytes.
  int w_off[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int k = tk + 4 * half;
    w_off[half] = k * 512 + (((tn_ >> 3) ^ (moe_wswz(k) << 1)) * 16) + (tn_ & 7) * 2;
  }

  v16f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // fragment f (0..7) of k-step ks (16 k) of a stage: f < 4 -> A rows 32f.. (one b128), else W columns 32(f-4)..
  // (two transposing b64 reads)
  auto load_frag = [&](V8(&af)[4], V8(&wf)[4], int stage, int ks, int f) {
    if (f < 4) {
      af[f] = *(const V8*)(&smem[stage][0][0] + a_base + f * 4096 + (ax ^ (ks * 32)));
    } else {
      const uint8_t* sw = &smem[stage][1][0];
      v4s part[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int off = (w_off[half] ^ ((f - 4) * 64)) + ks * 8192;
        part[half] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3)))*)(sw + off));
      }
      v8s both = (v8s){part[0][0], part[0][1], part[0][2], part[0][3], part[1][0], part[1][1], part[1][2], part[1][3]};
      wf[f - 4] = __builtin_bit_cast(V8, both);
    }
  };
  // One k-step: 16 MFMAs on the current fragments; pinned between them the 8 fragment loads of the next k-step and,
  // when DMA is set, NDMA DMA instructions starting at number D0 (one per MFMA), as in the fp8 GEMM.
  auto kstep = [&](V8(&ca)[4], V8(&cw)[4], V8(&na)[4], V8(&nw)[4], int nstage, int nks, bool load_next, bool dma, int dkt,
                   int dstage, int d0) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (load_next && i < 8) load_frag(na, nw, nstage, nks, i);
      acc[i >> 2][i & 3] = Mfma16<BF>::run(cw[i >> 2], ca[i & 3], acc[i >> 2][i & 3]);
      if (dma && (i & 1)) issue_one(dkt, dstage, d0 + (i >> 1));
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // software pipeline, as in the fp8 GEMM: k-tile kt in stage kt&1, four k-steps per tile, fragments double
  // buffered; the one barrier per tile sits before the last k-step's MFMAs; the 16 DMA instructions of tile kt+2 go
  // out under the MFMAs of (kt, ks=3) and (kt+1, ks=0), one every other MFMA.
  const int nk = K / MOE_BK;
  V8 fa0[4], fw0[4], fa1[4], fw1[4];
  issue(0, 0);
  if (nk > 1) issue(1, 1);
  if (nk > 1) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(16)); else HX_WAIT_VM0();
  __syncthreads();
#pragma unroll
  for (int f = 0; f < 8; ++f) load_frag(fa0, fw0, 0, 0, f);
  for (int kt = 0; kt < nk - 1; ++kt) {
    const int stage = kt & 1;
    // (kt, ks=0): second half of tile kt+1's DMA (its first half went out under (kt-1, ks=3)); stage^1 is free
    // since the last barrier, and both halves are complete at this iteration's barrier
    kstep(fa0, fw0, fa1, fw1, stage, 1, true, kt > 0, min(kt + 1, nk - 1), stage ^ 1, 8);
    kstep(fa1, fw1, fa0, fw0, stage, 2, true, false, 0, 0, 0);
    kstep(fa0, fw0, fa1, fw1, stage, 3, true, false, 0, 0, 0);
    HX_WAIT_VM0();
    __syncthreads();
    // (kt, ks=3): first half of tile kt+2's DMA into the stage just freed
    kstep(fa1, fw1, fa0, fw0, stage ^ 1, 0, true, true, min(kt + 2, nk - 1), stage, 0);
  }
  {
    const int stage = (nk - 1) & 1;
    kstep(fa0, fw0, fa1, fw1, stage, 1, true, nk > 1, nk - 1, stage ^ 1, 8);
    kstep(fa1, fw1, fa0, fw0, stage, 2, true, false, 0, 0, 0);
    kstep(fa0, fw0, fa1, fw1, stage, 3, true, false, 0, 0, 0);
    kstep(fa1, fw1, fa0, fw0, 0, 0, false, false, 0, 0, 0);
  }
  HX_WAIT_VM0();  // trailing re-fetches must land before the workgroup's LDS is released

  // ---- epilogue: acc[bj][bi][4a+b] is C[idx[row_start + wm*128 + bi*32 + lane%32]][n0 + wn*128 + bj*32 + 8a + 4g + b]
#pragma unroll
  for (int bi = 0; bi < 4; ++bi) {
    const int lr = wm * 128 + bi * 32 + r31;
    if (lr < mt.rows) {
      const int r = idx[mt.row_start + lr];
      if (r >= 0 && r < T) {
        out_t* crow = C + (long)r * N + n0 + wn * 128 + 4 * g;
#pragma unroll
        for (int bj = 0; bj < 4; ++bj)
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            typedef out_t ov4 __attribute__((ext_vector_type(4)));
            ov4 o;
#pragma unroll
            for (int b = 0; b < 4; ++b) o[b] = (out_t)acc[bj][bi][4 * a + b];
            // N % 8 == 0 and the piece starts at a multiple of 4: it is either wholly inside the row or wholly outside
            if (n0 + wn * 128 + 4 * g + bj * 32 + 8 * a < N) *(ov4*)(crow + bj * 32 + 8 * a) = o;
          }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// general: 64-row tiles, 64x64 outputs per workgroup, any K/N, fp32 FMAs
// ------------------------------------------------------------------------------------------
template <typename T16>
__global__ __launch_bounds__(256) void hx_moe_general(const T16* __restrict__ A, const T16* __restrict__ W, T16* __restrict__ C,
                                                     const int* __restrict__ num_tiles, const MoeTile* __restrict__ table,
                                                     const int32_t* __restrict__ idx, int T, int K, int N, int a_div) {
  const int tm = blockIdx.x;
  if (tm >= *num_tiles) return;
  const MoeTile mt = table[tm];
  __shared__ float sa[16][64 + 1];
  __shared__ float sb[16][64 + 1];
  __shared__ int srow[64];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  if (tid < 64) {
    int r = tid < mt.rows ? idx[mt.row_start + tid] : -1;
    srow[tid] = (r >= 0 && r < T) ? r : -1;
  }
  __syncthreads();
  const long n0 = (long)blockIdx.y * 64;
  const T16* We = W + (long)mt.expert * K * N;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int e = tid; e < 64 * 16; e += 256) {
      const int kk = e & 15, r = e >> 4;
      const int row = srow[r];
      const long k = k0 + kk;
      sa[kk][r] = (row >= 0 && k < K) ? (float)A[(long)(row / a_div) * K + k] : 0.f;
    }
    for (int e = tid; e < 64 * 16; e += 256) {
      const int c = e & 63, kk = e >> 6;
      const long k = k0 + kk, n = n0 + c;
      sb[kk][c] = (n < N && k < K) ? (float)We[k * N + n] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = sa[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = sb[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
  for (int i = 0; i < 4; ++i) {
    const int row = srow[ty * 4 + i];
    if (row < 0) continue;
    for (int j = 0; j < 4; ++j) {
      const long n = n0 + tx * 4 + j;
      if (n < N) C[(long)row * N + n] = (T16)acc[i][j];
    }
  }
}

// ------------------------------------------------------------------------------------------
extern "C" size_t hx_moe_workspace_bytes(int64_t T, int64_t E) {
  if (T < 0 || E < 0) return 0;
  // sized for the smaller row tile (64), which needs the longer table
  size_t b = moe_table_bytes(moe_max_tiles(T, E, 64));
  b = (b + 255) & ~(size_t)255;
  return b + (size_t)T + 256;
}

template <bool BF>
static int launch_moe(const void* A, const void* W, void* C, const int32_t* counts, const int32_t* offsets, const int32_t* idx,
                      int64_t T, int64_t K, int64_t N, int64_t E, int64_t a_div, void* ws, hipStream_t s) {
  typedef typename Mfma16<BF>::T T16;
  const bool fast = (K % MOE_BK == 0) && (N % 8 == 0) && K >= MOE_BK && (((T + a_div - 1) / a_div) * K * 2 < (1LL << 32)) && (N * 4 < (1LL << 31)) && (((uintptr_t)A | (uintptr_t)W | (uintptr_t)C) & 15) == 0;
  const int bm = fast ? MOE_BM : 64;
  const int max_tiles = (int)moe_max_tiles(T, E, bm);
  int* num_tiles = (int*)ws;
  MoeTile* table = (MoeTile*)((uint8_t*)ws + 16);
  size_t tb = moe_table_bytes(moe_max_tiles(T, E, 64));
  tb = (tb + 255) & ~(size_t)255;
  uint8_t* flags = (uint8_t*)ws + tb;

  const int prep_blocks = (int)((T + 256 * 64 - 1) / (256 * 64)) + 1;
  hipLaunchKernelGGL(hx_moe_prep, dim3(prep_blocks), dim3(256), 0, s, counts, offsets, (int)E, (int)T, bm, max_tiles, num_tiles, table,
                     flags);
  hipLaunchKernelGGL(hx_moe_mark, dim3(max_tiles < 1024 ? max_tiles : 1024), dim3(256), 0, s, (const int*)num_tiles,
                     (const MoeTile*)table, idx, (int)T, flags);
  if (fast) {
    const int tiles_n = (int)((N + MOE_BN - 1) / MOE_BN);
    hipLaunchKernelGGL(hx_moe_tile256<BF>, dim3(max_tiles * tiles_n), dim3(256), 0, s, (const uint8_t*)A, (const uint8_t*)W, (T16*)C,
                       (const int*)num_tiles, (const MoeTile*)table, idx, (int)T, (int)K, (int)N, max_tiles, tiles_n, (int)a_div);
  } else {
    dim3 grid((unsigned)max_tiles, (unsigned)((N + 63) / 64));
    hipLaunchKernelGGL(hx_moe_general<T16>, grid, dim3(256), 0, s, (const T16*)A, (const T16*)W, (T16*)C, (const int*)num_tiles,
                       (const MoeTile*)table, idx, (int)T, (int)K, (int)N, (int)a_div);
  }
  hipLaunchKernelGGL(hx_moe_zero_rows<T16>, dim3((unsigned)T), dim3(256), 0, s, (T16*)C, (long)N, (int)T, (int)N, (const uint8_t*)flags);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    hx_set_error("hx_moe_grouped_gemm: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

extern "C" int hx_moe_grouped_gemm(const void* A, const void* W, void* C, const int32_t* counts, const int32_t* offsets,
                                   const int32_t* idx, int64_t T, int64_t K, int64_t N, int64_t E, int64_t max_T, int dtype,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  if (T < 0 || K < 0 || N < 0 || E < 0 || max_T < 0) {
    hx_set_error("hx_moe_grouped_gemm: negative size");
    return HX_ERR_BAD_ARG;
  }
  if (dtype != HX_BF16 && dtype != HX_F16) {
    hx_set_error("hx_moe_grouped_gemm: dtype must be HX_BF16 or HX_F16, got %d", dtype);
    return HX_ERR_BAD_ARG;
  }
  if (T == 0 || N == 0) return 0;
  if (!A || !C || (E > 0 && (!W || !counts || !offsets)) || !idx) {
    hx_set_error("hx_moe_grouped_gemm: null pointer");
    return HX_ERR_BAD_ARG;
  }
  if (T >= (1LL << 31) || K >= (1LL << 31) || N >= (1LL << 31) || E >= (1LL << 24) || N > 65535LL * 64) {
    hx_set_error("hx_moe_grouped_gemm: dimension too large");
    return HX_ERR_UNSUPPORTED;
  }
  if (!workspace || workspace_bytes < hx_moe_workspace_bytes(T, E) || ((uintptr_t)workspace & 15)) {
    hx_set_error("hx_moe_grouped_gemm: workspace must be 16-byte aligned and at least %zu bytes (got %zu)",
                 hx_moe_workspace_bytes(T, E), workspace_bytes);
    return HX_ERR_WORKSPACE;
  }
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HX_BF16) return launch_moe<true>(A, W, C, counts, offsets, idx, T, K, N, E, 1, workspace, s);
  return launch_moe<false>(A, W, C, counts, offsets, idx, T, K, N, E, 1, workspace, s);
}

// ------------------------------------------------------------------------------------------
// top-k entry: routing on the device + grouped GEMM that gathers A rows as (sorted row / top_k)
// ------------------------------------------------------------------------------------------
extern "C" int hx_moe_routing(const void* expert_ids, int ids_are_int64, int64_t T, int64_t E, int32_t* counts, int32_t* offsets,
                              int32_t* idx, int32_t* max_count, void* workspace, size_t workspace_bytes, void* stream);
extern "C" size_t hx_moe_routing_workspace_bytes(int64_t T, int64_t E);

static inline size_t moe_topk_tables_bytes(int64_t T, int64_t E) {
  // counts[E] | offsets[E+1] | max_count | idx[T] | scratch of the routing kernels
  size_t b = (size_t)(2 * E + 2) * 4 + (size_t)T * 4 + hx_moe_routing_workspace_bytes(T, E);
  return (b + 255) & ~(size_t)255;
}

extern "C" size_t hx_moe_topk_workspace_bytes(int64_t T_tok, int64_t top_k, int64_t E) {
  if (T_tok < 0 || top_k < 1 || E < 0) return 0;
  const int64_t T = T_tok * top_k;
  return moe_topk_tables_bytes(T, E) + hx_moe_workspace_bytes(T, E);
}

extern "C" int hx_moe_topk_matmul(const void* A_tok, const void* W, void* C, const void* expert_ids, int ids_are_int64,
                                  int64_t T_tok, int64_t top_k, int64_t K, int64_t N, int64_t E, int dtype, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  if (T_tok < 0 || K < 0 || N < 0 || E < 0 || top_k < 1) {
    hx_set_error("hx_moe_topk_matmul: negative size or top_k < 1");
    return HX_ERR_BAD_ARG;
  }
  if (dtype != HX_BF16 && dtype != HX_F16) {
    hx_set_error("hx_moe_topk_matmul: dtype must be HX_BF16 or HX_F16, got %d", dtype);
    return HX_ERR_BAD_ARG;
  }
  if (T_tok >= (1LL << 31) / top_k) {
    hx_set_error("hx_moe_topk_matmul: dimension too large");
    return HX_ERR_UNSUPPORTED;
  }
  const int64_t T = T_tok * top_k;
  if (T == 0 || N == 0) return 0;
  if (!A_tok || !C || !expert_ids || (E > 0 && !W)) {
    hx_set_error("hx_moe_topk_matmul: null pointer");
    return HX_ERR_BAD_ARG;
  }
  if (T >= (1LL << 31) || K >= (1LL << 31) || N >= (1LL << 31) || E >= (1LL << 24) || N > 65535LL * 64) {
    hx_set_error("hx_moe_topk_matmul: dimension too large");
    return HX_ERR_UNSUPPORTED;
  }
  if (!workspace || workspace_bytes < hx_moe_topk_workspace_bytes(T_tok, top_k, E) || ((uintptr_t)workspace & 15)) {
    hx_set_error("hx_moe_topk_matmul: workspace must be 16-byte aligned and at least %zu bytes (got %zu)",
                 hx_moe_topk_workspace_bytes(T_tok, top_k, E), workspace_bytes);
    return HX_ERR_WORKSPACE;
  }
  int32_t* counts = (int32_t*)workspace;
  int32_t* offsets = counts + E;
  int32_t* max_count = offsets + E + 1;
  int32_t* idx = max_count + 1;
  void* ws2 = (uint8_t*)workspace + moe_topk_tables_bytes(T, E);
  int rc = hx_moe_routing(expert_ids, ids_are_int64, T, E, counts, offsets, idx, max_count, idx + T, hx_moe_routing_workspace_bytes(T, E),
                          stream);
  if (rc != 0) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HX_BF16) return launch_moe<true>(A_tok, W, C, counts, offsets, idx, T, K, N, E, top_k, ws2, s);
  return launch_moe<false>(A_tok, W, C, counts, offsets, idx, T, K, N, E, top_k, ws2, s);
}
