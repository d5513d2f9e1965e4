// MoE grouped GEMM for gfx950 — device side of examples/moe_matmul_ogs.py:25-80 of the reference
// (semantics: moe_matmul_ogs_reference, :125-148):
//   for expert e, i < counts[e]:  r = idx[offsets[e] + i];   C[r, :] = cast(A[r, :] @ W[e])
//   rows of C that no expert covers are zero.
// A [T,K], W [E,K,N] (N contiguous), C [T,N]; bf16 or fp16; fp32 accumulation.
//
// Launch sequence (all on the caller's stream, no host synchronisation):
//   1. hx_moe_prep       : builds the tile table (tile -> expert, first sorted row, row count) from
//                          counts/offsets on the device and clears the row-covered flags;
//   2. hx_moe_mark       : flags every row some expert covers (1 and 2 are one launch, hx_moe_prep_mark_small, for
//                          small problems);
//   3. hx_gemm16_tile256 / _tile128 / _rows32 or hx_moe_general : the grouped GEMM over (row tile, column tile) pairs;
//   4. hx_moe_zero_rows  : zero-fills rows whose flag is still clear.
// Padded rows of a tile are never stored, so there is no read-modify-write and no write race.
#include <mutex>

#include "gemm16_tile128.h"
#include "gemm16_rows32.h"
#include "gemm16_tile256p.h"

// workspace layout: [0] int num_tiles | [16 ..) MoeTile table[max_tiles] | flags[T] bytes
static inline size_t moe_table_bytes(int64_t max_tiles) { return 16 + (size_t)max_tiles * sizeof(MoeTile); }
static inline int64_t moe_max_tiles(int64_t T, int64_t E, int bm) { return (T + bm - 1) / bm + E; }

__global__ void hx_moe_prep(const int32_t* __restrict__ counts, const int32_t* __restrict__ offsets, int E, int T, int bm,
                            int max_tiles, int* __restrict__ num_tiles, MoeTile* __restrict__ table, uint8_t* __restrict__ flags) {
  const int tid = blockIdx.x * blockDim.x + threadIdx.x, nth = gridDim.x * blockDim.x;
  for (int i = tid; i < T; i += nth) flags[i] = 0;
  if (blockIdx.x != 0) return;
  // block 0 builds the tile table, 256 experts at a time: tile counts, an exclusive scan of them in LDS, then every
  // thread fills tiles of the chunk, finding a tile's expert by binary search in the scanned counts
  __shared__ int s_first[257];  // tiles of the chunk before its expert i; s_first[256] = tiles of the chunk
  __shared__ int s_start[256], s_cnt[256];
  __shared__ int s_base;        // tiles before the chunk
  const int t256 = threadIdx.x;
  if (t256 == 0) s_base = 0;
  for (int e0 = 0; e0 < E; e0 += 256) {
    const int e = e0 + t256;
    int c = 0, start = 0;
    if (e < E) {
      c = counts[e];
      c = c < 0 ? 0 : c;
      start = offsets[e];
      // clamp malformed tables so the GEMM never indexes outside idx[0..T)
      if (start < 0 || start > T) c = 0;
      if (c > T - start) c = T - start;
    }
    s_start[t256] = start;
    s_cnt[t256] = c;
    if (t256 == 0) s_first[0] = 0;
    s_first[t256 + 1] = (c + bm - 1) / bm;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {  // inclusive scan (Hillis-Steele), shifted by one
      const int v = t256 >= d ? s_first[t256 + 1 - d] : 0;
      __syncthreads();
      s_first[t256 + 1] += v;
      __syncthreads();
    }
    const int base = s_base, chunk_tiles = s_first[256];
    for (int i = t256; i < chunk_tiles && base + i < max_tiles; i += 256) {
      int lo = 0, hi = 256;  // invariant: s_first[lo] <= i < s_first[hi]
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_first[mid] <= i) lo = mid; else hi = mid;
      }
      const int j = i - s_first[lo];
      MoeTile mt;
      mt.expert = e0 + lo;
      mt.row_start = s_start[lo] + j * bm;
      mt.rows = min(bm, s_cnt[lo] - j * bm);
      mt.pad = 0;
      table[base + i] = mt;
    }
    __syncthreads();  // everybody has read s_base and the chunk's arrays
    if (t256 == 0) s_base = base + chunk_tiles;
    __syncthreads();
  }
  if (t256 == 0) *num_tiles = min(s_base, max_tiles);
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

// one workgroup per 256 rows: uncovered rows are rare, so most workgroups read 256 flags and leave
template <typename T16>
__global__ __launch_bounds__(256) void hx_moe_zero_rows(T16* __restrict__ C, long ldc, int T, int N, const uint8_t* __restrict__ flags) {
  __shared__ uint8_t s_flag[256];
  const int row0 = blockIdx.x * 256, tid = threadIdx.x;
  const bool uncovered = row0 + tid < T && !flags[row0 + tid];
  s_flag[tid] = uncovered;
  if (!__syncthreads_or(uncovered)) return;
  for (int r = 0; r < 256; ++r) {
    if (!s_flag[r]) continue;  // workgroup-uniform
    T16* c = C + (long)(row0 + r) * ldc;
    for (int n = tid; n < N; n += 256) c[n] = (T16)0.f;
  }
}

// Small problems (a decode step, a few thousand rows): one workgroup does what hx_moe_prep and hx_moe_mark do, so the
// grouped GEMM is preceded by one short launch instead of two.  E <= 1024, T <= 4096.
__global__ __launch_bounds__(1024) void hx_moe_prep_mark_small(const int32_t* __restrict__ counts, const int32_t* __restrict__ offsets,
                                                               const int32_t* __restrict__ idx, int E, int T, int bm, int max_tiles,
                                                               int* __restrict__ num_tiles, MoeTile* __restrict__ table,
                                                               uint8_t* __restrict__ flags) {
  __shared__ int s_first[1025];  // tiles before expert e (exclusive prefix), s_first[E] = total
  __shared__ int s_start[1024], s_cnt[1024];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < T; i += 1024) flags[i] = 0;
  int nt = 0;
  if (tid < E) {
    int c = counts[tid];
    c = c < 0 ? 0 : c;
    const int start = offsets[tid];
    // clamp malformed tables so the GEMM never indexes outside idx[0..T)
    if (start < 0 || start > T) c = 0;
    if (c > T - start) c = T - start;
    s_start[tid] = start;
    s_cnt[tid] = c;
    nt = (c + bm - 1) / bm;
  }
  // inclusive scan of the tile counts over the 1024 threads (Hillis-Steele in LDS), shifted into s_first[1..]
  if (tid == 0) s_first[0] = 0;
  s_first[tid + 1] = nt;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int v = tid >= d ? s_first[tid + 1 - d] : 0;
    __syncthreads();
    s_first[tid + 1] += v;
    __syncthreads();
  }
  const int total = min(s_first[E], max_tiles);
  if (tid == 0) *num_tiles = total;
  // tile t belongs to the expert e with s_first[e] <= t < s_first[e+1]
  auto tile_of = [&](int t, int& e, int& rs, int& rows) {
    int lo = 0, hi = E;  // invariant: s_first[lo] <= t < s_first[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_first[mid] <= t) lo = mid; else hi = mid;
    }
    e = lo;
    const int i = t - s_first[lo];
    rs = s_start[lo] + i * bm;
    rows = min(bm, s_cnt[lo] - i * bm);
  };
  for (int t = tid; t < total; t += 1024) {
    int e, rs, rows;
    tile_of(t, e, rs, rows);
    table[t].expert = e;
    table[t].row_start = rs;
    table[t].rows = rows;
    table[t].pad = 0;
  }
  __syncthreads();  // (includes the wait for the flag stores above: they are cleared before any is set)
  for (int t = wave; t < total; t += 16) {
    int e, rs, rows;
    tile_of(t, e, rs, rows);
    for (int i = lane; i < rows; i += 64) {
      const int r = idx[rs + i];
      if (r >= 0 && r < T) flags[r] = 1;
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
  // sized for the smallest row tile (32), which needs the longest table
  size_t b = moe_table_bytes(moe_max_tiles(T, E, 32));
  b = (b + 255) & ~(size_t)255;
  // (with the persistent kernel switched on: room behind the flags for its store sink, 16-byte aligned)
  return b + (size_t)T + 256 + (hx_feature(HX_FEATURE_MOE_PERSISTENT) ? G16P_SINK_BYTES + 16 : 0);
}

// Which kernel multiplies a grouped GEMM: 0 = hx_moe_general (fp32 FMAs; rows that are not 16-byte aligned, K % 8 != 0 or
// N % 8 != 0), 1 = 32-row tiles, 2 = 128-row tiles, 3 = 256-row tiles, 4 = 128-row tiles with a partial last k-tile
// (K % 64 != 0), 5 = the same with A fetched in 4-byte pieces (K even but not a multiple of 8: 4-byte aligned rows, e.g.
// the K = 500 of the reference's own check); 1-5 are MFMA kernels.  6 (opt-in, HX_FEATURE_MOE_PERSISTENT): the 256-row
// tiles in persistent workgroups, where 3 would run and N % 256 == 0, K % 128 == 0, K >= 256.
static int moe_path(const void* A, const void* W, const void* C, int64_t T, int64_t K, int64_t N, int64_t E, int64_t a_div) {
  const bool fast = (K % 2 == 0) && (N % 8 == 0) && K >= 2 && (((T + a_div - 1) / a_div) * K * 2 < (1LL << 32)) && (N * 4 < (1LL << 31)) &&
                    (((uintptr_t)A | (uintptr_t)W | (uintptr_t)C) & 15) == 0;
  if (!fast) return 0;
  if (K % 8 != 0) return 5;
  if (K % MOE_BK != 0) return 4;
  // 128-row tiles while the experts are small (less padding in each expert's last row tile) or the 256-row tiles would
  // not fill the chip; 256-row tiles otherwise (half the operand traffic per flop)
  const int64_t tn256 = (N + MOE_BN - 1) / MOE_BN;
  const bool small = E > 0 && (T / E < 512 || ((T + MOE_BM - 1) / MOE_BM + E / 2) * tn256 < 192);
  // a handful of rows in all: 32-row tiles (a quarter of the A bytes per stage, more weight bytes in flight per CU)
  if (T <= R32_BM) return 1;
  if (small) return 2;
  if (hx_feature(HX_FEATURE_MOE_PERSISTENT) && N % MOE_BN == 0 && K % (2 * MOE_BK) == 0 && K >= 4 * MOE_BK && hx_cu_count() >= 8) return 6;
  return 3;
}

extern "C" int hx_moe_path(int64_t T, int64_t K, int64_t N, int64_t E, int64_t a_div, const void* A, const void* W, const void* C) {
  if (T < 0 || K < 0 || N < 0 || E < 0 || a_div < 1) return -1;
  return moe_path(A, W, C, T, K, N, E, a_div);
}

template <bool BF>
static int launch_moe(const void* A, const void* W, void* C, const int32_t* counts, const int32_t* offsets, const int32_t* idx,
                      int64_t T, int64_t K, int64_t N, int64_t E, int64_t a_div, void* ws, hipStream_t s) {
  typedef typename Mfma16<BF>::T T16;
  const int path = moe_path(A, W, C, T, K, N, E, a_div);
  const bool fast = path != 0;
  const int bm = path == 1 ? R32_BM : (path == 3 || path == 6) ? MOE_BM : path == 0 ? 64 : G128_BM;
  const int max_tiles = (int)moe_max_tiles(T, E, bm);
  int* num_tiles = (int*)ws;
  MoeTile* table = (MoeTile*)((uint8_t*)ws + 16);
  size_t tb = moe_table_bytes(moe_max_tiles(T, E, 32));
  tb = (tb + 255) & ~(size_t)255;
  uint8_t* flags = (uint8_t*)ws + tb;

  if (E <= 1024 && T <= 4096) {
    hx_launch(hx_moe_prep_mark_small, dim3(1), dim3(1024), 0, s, counts, offsets, idx, (int)E, (int)T, bm, max_tiles, num_tiles,
                       table, flags);
  } else {
    const int prep_blocks = (int)((T + 256 * 64 - 1) / (256 * 64)) + 1;
    hx_launch(hx_moe_prep, dim3(prep_blocks), dim3(256), 0, s, counts, offsets, (int)E, (int)T, bm, max_tiles, num_tiles, table,
                       flags);
    hx_launch(hx_moe_mark, dim3(max_tiles < 1024 ? max_tiles : 1024), dim3(256), 0, s, (const int*)num_tiles,
                       (const MoeTile*)table, idx, (int)T, flags);
  }
  if (fast) {
    G16Dense d = {};
    d.lda = K; d.ldb = N; d.ldc = N;
    if (path == 6) {
      const int tiles_n = (int)(N / MOE_BN), grid = (hx_cu_count() / 8) * 8;
      uint8_t* sink = (uint8_t*)(((uintptr_t)flags + (size_t)T + 15) & ~(uintptr_t)15);  // behind the flags (hx_moe_workspace_bytes)
      hx_launch((hx_gemm16_tile256p<BF, false>), dim3(grid), dim3(256), 0, s, (const uint8_t*)A, (const uint8_t*)W, (void*)C,
                (const int*)num_tiles, (const MoeTile*)table, idx, (int)T, (int)K, (int)N, tiles_n, (int)a_div, sink, (long)K, (long)N,
                (long)N, 0);
    } else if (bm == R32_BM) {
      const int tiles_n = (int)((N + R32_BN - 1) / R32_BN);
      hx_launch((hx_gemm16_rows32<BF, 3>), dim3(max_tiles * tiles_n), dim3(256), 0, s, (const uint8_t*)A, (const uint8_t*)W,
                         (void*)C, (const int*)num_tiles, (const MoeTile*)table, idx, (int)T, (int)K, (int)N, max_tiles, tiles_n,
                         (int)a_div, d);
    } else if (path == 5) {
      const int tiles_n = (int)((N + G128_BN - 1) / G128_BN);
      hx_launch((hx_gemm16_tile128<BF, 0, false, 2, true, true>), dim3(max_tiles * tiles_n), dim3(256), 0, s, (const uint8_t*)A,
                (const uint8_t*)W, (void*)C, (const int*)num_tiles, (const MoeTile*)table, idx, (int)T, (int)K, (int)N, max_tiles,
                tiles_n, (int)a_div, d);
    } else if (path == 4) {
      const int tiles_n = (int)((N + G128_BN - 1) / G128_BN);
      hx_launch((hx_gemm16_tile128<BF, 0, false, 2, true>), dim3(max_tiles * tiles_n), dim3(256), 0, s, (const uint8_t*)A,
                (const uint8_t*)W, (void*)C, (const int*)num_tiles, (const MoeTile*)table, idx, (int)T, (int)K, (int)N, max_tiles,
                tiles_n, (int)a_div, d);
    } else if (bm == MOE_BM) {
      const int tiles_n = (int)((N + MOE_BN - 1) / MOE_BN);
      hx_launch((hx_gemm16_tile256<BF, 0>), dim3(max_tiles * tiles_n), dim3(256), 0, s, (const uint8_t*)A, (const uint8_t*)W,
                         (void*)C, (const int*)num_tiles, (const MoeTile*)table, idx, (int)T, (int)K, (int)N, max_tiles, tiles_n,
                         (int)a_div, d);
    } else {
      const int tiles_n = (int)((N + G128_BN - 1) / G128_BN);
      hx_launch((hx_gemm16_tile128<BF, 0>), dim3(max_tiles * tiles_n), dim3(256), 0, s, (const uint8_t*)A, (const uint8_t*)W,
                         (void*)C, (const int*)num_tiles, (const MoeTile*)table, idx, (int)T, (int)K, (int)N, max_tiles, tiles_n,
                         (int)a_div, d);
    }
  } else {
    dim3 grid((unsigned)max_tiles, (unsigned)((N + 63) / 64));
    hx_launch(hx_moe_general<T16>, grid, dim3(256), 0, s, (const T16*)A, (const T16*)W, (T16*)C, (const int*)num_tiles,
                       (const MoeTile*)table, idx, (int)T, (int)K, (int)N, (int)a_div);
  }
  hx_launch(hx_moe_zero_rows<T16>, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, s, (T16*)C, (long)N, (int)T, (int)N,
                     (const uint8_t*)flags);
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_moe_grouped_gemm: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

// ------------------------------------------------------------------------------------------
// Any K, any N through the MFMA kernels (opt-in, HX_FEATURE_MOE_ANY_SHAPE): an odd K leaves the rows of A only 2-byte
// aligned and N % 8 != 0 those of W and C, which no DMA instruction can fetch - such calls ran the fp32-FMA kernel.  With
// room in the workspace the operands are copied once into 16-byte-friendly form, zero-padded (zeros add nothing to a dot
// product): A as [rows][K8], W as [E][K8][N8] with K8 / N8 the next multiples of 8, and, when N itself is padded, C as
// [T][N8] with a crop back afterwards.  Cost: one read and write of A and W (and C) against 2 T K N flops.
// ------------------------------------------------------------------------------------------
// dst[b][r][c] = src[b][r][c] inside rows x cols, 0 in the padding; 16-bit elements; one work-item per 8 elements of dst
__global__ __launch_bounds__(256) void hx_pad2d_u16(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int rows, int cols,
                                                   int drows, int dcols, long n_chunks) {
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= n_chunks) return;
  const int cpr = dcols / 8;
  const long br = id / cpr;  // batch * drows + row
  const int c0 = (int)(id % cpr) * 8, r = (int)(br % drows);
  const long b = br / drows;
  uint16_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (r < rows && c0 + i < cols) ? src[(b * rows + r) * (long)cols + c0 + i] : (uint16_t)0;
  *(v4i*)(dst + (br * dcols + c0)) = *(const v4i*)v;
}
// dst[r][c] = src[r][c] for c < cols; src rows are scols apart
__global__ __launch_bounds__(256) void hx_crop2d_u16(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, long rows, int cols, int scols) {
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= rows * cols) return;
  dst[id] = src[(id / cols) * scols + id % cols];
}

static bool moe_repack_wanted(int64_t K, int64_t N) { return hx_feature(HX_FEATURE_MOE_ANY_SHAPE) && K >= 1 && N >= 1 && (K % 2 != 0 || N % 8 != 0); }
static inline size_t up256(size_t b) { return (b + 255) & ~(size_t)255; }
struct MoeRepack {
  int64_t K8, N8, rows_a;
  size_t a_off, w_off, c_off, total;  // byte offsets in the workspace behind the plain layout; c_off == 0: C is written in place
};
static MoeRepack moe_repack_plan(int64_t T, int64_t K, int64_t N, int64_t E, int64_t a_div) {
  MoeRepack r;
  r.K8 = (K + 7) & ~(int64_t)7, r.N8 = (N + 7) & ~(int64_t)7, r.rows_a = (T + a_div - 1) / a_div;
  r.a_off = up256(hx_moe_workspace_bytes(T, E));
  r.w_off = r.a_off + up256((size_t)r.rows_a * r.K8 * 2);
  const size_t end_w = r.w_off + up256((size_t)E * r.K8 * r.N8 * 2);
  r.c_off = N % 8 != 0 ? end_w : 0;
  r.total = N % 8 != 0 ? end_w + up256((size_t)T * r.N8 * 2) : end_w;
  return r;
}

extern "C" size_t hx_moe_workspace_bytes_shape(int64_t T, int64_t K, int64_t N, int64_t E) {
  if (T < 0 || K < 0 || N < 0 || E < 0) return 0;
  if (!moe_repack_wanted(K, N) || T == 0) return hx_moe_workspace_bytes(T, E);
  return moe_repack_plan(T, K, N, E, 1).total;
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
  if (moe_repack_wanted(K, N) && E > 0) {
    const MoeRepack rp = moe_repack_plan(T, K, N, E, 1);
    if (workspace_bytes >= rp.total && (size_t)rp.rows_a * rp.K8 * 2 < (1ULL << 32)) {
      uint8_t* base = (uint8_t*)workspace;
      uint16_t* a2 = (uint16_t*)(base + rp.a_off);
      uint16_t* w2 = (uint16_t*)(base + rp.w_off);
      uint16_t* c2 = rp.c_off ? (uint16_t*)(base + rp.c_off) : (uint16_t*)C;
      const long ca = (long)rp.rows_a * (rp.K8 / 8), cw = (long)E * rp.K8 * (rp.N8 / 8);
      hx_launch(hx_pad2d_u16, dim3((unsigned)((ca + 255) / 256)), dim3(256), 0, s, (const uint16_t*)A, a2, (int)rp.rows_a, (int)K, (int)rp.rows_a,
                (int)rp.K8, ca);
      hx_launch(hx_pad2d_u16, dim3((unsigned)((cw + 255) / 256)), dim3(256), 0, s, (const uint16_t*)W, w2, (int)K, (int)N, (int)rp.K8, (int)rp.N8, cw);
      const int rc = dtype == HX_BF16 ? launch_moe<true>(a2, w2, c2, counts, offsets, idx, T, rp.K8, rp.N8, E, 1, workspace, s)
                                      : launch_moe<false>(a2, w2, c2, counts, offsets, idx, T, rp.K8, rp.N8, E, 1, workspace, s);
      if (rc != 0 || !rp.c_off) return rc;
      const long n = (long)T * N;
      hx_launch(hx_crop2d_u16, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const uint16_t*)c2, (uint16_t*)C, (long)T, (int)N, (int)rp.N8);
      const hipError_t e = hx_launch_status();
      if (e != hipSuccess) {
        hx_set_error("hx_moe_grouped_gemm: launch failed: %s", hipGetErrorString(e));
        return (int)e;
      }
      return 0;
    }
  }
  if (dtype == HX_BF16) return launch_moe<true>(A, W, C, counts, offsets, idx, T, K, N, E, 1, workspace, s);
  return launch_moe<false>(A, W, C, counts, offsets, idx, T, K, N, E, 1, workspace, s);
}

// ------------------------------------------------------------------------------------------
// hx_moe_grouped_gemm for callers that cannot allocate: the tile table and the row flags live in a file-scope
// device array instead of a caller-provided workspace.  Every GPU holds its own copy of the array at its own
// address; the address is looked up once per device (with that device current) and only that pointer is ever
// handed to kernels -- the array's name is a host-side stand-in, not a device address.
// ------------------------------------------------------------------------------------------
#define HX_MOE_STATIC_SCRATCH_BYTES (256 * 1024)
static __device__ __align__(256) uint8_t scratch[HX_MOE_STATIC_SCRATCH_BYTES];

static std::mutex g_scratch_mu;
static void* g_scratch_ptr[64];  // per device ordinal; nullptr = not looked up yet

// Device address of this GPU's copy of `scratch` (cached after the first call on the device); nullptr + error set
// on failure.
static void* moe_static_scratch() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= 64) {
    hx_set_error("hx_moe_grouped_gemm_static: hipGetDevice failed or device ordinal %d out of range: %s", dev, hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      hx_set_error("hx_moe_grouped_gemm_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

extern "C" int hx_moe_grouped_gemm_static(const void* A, const void* W, void* C, const int32_t* counts, const int32_t* offsets,
                                          const int32_t* idx, int64_t T, int64_t K, int64_t N, int64_t E, int64_t max_T, int dtype,
                                          void* stream) {
  if (T < 0 || K < 0 || N < 0 || E < 0 || max_T < 0) {
    hx_set_error("hx_moe_grouped_gemm_static: negative size");
    return HX_ERR_BAD_ARG;
  }
  if (T > HX_MOE_STATIC_MAX_ROWS || E > HX_MOE_STATIC_MAX_EXPERTS || hx_moe_workspace_bytes(T, E) > HX_MOE_STATIC_SCRATCH_BYTES) {
    hx_set_error("hx_moe_grouped_gemm_static: T = %lld rows / E = %lld experts exceed the built-in scratch (at most %d rows and %d "
                 "experts); use hx_moe_grouped_gemm with a workspace", (long long)T, (long long)E, HX_MOE_STATIC_MAX_ROWS,
                 HX_MOE_STATIC_MAX_EXPERTS);
    return HX_ERR_UNSUPPORTED;
  }
  if (T == 0 || N == 0) return 0;
  void* ptr = moe_static_scratch();
  if (!ptr) return HX_ERR_WORKSPACE;
  // same checks, same kernels: the workspace is this device's copy of the static array
  return hx_moe_grouped_gemm(A, W, C, counts, offsets, idx, T, K, N, E, max_T, dtype, ptr, HX_MOE_STATIC_SCRATCH_BYTES, stream);
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
