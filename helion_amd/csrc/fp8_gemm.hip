// FP8 (OCP e4m3fn) GEMM for gfx950: C[M,N] = cast((A[M,K] @ B[K,N]) * scale_a*scale_b), fp32 accumulate.
// Drop-in device side of examples/fp8_gemm.py:29-57 of the reference.
//
// The kernels:
//   hx_fp8_gemm_tile256 : 256x256x128 workgroup tile, 4 waves (2x2) of 128x128, 16x16x128 fp8 MFMA,
//                         A/B k-tiles DMA'd global->LDS (double buffered, XOR-swizzled 16B chunks).
//   hx_fp8_gemm_tileN128 : 64/128/256 x 128 tiles with a deeper LDS ring, for problems with too few 256x256 tiles
//                         (decode batches, mid-size products), with split-K (+ hx_fp8_gemm_split_reduce) when even
//                         those tiles are few and K is long.
//   hx_fp8_gemm_skinny_direct : M <= 32, K <= 8192; HBM-bound streaming of B^T through registers into
//                         16x16x128 MFMA, K split across the 8 waves of a workgroup, partials summed in LDS.
//   hx_fp8_gemm_skinny  : M <= 16, larger K; same split, A panel staged through LDS in 8 KB chunks of K.
//   hx_fp8_gemm_general : bounds-checked, arbitrary strides (fallback for ragged/unaligned inputs).
#include "hx_common.h"

#include <atomic>
#include <chrono>
#include <type_traits>

// ------------------------------------------------------------------------------------------
// tile256
// ------------------------------------------------------------------------------------------
// LDS tile layout (A and B alike; B is addressed as B^T[N][K], K contiguous):
//   tile[row 0..255][pos 0..7] of 16-byte chunks, row stride 128 B (one 128-byte k-tile per row);
//   the chunk stored at (row, pos) is global chunk  pos ^ swz(row),  swz(row) = (row >> 1) & 7.
// One DMA instruction of a wave moves 8 rows x 128 B (lane = row_in_8 * 8 + pos), so global reads
// are whole 128-byte lines and LDS writes are 1024 contiguous bytes.
// MFMA operand fetch (16x16x128, one instruction spans the whole 128-byte k-tile): lane (r = lane%16, g = lane/16)
// reads chunks 2g and 2g+1 of row r: two ds_read_b128.  A and B use the same lane->k mapping, which is all the
// contraction needs.  (Against the 32x32x64 shape this halves the accumulator traffic per flop: +3 % measured.)

#define T256_BM 256
#define T256_BN 256
#define T256_BK 128
#define T256_TILE_BYTES (256 * 128)

// EDGE: M and/or N are not multiples of 256.  Rows past the end are clamped to the last row on load (their
// products land in accumulators that are never stored) and the stores are guarded.
// BROW: B is row-major ([K][N], N contiguous; `Bt`/`ldb` are then B itself and its row stride).  The B tile sits in
// LDS as [128 k][256 B of n], chunk stored at pos = chunk ^ (((k&7)<<1) | ((k>>5)&1)), and the MFMA operand (32
// consecutive k of one column per lane) is formed by four transposing reads (ds_read_b64_tr_b8: 8 k x 16 n per 16
// lanes) instead of two 16-byte reads; one DMA instruction moves 4 k-rows x 256 B.  N must be a multiple of 16; with EDGE, chunks past
// the end re-read the row's last valid chunk.
template <int OUT, bool EDGE, bool BROW>
__global__ __launch_bounds__(256) void hx_fp8_gemm_tile256(const uint8_t* __restrict__ A, const uint8_t* __restrict__ Bt,
                                                          typename OutT<OUT>::T* __restrict__ C, int M, int N, int K, long lda,
                                                          long ldb, long ldc, const float* __restrict__ scale_a,
                                                          const float* __restrict__ scale_b, int tiles_m, int tiles_n) {
  typedef typename OutT<OUT>::T out_t;
  // [stage][A|B][256 rows x 128 B]
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2][2][T256_TILE_BYTES];

  // ---- workgroup -> tile. Workgroup i runs on XCD i%8 (each XCD has its own 4 MB L2): give every
  // XCD a contiguous range of a grouped (8 tile-rows tall) raster so concurrently resident tiles of
  // one XCD share A row-panels and B column-panels in that L2.
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
  const int gm = min(tiles_m - first_m, GM);
  const int tm = first_m + (tile % group_size) % gm;
  const int tn = (tile % group_size) / gm;
  const long m0 = (long)tm * T256_BM, n0 = (long)tn * T256_BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;

  // ---- DMA addressing: wave w owns tile rows [64w, 64w+64); instruction j covers rows 64w+8j .. +7.
  // address = uniform base (row block, k-tile) + per-lane offset (row in block, swizzled chunk)
  const int lrow = lane >> 3, lpos = lane & 7;
  const uint32_t a_vo0 = (uint32_t)(lrow * lda + (lpos ^ ((lrow >> 1) & 7)) * 16);        // j even
  const uint32_t a_vo1 = (uint32_t)(lrow * lda + (lpos ^ ((4 + (lrow >> 1)) & 7)) * 16);  // j odd
  // row-major B: wave w owns k rows [32w, 32w+32) of the k-tile; instruction j covers rows 32w+4j .. +3, 16 chunks each
  const int brow = lane >> 4, bpos = lane & 15;
  const int bcmax = BROW ? (int)((min((long)N - n0, (long)T256_BN) >> 4) - 1) : 0;  // last valid chunk of this tile's rows
  auto brow_vo = [&](int kodd) {  // kodd: (row within the 8-row swizzle period) >= 4, i.e. j odd
    int chunk = bpos ^ ((((4 * kodd + brow) & 7) << 1) | (w & 1));  // k = 32w + 4j + brow: (k>>5)&1 = w&1
    if (EDGE) chunk = min(chunk, bcmax);
    return (uint32_t)(brow * ldb + chunk * 16);
  };
  const uint32_t b_vo0 = BROW ? brow_vo(0) : (uint32_t)(lrow * ldb + (lpos ^ ((lrow >> 1) & 7)) * 16);
  const uint32_t b_vo1 = BROW ? brow_vo(1) : (uint32_t)(lrow * ldb + (lpos ^ ((4 + (lrow >> 1)) & 7)) * 16);
  const uint8_t* gA = A + (m0 + w * 64) * lda;                                  // wave-uniform
  const uint8_t* gB = BROW ? Bt + (long)(w * 32) * ldb + n0 : Bt + (n0 + w * 64) * ldb;  // wave-uniform
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]) + (uint32_t)w * 64 * 128;
  const uint8_t* gB0 = Bt + n0;  // row-major B, edge tiles: per-lane k rows

  // k-tiles; with EDGE the last one may be partial (K % 16 == 0): its DMA re-reads valid chunks / rows instead of
  // running off the operands, and the part past K is zeroed in LDS once it has landed (zero_tail below)
  const int nk = EDGE ? (K + T256_BK - 1) / T256_BK : K / T256_BK;
  const int ktail = K - (nk - 1) * T256_BK;  // valid k of the last tile: 128 unless EDGE
  // DMA instruction i (0..15) of a k-tile: i < 8 -> A rows 64w + 8i .., else B rows 64w + 8(i-8) ..
  auto issue_one = [&](int kt, int stage, int i) {
    const long kb = (long)kt * T256_BK;
    const uint32_t la = lds0 + (uint32_t)stage * 2 * T256_TILE_BYTES, lb = la + T256_TILE_BYTES;
    if (BROW && i >= 8) {  // 4 k-rows x 256 B; column clamping (EDGE) is already in the per-lane offsets
      if (EDGE) {  // k rows past K re-read row K-1; the whole of B is below 4 GB (checked by the host)
        const uint32_t krow = (uint32_t)min((int)kb + w * 32 + (i - 8) * 4 + brow, K - 1);
        hx_g2l16_s(hx_uniform_ptr(gB0), krow * (uint32_t)ldb + (((i & 1) ? b_vo1 : b_vo0) - (uint32_t)(brow * ldb)), lb + (i - 8) * 1024);
      } else {
        hx_g2l16_s(gB + (kb + (long)(i - 8) * 4) * ldb, (i & 1) ? b_vo1 : b_vo0, lb + (i - 8) * 1024);
      }
    } else if (!EDGE) {
      if (i < 8) hx_g2l16_s(gA + (long)i * 8 * lda + kb, (i & 1) ? a_vo1 : a_vo0, la + i * 1024);
      else hx_g2l16_s(gB + (long)(i - 8) * 8 * ldb + kb, (i & 1) ? b_vo1 : b_vo0, lb + (i - 8) * 1024);
    } else {  // per-lane clamped row; the whole matrix is below 4 GB (checked by the host), so the offset fits 32 bits
      const int swz = (((i & 1) ? 4 : 0) + (lrow >> 1)) & 7;
      const int chunk = min(lpos ^ swz, (kt == nk - 1 ? ktail / 16 : 8) - 1);  // chunks past K re-read the last valid one
      if (i < 8) {
        const uint32_t row = (uint32_t)min((int)m0 + w * 64 + i * 8 + lrow, M - 1);
        hx_g2l16_s(hx_uniform_ptr(A + kb), row * (uint32_t)lda + (uint32_t)(chunk * 16), la + i * 1024);
      } else {
        const uint32_t row = (uint32_t)min((int)n0 + w * 64 + (i - 8) * 8 + lrow, N - 1);
        hx_g2l16_s(hx_uniform_ptr(Bt + kb), row * (uint32_t)ldb + (uint32_t)(chunk * 16), lb + (i - 8) * 1024);
      }
    }
  };
  auto issue = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < 16; ++i) issue_one(kt, stage, i);
  };

  // ---- MFMA operand addressing (16x16x128: lane = row/column lane%16, k-slots 32*(lane/16) .. +31)
  // The product does not care which 32 of the 128 k a lane group multiplies as long as A and B agree, and the LDS
  // serves a 16-byte read in four passes of the lanes {0-3, 12-15, 20-23, 24-27}, the same + 32, {4-7, 8-11, 16-19,
  // 28-31}, the same + 32.  With lane group gq on k-block gq, rows 0-3 of group 0 and rows 4-7 of group 1 meet in one
  // pass on the same banks (measured: every fragment read took twice its cycles); with k-blocks 0, 3, 1, 2 for groups
  // 0..3 the sixteen lanes of every pass land in sixteen different 16-byte bank groups.
  const int r16 = lane & 15, gq = lane >> 4;
  const int kq = (gq >> 1) ^ ((gq & 1) * 3);             // k-block (32 k) of this lane group
  const int x16 = ((2 * kq) ^ ((r16 >> 1) & 7)) * 16;  // chunk 2kq of the row, swizzled; chunk 2kq+1 is at x16 ^ 16
  const int a_base = (wm * 128 + r16) * 128;
  const int b_base = (wn * 128 + r16) * 128;
  // row-major B: transposing read j (0..3) of column block bj fetches k = 32kq + 8j .. +7; this lane supplies 8 bytes of
  // row (that k) + (lane%16)/2, columns 8*(lane&1) .. +7 of the block's 16-byte chunk, and receives column lane%16.
  // The chunk index wn*8 + bj enters by xor, which commutes with the swizzle's xor.
  const int bt_off = (32 * kq + (r16 >> 1)) * 256 + ((((r16 >> 1) << 1) | (kq & 1)) * 16) + (lane & 1) * 8;

  // acc[bj][bi][r] is C[m0 + wm*128 + 16 bi + lane%16][n0 + wn*128 + 16 bj + 4*(lane/16) + r]
  v4f acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  auto load_a = [&](v8i& f, int stage, int bi) {
    const uint8_t* base = &smem[stage][0][0] + a_base + bi * 2048;
    v4i lo = *(const v4i*)(base + x16);
    v4i hi = *(const v4i*)(base + (x16 ^ 16));
    f = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  auto load_b = [&](v8i& f, int stage, int bj) {
    if (BROW) {
      const uint8_t* sb = &smem[stage][1][0] + (bt_off ^ ((wn * 8 + bj) * 16));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const v2i part = __builtin_amdgcn_ds_read_tr8_b64_v2i32((v2i __attribute__((address_space(3)))*)(sb + j * 2048));
        f[2 * j] = part[0];
        f[2 * j + 1] = part[1];
      }
    } else {
      const uint8_t* base = &smem[stage][1][0] + b_base + bj * 2048;
      v4i lo = *(const v4i*)(base + x16);
      v4i hi = *(const v4i*)(base + (x16 ^ 16));
      f = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  };
  // One k-tile = 64 MFMAs in two halves, row-block-major: half h multiplies the 8 A fragments with B fragments
  // 4h .. 4h+3.  Other work is slotted between the MFMAs in an order pinned by scheduling barriers:
  //   first half : the B fragments 4..7 of this k-tile (from its own stage);
  //   barrier    : "tile kt+1 has landed in every wave's view and nobody reads stage kt&1 any more";
  //   second half: A fragment bi of the NEXT k-tile goes into the registers of A fragment bi as soon as its last MFMA of
  //                this tile has been issued (28 MFMAs before its first use), B fragments 0..3 of the next tile replace
  //                the dead ones, and one DMA instruction of tile kt+2 goes out every other MFMA into the stage just
  //                freed.  Spreading the DMA keeps the wave's in-order instruction stream from stalling behind a burst
  //                of address-coalescing requests right after the barrier.
  // No register set is double-buffered, so every k-tile runs the same code.  The last one reads "next" fragments that
  // nobody uses (from a stage that holds an older tile, or nothing yet when there is a single k-tile): cheaper than a
  // peeled copy of the tile, which costs the accumulators their fixed registers.
  // Zero the part of the last k-tile past K, each wave in the rows it fetched itself (so its own vmcnt wait covers
  // them): A and K-contiguous B rows 64w + lane, chunks ktail/16 .. 7; row-major B: whole k rows >= ktail.
  auto zero_tail = [&](int stage) {
    const v4i z = {0, 0, 0, 0};
    const int row = w * 64 + lane;
    for (int c = ktail / 16; c < 8; ++c) {
      const int off = row * 128 + ((c ^ ((row >> 1) & 7)) * 16);
      *(v4i*)(&smem[stage][0][0] + off) = z;
      if (!BROW) *(v4i*)(&smem[stage][1][0] + off) = z;
    }
    if (BROW)
      for (int r = w * 32 + (lane >> 4); r < w * 32 + 32; r += 4)
        if (r >= ktail) *(v4i*)(&smem[stage][1][0] + r * 256 + (lane & 15) * 16) = z;
  };
  const bool has_tail = EDGE && ktail != T256_BK;
  // EARLY (full tiles of a K-contiguous B): all sixteen fragments of the next tile are fetched in the second half, a
  // second barrier at the end of the tile frees this tile's stage a half tile sooner, and the DMA of tile kt+2 goes out
  // under the first half: it has a whole tile to land instead of half of one.
  constexpr bool EARLY = !EDGE && !BROW;
  v8i fa[8], fb[8];
  auto ktile = [&](int kt, auto with_dma) {
    constexpr bool dma = decltype(with_dma)::value;
    const int stage = kt & 1;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int bi = i >> 2, bj = i & 3;
      if (!EARLY && (i & 7) == 0) load_b(fb[4 + (i >> 3)], stage, 4 + (i >> 3));
      acc[bj][bi] = hx_mfma_16x16x128_e4m3(fb[bj], fa[bi], acc[bj][bi]);
      if (EARLY && (i & 1) && dma) issue_one(kt + 2, stage, i >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (EARLY && dma) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(16));  // tile kt+1 has landed; tile kt+2 stays in flight
    else HX_WAIT_VM0();
    // the last tile has just landed in the other stage.  (Only in the copy of the loop that runs the last two tiles:
    // with this branch in the main loop the compiler moves the accumulators around it, one move per MFMA.)
    if (!dma && has_tail && kt == nk - 2) zero_tail(stage ^ 1);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int bi = i >> 2, bj = 4 + (i & 3);
      acc[bj][bi] = hx_mfma_16x16x128_e4m3(fb[bj], fa[bi], acc[bj][bi]);
      if ((i & 3) == 3) load_a(fa[bi], stage ^ 1, bi);
      if ((i & 7) == 1) load_b(fb[i >> 3], stage ^ 1, i >> 3);
      if (EARLY && i >= 28) load_b(fb[4 + (i - 28)], stage ^ 1, 4 + (i - 28));  // its last MFMA of this tile is out
      if (!EARLY && (i & 1) && dma) issue_one(kt + 2, stage, i >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (EARLY) __syncthreads();  // every wave has read tile kt+1's fragments out of the other stage: it is free
  };
  issue(0, 0);
  if (nk > 1) issue(1, 1);
  if (nk > 1) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(16)); else HX_WAIT_VM0();
  if (has_tail && nk == 1) zero_tail(0);
  __syncthreads();
#pragma unroll
  for (int f = 0; f < 8; ++f) load_a(fa[f], 0, f);
#pragma unroll
  for (int f = 0; f < (EARLY ? 8 : 4); ++f) load_b(fb[f], 0, f);
  if (EARLY) __syncthreads();  // ... of stage 0
  int kt = 0;
  for (; kt + 2 < nk; ++kt) ktile(kt, std::true_type{});
  for (; kt < nk; ++kt) ktile(kt, std::false_type{});  // the last two k-tiles have nothing left to fetch
  __syncthreads();  // every wave is past its last fragment read: the LDS can be reused

  // ---- epilogue.  A lane holds only 4 consecutive columns of a row, so direct stores would hit every 128-byte line
  // of C with eight separate 16-byte writes.  Each wave instead passes 32 rows x 128 columns at a time through its own
  // quarter of the LDS and writes whole rows: 16 bytes per lane, consecutive lanes on consecutive bytes.
  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;
  constexpr int ESZ = (int)sizeof(out_t);
  constexpr int ROWB = 128 * ESZ;                    // bytes of one output row of this wave
  constexpr int RSTR = ROWB + 16;                    // padded row stride: conflict-free 8/16-byte writes down a column
  constexpr int LPR = ROWB / 16;                     // lanes per row when reading back 16 bytes per lane
  constexpr int RPI = 64 / LPR;                      // rows per store instruction
  constexpr int NBUF = (2 * 32 * RSTR <= T256_TILE_BYTES) ? 2 : 1;  // 16-bit outputs: two staging blocks per wave
  uint8_t* st = &smem[0][0][0] + w * T256_TILE_BYTES;               // this wave's 32 KB
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
  const int rb_row = lane / LPR, rb_ch = lane % LPR;
  auto stage_rows = [&](int b32) {  // accumulators of rows 32 b32 .. +31 -> staging block b32 % NBUF
    uint8_t* sb = st + (b32 % NBUF) * (32 * RSTR);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int bj = 0; bj < 8; ++bj) {
        ov4 o;
#pragma unroll
        for (int b = 0; b < 4; ++b) o[b] = (out_t)(acc[bj][2 * b32 + h][b] * alpha);
        *(ov4*)(sb + (h * 16 + r16) * RSTR + (bj * 16 + 4 * gq) * ESZ) = o;
      }
  };
  auto drain = [&](int b32) {  // staging block -> C, whole row pieces
    const uint8_t* sb = st + (b32 % NBUF) * (32 * RSTR);
#pragma unroll
    for (int p = 0; p < 32 / RPI; ++p) {
      const int row = p * RPI + rb_row;
      const v4i v = *(const v4i*)(sb + row * RSTR + rb_ch * 16);
      const long m = m0 + wm * 128 + b32 * 32 + row;
      out_t* dst = C + m * ldc + n0 + wn * 128 + rb_ch * (16 / ESZ);
      if (!EDGE) {
        *(v4i*)dst = v;
      } else if (m < M) {
        const long n = n0 + wn * 128 + rb_ch * (16 / ESZ);
        if (n + 16 / ESZ <= N && ((uintptr_t)dst & 15) == 0) {
          *(v4i*)dst = v;
        } else {
          const out_t* e = (const out_t*)&v;
          for (int b = 0; b < 16 / ESZ; ++b)
            if (n + b < N) dst[b] = e[b];
        }
      }
    }
  };
  // The LDS executes one wave's operations in order, so a block may be refilled as soon as the reads that drain it
  // have been issued; the fences only pin that program order.  With two blocks the conversion of the next row group
  // runs under the LDS and store latency of the previous one.
#pragma unroll
  for (int b32 = 0; b32 < 4 + NBUF - 1; ++b32) {
    if (b32 < 4) stage_rows(b32);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    if (b32 >= NBUF - 1) drain(b32 - (NBUF - 1));
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// ------------------------------------------------------------------------------------------
// byte transpose: src[K][N] (row stride lds_, N contiguous) -> dst[N][K] contiguous.  Turns a row-major B into
// the K-contiguous layout the MFMA kernels read; 64x64 tiles through LDS.
// ------------------------------------------------------------------------------------------
// dst_ld >= K: row stride of dst; its bytes K .. dst_ld-1 are written as zeros (a K that is padded up to the next multiple
// of 16 for the MFMA kernels).
__global__ __launch_bounds__(256) void hx_transpose_u8(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int K, int N,
                                                      long src_ld, int dst_ld) {
  __shared__ uint8_t t[64][64 + 4];
  const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    const int k = k0 + r, n = n0 + tx;
    t[r][tx] = (k < K && n < N) ? src[(long)k * src_ld + n] : (uint8_t)0;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    const int n = n0 + r, k = k0 + tx;
    if (n < N && k < dst_ld) dst[(long)n * dst_ld + k] = t[tx][r];  // k >= K: the tile holds zeros there
  }
}

// rows of K bytes (row stride src_ld, any alignment) -> rows of K16 = dst_ld bytes, zero-padded; 16 bytes per work-item
__global__ __launch_bounds__(256) void hx_pad_rows_u8(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int rows, int K,
                                                     long src_ld, int dst_ld) {
  const int cpr = dst_ld >> 4;
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long)rows * cpr) return;
  const int row = (int)(id / cpr), k0 = (int)(id % cpr) * 16;
  const uint8_t* s = src + (long)row * src_ld;
  uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
  for (int b = 0; b < 16; ++b)
    if (k0 + b < K) w[b >> 2] |= (uint32_t)s[k0 + b] << (8 * (b & 3));
  *(v4i*)(dst + (long)row * dst_ld + k0) = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
}

// ------------------------------------------------------------------------------------------
// tileN128: BM x 128 x 128 workgroup tile (BM = 64, 128 or 256), for problems that 256x256 tiles cut into too few pieces
// to occupy the chip: a decode batch of 33..256 rows against a wide weight matrix (one row tile: the kernel is then a
// weight-streaming loop and wants every CU busy and several k-tiles in flight per CU), or a mid-size square product.
// Column-major B (B^T rows of K).  4 waves (2x2) of (BM/2) x 64, 16x16x128 MFMAs, same LDS tile layout and k-block
// assignment as tile256.  LDS ring of NS stages of (A BM x 128 B + B 128 x 128 B): NS - 1 k-tiles in flight; one set
// of fragments per wave, refilled in place with k-tile kt+1's behind the MFMAs of tile kt.  Rows and columns past
// M / N re-read the last valid one and are never stored, so ragged M and N need no second instantiation.
// bn (a multiple of 16, 64..128) is the column pitch of the tiles: with a single row tile the host picks it so that
// the column tiles come to about one per CU (N = 28672: 112 columns, 256 tiles); the columns of a tile past bn
// re-read its last column (an L2 hit, no HBM traffic) and are not stored.
// ------------------------------------------------------------------------------------------
// BNT: B is streamed past a single row tile (every byte of it read once by the launch): its DMA carries the non-temporal hint.
template <int OUT, int BM, bool PAIR = false, bool BNT = false>
__global__ __launch_bounds__(256) void hx_fp8_gemm_tileN128(const uint8_t* __restrict__ A_, const uint8_t* __restrict__ Bt_,
                                                           typename OutT<OUT>::T* __restrict__ C_, int M, int N, int K, long lda,
                                                           long ldb, long ldc, const float* __restrict__ scale_a,
                                                           const float* __restrict__ scale_b, int tiles_m, int bn,
                                                           int kt_per_split) {
  typedef typename OutT<OUT>::T out_t;
  // split-K (kt_per_split != 0): workgroup row blockIdx.y multiplies k-tiles [kt0, kt0 + nk) into its own M x N slab of C_
  const int kt0 = kt_per_split * (int)blockIdx.y;
  const int nk = kt_per_split ? min(kt_per_split, K / T256_BK - kt0) : K / T256_BK;
  const uint8_t* A = A_ + (long)kt0 * T256_BK;
  const uint8_t* Bt = Bt_ + (long)kt0 * T256_BK;
  out_t* C = C_ + (kt_per_split ? (long)blockIdx.y * M * ldc : 0);
  constexpr int NS = BM == 64 ? 6 : BM == 128 ? 4 : 3;   // 144, 128 or 144 KB of LDS
  constexpr int STAGE = (BM + 128) * 128;                // bytes of one stage: A tile, then B tile
  constexpr int WMB = BM / 32;                           // 16-row blocks per wave
  constexpr int AJ = BM / 32, IPW = AJ + 4;              // DMA instructions per wave per k-tile: A, B
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NS][STAGE];

  // Grouped raster, GM row tiles tall; every 256 consecutive tiles of that order are spread over the XCDs (workgroup i
  // runs on XCD i % 8) in blocks of 32, so the tiles resident on one XCD share A and B panels in its L2.
  int tm, tn;
  {
    const int nwg = gridDim.x, wg = blockIdx.x, chunk = wg >> 8, tiles_n = nwg / tiles_m;
    // (the last, partial run of R tiles likewise in 8 blocks of R / 8 when R is a multiple of 8)
    const int rem = nwg & 255, l = wg & 255;
    const int tile = chunk < (nwg >> 8) ? (chunk << 8) + ((wg & 7) << 5) + ((wg >> 3) & 31)
                     : (rem & 7) == 0   ? (chunk << 8) + (l & 7) * (rem >> 3) + (l >> 3)
                                        : wg;
    constexpr int GM = 8;
    const int group_size = GM * tiles_n, first_m = (tile / group_size) * GM;
    const int gm = min(tiles_m - first_m, GM);
    tm = first_m + (tile % group_size) % gm;
    tn = (tile % group_size) / gm;
  }
  const long m0 = (long)tm * BM, n0 = (long)tn * bn;
  const int nlast = (int)min(n0 + bn, (long)N) - 1;  // last column this tile owns
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;

  // ---- DMA: instruction j of a tile covers rows 8j .. 8j+7; wave w issues j = w, w+4, ...  The swizzle of a lane's
  // row, ((8j + lrow) >> 1) & 7 = (4 (w & 1) + (lrow >> 1)) & 7, is the same for all of them.
  const int lrow = lane >> 3, lpos = lane & 7;
  const uint32_t chunk = (uint32_t)((lpos ^ ((4 * (w & 1) + (lrow >> 1)) & 7)) * 16);
  uint32_t a_vo[AJ], b_vo[4];
#pragma unroll
  for (int jj = 0; jj < AJ; ++jj) a_vo[jj] = (uint32_t)min((int)m0 + 8 * (w + 4 * jj) + lrow, M - 1) * (uint32_t)lda + chunk;
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) b_vo[jj] = (uint32_t)min((int)n0 + 8 * (w + 4 * jj) + lrow, nlast) * (uint32_t)ldb + chunk;
  const uint32_t lds0 = hx_lds_addr(&smem[0][0]);
  // instruction i (0 .. IPW-1) of this wave for k-tile kt; past the end: the last tile again, so that every step
  // issues IPW instructions and the counted waits stay exact
  auto issue_one = [&](int kt, int i) {
    const int t = min(kt, nk - 1);
    const uint32_t base = lds0 + (uint32_t)(kt % NS) * STAGE;
    if (i < AJ) hx_g2l16_s(hx_uniform_ptr(A + (long)t * T256_BK), a_vo[i], base + (w + 4 * i) * 1024);
    else if (BNT) hx_g2l16_s_nt(hx_uniform_ptr(Bt + (long)t * T256_BK), b_vo[i - AJ], base + BM * 128 + (w + 4 * (i - AJ)) * 1024);
    else hx_g2l16_s(hx_uniform_ptr(Bt + (long)t * T256_BK), b_vo[i - AJ], base + BM * 128 + (w + 4 * (i - AJ)) * 1024);
  };
  auto issue = [&](int kt) {
#pragma unroll
    for (int i = 0; i < IPW; ++i) issue_one(kt, i);
  };

  // ---- MFMA operands: lane (r16, gq) reads chunks 2kq, 2kq + 1 of its row (kq: k-block of the lane group, as in tile256)
  const int r16 = lane & 15, gq = lane >> 4;
  const int kq = (gq >> 1) ^ ((gq & 1) * 3);
  const int x16 = ((2 * kq) ^ ((r16 >> 1) & 7)) * 16;
  const int a_base = (wm * (BM / 2) + r16) * 128;
  const int b_base = BM * 128 + (wn * 64 + r16) * 128;
  // One set of fragments per wave, refilled in place: fragment f of A (of B) takes tile kt's rows a_base + 16 f ...
  v8i fa[WMB], fb[4];
  auto load_a = [&](int f, int kt) {
    const uint8_t* st = &smem[kt % NS][0] + a_base + f * 2048;
    const v4i lo = *(const v4i*)(st + x16), hi = *(const v4i*)(st + (x16 ^ 16));
    fa[f] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  auto load_b = [&](int f, int kt) {
    const uint8_t* st = &smem[kt % NS][0] + b_base + f * 2048;
    const v4i lo = *(const v4i*)(st + x16), hi = *(const v4i*)(st + (x16 ^ 16));
    fb[f] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  // acc[bj][bi][r] is C[m0 + wm*BM/2 + 16 bi + lane%16][n0 + wn*64 + 16 bj + 4*(lane/16) + r]
  v4f acc[4][WMB];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < WMB; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  // the MFMAs of one k-tile with the DMA instructions of tile dkt between them, one after every other MFMA (after
  // every MFMA where there are fewer than two per instruction): a burst of them right after the barrier would hold the
  // in-order instruction stream up
  constexpr int EVERY = 4 * WMB >= 2 * IPW ? 2 : 1;
  constexpr int PER = (2 * IPW + 4 * WMB - 1) / (4 * WMB);  // PAIR: DMA instructions after each MFMA of an issuing step
  // PAIR: instructions that may still be outstanding when tile kt+1 must have landed, at even / odd steps.  Pairs go out
  // at even steps as (kt+NS-1, kt+NS), interleaved, so the tile needed is the first of its pair (the pair's last
  // instruction is not its own) at even steps for an even NS and at odd steps for an odd NS.
  constexpr int W_EVEN = NS % 2 == 0 ? IPW * (NS - 4) + 1 : IPW * (NS - 3);
  constexpr int W_ODD = NS % 2 == 0 ? IPW * (NS - 2) : IPW * (NS - 3) + 1;
  static_assert(4 * WMB >= EVERY * IPW, "every DMA instruction of a k-tile has an MFMA to follow");
  // PAIR: the DMA of two consecutive k-tiles is issued in the same step, at every other step and row piece by row
  // piece, so that memory sees both 128-byte halves of 256 contiguous bytes of a row back to back (a single row tile
  // streams its weights from HBM, and lone 128-byte pieces 8 KB apart cost a DRAM row activation each: 50.5 -> 47.5 us
  // for 33..64 rows against 28672 x 8192 weights).  It needs the six-stage ring of the 64-row tile: with four stages
  // the wait for the first tile of a pair leaves nothing in flight, and 65..128 rows measured slower paired (with five
  // stages as well).
  // step kt: the fragments hold tile kt; tiles kt+1 .. are landed or in flight.  The MFMAs run A row block by row
  // block; a fragment is refilled with tile kt+1's as soon as its last MFMA of this tile has been issued (A fragment
  // bi after the four MFMAs of its row block, the B fragments during the last row block), so there is no second
  // register set and every step is the same code.  Past the last tile the refills read the ring's copy of the last
  // tile again.  Without PAIR every step issues the DMA of tile kt+NS; with it the even steps issue tiles kt+NS-1 and
  // kt+NS (the stages of tiles kt-1 and kt) and the odd steps none.
  auto step = [&](int kt, bool even) {
    // this wave's part of tile kt+1 has landed
    // (PAIR, even step: tile kt+1 is the first of its pair, so only the last instruction of that pair, which belongs to
    // the second tile, and the pairs issued since may be outstanding)
    if (!PAIR) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((NS - 2) * IPW));
    else if (even) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(PAIR ? W_EVEN : 0));
    else __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(PAIR ? W_ODD : 0));
    __syncthreads();  // ... everybody's has, and every wave has read tile kt out of its stage: that stage is free
    const int dkt = kt + NS;
#pragma unroll
    for (int i = 0; i < 4 * WMB; ++i) {
      const int bj = i & 3, bi = i >> 2;
      acc[bj][bi] = hx_mfma_16x16x128_e4m3(fb[bj], fa[bi], acc[bj][bi]);
      if (!PAIR) {
        if (i % EVERY == EVERY - 1 && i / EVERY < IPW) issue_one(dkt, i / EVERY);
      } else if (even) {  // row piece by row piece: (dkt-1, 0), (dkt, 0), (dkt-1, 1), ...; the counted waits rely on that order
#pragma unroll
        for (int q = PER * i; q < PER * (i + 1) && q < 2 * IPW; ++q) issue_one((q & 1) ? dkt : dkt - 1, q >> 1);
      }
      if (bj == 3) load_a(bi, kt + 1);
      if (bi == WMB - 1) load_b(bj, kt + 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  for (int t = 0; t < (PAIR ? NS - 1 : NS); ++t) issue(t);
  __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((PAIR ? NS - 2 : NS - 1) * IPW));
  __syncthreads();
#pragma unroll
  for (int f = 0; f < WMB; ++f) load_a(f, 0);
#pragma unroll
  for (int f = 0; f < 4; ++f) load_b(f, 0);
  // (one loop body for both kinds of step: with two copies of it the compiler shuffles the accumulators between them)
  for (int kt = 0; kt < nk; ++kt) step(kt, (kt & 1) == 0);
  HX_WAIT_VM0();  // no DMA may still be writing this workgroup's LDS when it ends

  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
  const bool vec_ok = (ldc % 4 == 0) && (((uintptr_t)C & (4 * sizeof(out_t) - 1)) == 0);
#pragma unroll
  for (int bi = 0; bi < WMB; ++bi) {
    const long m = m0 + wm * (BM / 2) + 16 * bi + r16;
    if (m >= M) continue;
#pragma unroll
    for (int bj = 0; bj < 4; ++bj) {
      const long n = n0 + wn * 64 + 16 * bj + 4 * gq;
      out_t* dst = C + m * ldc + n;
      if (n + 3 <= nlast && vec_ok) {
        ov4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = (out_t)(acc[bj][bi][r] * alpha);
        *(ov4*)dst = o;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r <= nlast) dst[r] = (out_t)(acc[bj][bi][r] * alpha);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// skinny (M <= 16): one workgroup = 8 waves; the workgroup owns column groups of 16 columns and
// streams the 16 x K bytes of B^T for each exactly once from HBM.  K is split across the waves in
// 128-byte steps (wave w takes steps w, w+8, ...); each wave accumulates a 16x16 fp32 partial with
// 16x16x128 MFMA and the 8 partials are summed through LDS.  The A panel (16 x K bytes) sits in LDS
// in MFMA-fragment order for the whole kernel when K <= SK_KC, else it is re-staged per K chunk.
// ------------------------------------------------------------------------------------------
#define SK_WAVES 8
#define SK_KC 8192        // bytes of K per LDS-resident A chunk (16 rows -> 128 KB)
#define SK_U 4            // k-steps (of 128 B) a wave loads per batch: 4 x 2 KB in flight per wave

template <int OUT>
__global__ __launch_bounds__(512) void hx_fp8_gemm_skinny(const uint8_t* __restrict__ A, const uint8_t* __restrict__ Bt,
                                                         typename OutT<OUT>::T* __restrict__ C, int M, int N, int K, long lda,
                                                         long ldb, long ldc, const float* __restrict__ scale_a,
                                                         const float* __restrict__ scale_b) {
  typedef typename OutT<OUT>::T out_t;
  __shared__ __attribute__((aligned(1024))) uint8_t sA[16 * SK_KC];  // [k-step][half][lane][16 B]
  __shared__ __attribute__((aligned(16))) float red[2][SK_WAVES][64][4];

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, g = lane >> 4;

  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;

  const int ncg = (N + 15) >> 4;
  const int nchunk = (K + SK_KC - 1) / SK_KC;
  const int arow = min(li, M - 1);
  const uint8_t* gArow = A + (long)arow * lda + g * 16;

  auto stage_A = [&](int chunk) {  // all 8 waves: k-steps of this chunk, two 1 KB DMA each
    const int k0 = chunk * SK_KC;
    const int steps = (min(K - k0, SK_KC)) >> 7;
    for (int s = w; s < steps; s += SK_WAVES) {
      hx_g2l16(gArow + k0 + s * 128, sA + s * 2048);
      hx_g2l16(gArow + k0 + s * 128 + 64, sA + s * 2048 + 1024);
    }
  };

  if (nchunk == 1) {
    stage_A(0);
    HX_WAIT_VM0();
    __syncthreads();
  }

  int parity = 0;
  for (int cg = blockIdx.x; cg < ncg; cg += gridDim.x) {
    const int brow = min(cg * 16 + li, N - 1);
    const uint8_t* gBrow = Bt + (long)brow * ldb + g * 16;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    for (int chunk = 0; chunk < nchunk; ++chunk) {
      const int k0 = chunk * SK_KC;
      const int steps = (min(K - k0, SK_KC)) >> 7;
      if (nchunk > 1) {
        __syncthreads();  // everyone done reading the previous chunk
        stage_A(chunk);
        HX_WAIT_VM0();
        __syncthreads();
      }
      // wave w: steps w, w+8, ... in batches of SK_U, register double-buffered
      const int nmine = (steps - w + SK_WAVES - 1) / SK_WAVES;  // may be <= 0
      v4i b0[SK_U][2], b1[SK_U][2];
      auto load_batch = [&](v4i(&dst)[SK_U][2], int first) {
#pragma unroll
        for (int u = 0; u < SK_U; ++u) {
          const int idx = first + u;
          if (idx < nmine) {
            const uint8_t* p = gBrow + k0 + (long)(w + idx * SK_WAVES) * 128;
            dst[u][0] = __builtin_nontemporal_load((const v4i*)p);
            dst[u][1] = __builtin_nontemporal_load((const v4i*)(p + 64));
          }
        }
      };
      auto mma_batch = [&](v4i(&src)[SK_U][2], int first) {
#pragma unroll
        for (int u = 0; u < SK_U; ++u) {
          const int idx = first + u;
          if (idx < nmine) {
            const uint8_t* pa = sA + (w + idx * SK_WAVES) * 2048 + lane * 16;
            v4i alo = *(const v4i*)pa;
            v4i ahi = *(const v4i*)(pa + 1024);
            v8i af = (v8i){alo.x, alo.y, alo.z, alo.w, ahi.x, ahi.y, ahi.z, ahi.w};
            v8i bf = (v8i){src[u][0].x, src[u][0].y, src[u][0].z, src[u][0].w,
                           src[u][1].x, src[u][1].y, src[u][1].z, src[u][1].w};
            acc = hx_mfma_16x16x128_e4m3(af, bf, acc);
          }
        }
      };
      load_batch(b0, 0);
      for (int first = 0; first < nmine; first += 2 * SK_U) {
        load_batch(b1, first + SK_U);
        mma_batch(b0, first);
        load_batch(b0, first + 2 * SK_U);
        mma_batch(b1, first + SK_U);
      }
    }
    // ---- reduce the 8 wave partials: acc[r] is C[4g + r][cg*16 + li]
    *(v4f*)&red[parity][w][lane][0] = acc;
    __syncthreads();
    if (tid < 256) {
      const int l2 = tid & 63, r = tid >> 6;
      float s = 0.f;
#pragma unroll
      for (int ww = 0; ww < SK_WAVES; ++ww) s += red[parity][ww][l2][r];
      const int m = 4 * (l2 >> 4) + r, n = cg * 16 + (l2 & 15);
      if (m < M && n < N) C[(long)m * ldc + n] = (out_t)(s * alpha);
    }
    parity ^= 1;
  }
}

// ------------------------------------------------------------------------------------------
// skinny, direct variant (M <= 16, K <= 8192): the bandwidth path.  No LDS on the load path.
// Each of the 8 waves owns k-steps w, w+8, ... (at most 8) of every column group and keeps the matching A
// fragments in registers for the whole kernel.  B^T goes straight to VGPRs with loads that cover whole
// 128-byte lines: one instruction reads 8 rows x 128 B, lane (j = lane%16, g = lane/16) taking row j>>1,
// chunk 2g + (j&1); a second instruction does rows 8..15 with the chunk parity flipped.  One exchange
// between neighbouring lanes (DPP quad_perm [1,0,3,2]) then leaves lane (j, g) with chunks 2g and 2g+1 of
// row (j>>1) + 8*(j&1): an MFMA B operand whose column j is that row.  (A lane must supply 32 bytes of ONE
// row to the MFMA, and loads of 16 rows x 64 B per instruction run ~15 % slower than whole lines.)
// The registers of a k-step are refilled with the same k-step of the next column group as soon as the MFMA
// operand has been built from them, so about one column group per wave (128 KB per CU) is always in flight,
// also across the barrier that sums the eight wave partials.
// ------------------------------------------------------------------------------------------
#define SKD_MAXS 8
// The last column groups of a launch are handed out dynamically when the caller provides a ticket word: the XCDs of an
// MI355X do not stream at the same rate (every second one finishes a static share 8-10 % later), and with one workgroup
// per CU the launch ends with its slowest CU.  Each workgroup multiplies `nstatic` groups of a fixed, strided share and
// then draws tickets (one fetch-and-add each; compare-and-swap loops of 256 workgroups on one word cost milliseconds)
// until it is told to stop, so a launch makes (dynamic groups + workgroups) draws.
// The word needs no initialisation: it holds a 40-bit tag that differs from launch to launch and a 24-bit count.
// Workgroup 0, which the hardware dispatches first, installs {tag, 0} before anything else; a draw that finds another
// tag was made before that store landed, waits for the tag and draws again (workgroup 0 waits for nobody, so the wait
// ends).  The last draw of the launch clears the word, so the replay of a captured launch finds no stale tag.
// The wait is bounded (a few milliseconds): a workgroup whose tag never comes back - two launches sharing one word at the
// same time, a misuse - stops drawing and stores {1 << 63 | tag} into the word after the ticket word; the launch then ends
// normally with the column groups that workgroup would have drawn not computed.  The library only ever sets that second
// word: a caller who wants to know zeroes it beforehand and looks at it afterwards.
#define SKD_MAX_SPINS (1 << 12)
__device__ __forceinline__ unsigned long long skd_draw_issue(unsigned long long* word) {
  // the zero offset is opaque to the compiler on purpose: for an address it can prove uniform it turns the add into a
  // wave-wide reduction and reads the answer back on the spot, and the answer is to be awaited where it is used
  long zero = 0;
  asm volatile("" : "+v"(zero));
  return __hip_atomic_fetch_add(word + zero, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int skd_draw_result(unsigned long long* word, unsigned long long old, unsigned long long tag, int nwork,
                                               int total) {
  for (int spins = 0; (old >> 24) != tag; ) {
    while ((__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 24) != tag) {
      if (++spins > SKD_MAX_SPINS) {
        __hip_atomic_store(word + 1, (1ull << 63) | tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return -1;
      }
      __builtin_amdgcn_s_sleep(32);
    }
    old = skd_draw_issue(word);
  }
  const unsigned cnt = (unsigned)(old & 0xFFFFFF);
  if (cnt + 1 == (unsigned)total) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return cnt < (unsigned)nwork ? (int)cnt : -1;
}

template <int OUT, int NS, int MB>
__global__ __launch_bounds__(512) void hx_fp8_gemm_skinny_direct(const uint8_t* __restrict__ A, const uint8_t* __restrict__ Bt,
                                                                typename OutT<OUT>::T* __restrict__ C, int M, int N, int K,
                                                                long lda, long ldb, long ldc, const float* __restrict__ scale_a,
                                                                const float* __restrict__ scale_b, unsigned long long* tickets,
                                                                unsigned long long tag) {
  typedef typename OutT<OUT>::T out_t;
  __shared__ __attribute__((aligned(16))) float red[2][SK_WAVES][MB * 4][64];  // [parity][wave][4*mb + r][lane]
  __shared__ int s_next[2];

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 15, g = lane >> 4, odd = j & 1;
  const int steps = K >> 7;
  // this wave's k-steps (wave-uniform).  NS > 0: K is NS*1024, every wave has NS steps and the compiler can count the
  // loads in flight; NS == 0: any K % 128 == 0, the steps are guarded at run time and every wait is for all loads.
  constexpr bool FULL = NS > 0;
  const int nmine = FULL ? NS : (steps - w + SK_WAVES - 1) / SK_WAVES;

  const int ncg = (N + 15) >> 4, grid = (int)gridDim.x;  // grid <= ncg: every workgroup has a first group, its own index
  const bool dynamic = MB == 1 && tickets != nullptr && ncg > grid;  // (the 32-row variant has no registers to spare)
  // static share: groups b, b + grid, ... (nstatic of them, all but the last two full rounds); ticket t is group
  // nstatic*grid + t
  const int nstatic = dynamic ? max(1, ncg / grid - 2) : 0x7fffffff;
  const int first_ticket = dynamic ? nstatic * grid : 0, nwork = ncg - first_ticket, ndraws = nwork + grid;
  if (dynamic && blockIdx.x == 0 && tid == 0)
    __hip_atomic_store(tickets, tag << 24, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  int cg = (int)blockIdx.x, cg1;  // the group being multiplied and the one after it (-1: none)
  if (nstatic > 1) {
    cg1 = cg + grid < ncg ? cg + grid : -1;
  } else {
    if (tid == 0) s_next[0] = skd_draw_result(tickets, skd_draw_issue(tickets), tag, nwork, ndraws);
    __syncthreads();
    const int t1 = __builtin_amdgcn_readfirstlane(s_next[0]);
    cg1 = t1 >= 0 ? first_ticket + t1 : -1;
  }

  // per-lane source pointers of a column group (rows clamp to N-1: those columns are never stored)
  const int c_lo = (2 * g + odd) * 16, c_hi = (2 * g + (odd ^ 1)) * 16;
  const uint8_t *p0 = Bt, *p1 = Bt;
  auto point_at = [&](int cg) {
    p0 = Bt + (long)min(cg * 16 + (j >> 1), N - 1) * ldb + c_lo + (long)w * 128;
    p1 = Bt + (long)min(cg * 16 + 8 + (j >> 1), N - 1) * ldb + c_hi + (long)w * 128;
  };
  v4i x0[SKD_MAXS], x1[SKD_MAXS];
  auto load_step = [&](int s) {
    x0[s] = __builtin_nontemporal_load((const v4i*)(p0 + (long)s * SK_WAVES * 128));
    x1[s] = __builtin_nontemporal_load((const v4i*)(p1 + (long)s * SK_WAVES * 128));
  };
  // the B stream starts before anything else touches memory
  point_at(cg);
#pragma unroll
  for (int s = 0; s < SKD_MAXS; ++s)
    if (FULL ? s < NS : s < nmine) load_step(s);

  // ---- A fragments, fetched exactly like the B rows (whole 128-byte lines per instruction, one exchange between
  // neighbouring lanes): lane (j, g) ends up with A[16*mb + (j>>1) + 8*(j&1)][128*(w + 8s) + 32g .. +31], i.e. MFMA row i
  // is matrix row (i>>1) + 8*(i&1) of the block - the store below undoes that.  (Every CU reads the same A at the same
  // moment; with 16 rows x 32 bytes per instruction, each line fetched by two instructions, those reads held the first
  // column group up for 3 us.)
  v8i af[MB][SKD_MAXS];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const uint8_t* ap0 = A + (long)min(mb * 16 + (j >> 1), M - 1) * lda + c_lo + (long)w * 128;
    const uint8_t* ap1 = A + (long)min(mb * 16 + 8 + (j >> 1), M - 1) * lda + c_hi + (long)w * 128;
#pragma unroll
    for (int s = 0; s < SKD_MAXS; ++s)
      if (FULL ? s < NS : s < nmine) {
        const v4i a0 = *(const v4i*)(ap0 + (long)s * SK_WAVES * 128);
        const v4i a1 = *(const v4i*)(ap1 + (long)s * SK_WAVES * 128);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          af[mb][s][d] = odd ? a1[d] : a0[d];
          af[mb][s][4 + d] = __builtin_amdgcn_mov_dpp(odd ? a0[d] : a1[d], 0xB1, 0xF, 0xF, true);  // from lane ^ 1
        }
        if (MB > 1) __builtin_amdgcn_sched_barrier(0);  // bounds the raw lines in flight (registers)
      }
  }
  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;

  int parity = 0, gi = 0;
  // One column group.  Whether a next group exists is a compile-time property of the body: with the refill loads under
  // a run-time condition the compiler cannot count the loads in flight and waits for the newest ones, i.e. for one full
  // memory latency per group.
  auto one_group = [&](auto more_c) {
    constexpr bool more = decltype(more_c)::value;
    // the ticket for the group after next is drawn now; its answer is picked up just before this group's barrier
    const bool draws = more && gi + 2 >= nstatic;  // uniform; no next group: told to stop (or nothing is handed out)
    unsigned long long drawn = 0;
    if (draws && tid == 0) drawn = skd_draw_issue(tickets);
    if (more) point_at(cg1);
    v4f acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SKD_MAXS; ++s)
      if (FULL ? s < NS : s < nmine) {
        v8i bf;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int lo = odd ? x1[s][d] : x0[s][d];
          const int send = odd ? x0[s][d] : x1[s][d];
          bf[d] = lo;
          bf[4 + d] = __builtin_amdgcn_mov_dpp(send, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]: lane ^ 1
        }
        if (more) load_step(s);  // the registers just consumed take this k-step of the next column group
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb] = hx_mfma_16x16x128_e4m3(af[mb][s], bf, acc[mb]);
      }
    // ---- sum the 8 wave partials: acc[mb][r] belongs to MFMA row 4g + r, column j (matrix rows / columns as below)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[parity][w][4 * mb + r][lane] = acc[mb][r];
    if (draws && tid == 0) s_next[gi & 1] = skd_draw_result(tickets, drawn, tag, nwork, ndraws);
    __syncthreads();
    if (tid < 256 * MB) {  // MB <= 2: 512 threads cover 16*MB rows x 16 columns
      const int l2 = tid & 63, rr = tid >> 6;  // rr = 4*mb + r
      float sum = 0.f;
#pragma unroll
      for (int ww = 0; ww < SK_WAVES; ++ww) sum += red[parity][ww][rr][l2];
      const int j2 = l2 & 15, i2 = 4 * (l2 >> 4) + (rr & 3);  // MFMA column / row of this value
      const int m = 16 * (rr >> 2) + (i2 >> 1) + 8 * (i2 & 1), n = cg * 16 + (j2 >> 1) + 8 * (j2 & 1);
      if (m < M && n < N) C[(long)m * ldc + n] = (out_t)(sum * alpha);
    }
    parity ^= 1;  // the next group writes the other buffer, so one barrier per group is enough
    int cg2 = -1;  // the group after next
    if (draws) {
      const int t2 = __builtin_amdgcn_readfirstlane(s_next[gi & 1]);  // slot gi & 1 is rewritten two barriers from here
      cg2 = t2 >= 0 ? first_ticket + t2 : -1;
    } else if (more && gi + 2 < nstatic) {
      cg2 = cg1 + grid < ncg ? cg1 + grid : -1;
    }
    cg = cg1;
    cg1 = cg2;
    ++gi;
  };
  while (cg1 >= 0) one_group(std::true_type{});
  one_group(std::false_type{});
}

#include "fp8_gemm_skinny_rm.h"
#include "fp8_gemm_tile256p.h"
#include "fp8_gemm_decode_ring.h"

// ------------------------------------------------------------------------------------------
// general: 64x64 tile, 256 threads, 4x4 outputs per thread, fp32 FMAs on decoded e4m3.
// ------------------------------------------------------------------------------------------
template <int OUT>
__global__ __launch_bounds__(256) void hx_fp8_gemm_general(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                          typename OutT<OUT>::T* __restrict__ C, int M, int N, int K, long lda,
                                                          long ldb_k, long ldb_n, long ldc, const float* __restrict__ scale_a,
                                                          const float* __restrict__ scale_b) {
  typedef typename OutT<OUT>::T out_t;
  __shared__ float sa[16][64 + 1];
  __shared__ float sb[16][64 + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const long m0 = (long)blockIdx.y * 64, n0 = (long)blockIdx.x * 64;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int e = tid; e < 64 * 16; e += 256) {
      const int kk = e & 15, r = e >> 4;
      const long m = m0 + r, k = k0 + kk;
      sa[kk][r] = (m < M && k < K) ? hx_e4m3_to_f32(A[m * lda + k]) : 0.f;
      const long n = n0 + r;
      sb[kk][r] = (n < N && k < K) ? hx_e4m3_to_f32(B[k * ldb_k + n * ldb_n]) : 0.f;
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
  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j) {
      const long m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < M && n < N) C[m * ldc + n] = (out_t)(acc[i][j] * alpha);
    }
}

// split-K: C = cast(alpha * sum over the splits' fp32 slabs [split][M][N]); one thread per four columns
template <int OUT>
__global__ __launch_bounds__(256) void hx_fp8_gemm_split_reduce(const float* __restrict__ part, typename OutT<OUT>::T* __restrict__ C,
                                                                int M, int N, long ldc, int splits,
                                                                const float* __restrict__ scale_a,
                                                                const float* __restrict__ scale_b) {
  typedef typename OutT<OUT>::T out_t;
  const int n4 = (N + 3) >> 2;
  const long id = (long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long)M * n4) return;
  const int m = (int)(id / n4), n = (int)(id % n4) * 4;
  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;
  const float* p = part + (long)m * N + n;
  const long slab = (long)M * N;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if ((N & 3) == 0) {
    for (int sp = 0; sp < splits; ++sp) {
      const v4f v = *(const v4f*)(p + sp * slab);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] += v[r];
    }
  } else {
    for (int sp = 0; sp < splits; ++sp)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) acc[r] += p[sp * slab + r];
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (n + r < N) C[(long)m * ldc + n + r] = (out_t)(acc[r] * alpha);
}

// ------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------
static inline bool aligned(const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// Which tile for a K-contiguous problem: 256x256 (returns 0) or 128 columns wide (returns the tile's rows: 64, 128 or
// 256).  Up to 256 rows it is one row tile, a decode batch that streams weights from HBM.  Beyond that all kernels run
// one workgroup per CU, so a launch takes ceil(tiles / 256) rounds, each of K / 128 k-tile steps plus a prologue and an
// epilogue, and the cheapest estimate wins.  Measured with every CU busy, per step and per round outside the loop:
// 256x256 1.37 us and 6 us; 128x128 0.43 us and 4.6 us (it is bound by what the CUs can pull out of the L2s, not by
// its MFMAs); 256x128 0.8 us and 9 us, and only with at least three row tiles (with two, an XCD's tiles share too few
// operand panels: 512 x 14336 x 4096 measured 40 us against 36 for 128x128).
static int tileN128_rows(int64_t M, int64_t N, int64_t K) {
  const int64_t cus = hx_cu_count();  // 256 on an MI355X
  auto rounds = [&](int64_t bm, int64_t bn) { return (((M + bm - 1) / bm) * ((N + bn - 1) / bn) + cus - 1) / cus; };
  if (M <= 64) return 64;
  if (M <= 128) return 128;
  if (M <= 256) return 256;
  const int64_t nk = (K + T256_BK - 1) / T256_BK;
  const int64_t c256 = rounds(256, 256) * (137 * nk + 600), c128 = rounds(128, 128) * (43 * nk + 460);
  const int64_t c21 = M > 512 ? rounds(256, 128) * (80 * nk + 900) : INT64_MAX;
  if (c256 <= c128 && c256 <= c21) return 0;
  return c21 < c128 ? 256 : 128;
}

// column pitch of the 128-column tiles: 128, except that a single row tile of at most 128 rows (a decode batch) gets
// about one column tile per CU (with a 256-row tile the MFMA work on the unused columns costs more than the idle CUs)
static int tileN128_pitch(int64_t M, int64_t N) {
  if (M > 128) return 128;
  const int64_t blocks = (N + 15) / 16, per = (blocks + 255) / 256;  // 16-column blocks per tile for <= 256 tiles
  return per <= 8 ? (int)(16 * (per < 4 ? 4 : per)) : 128;
}

// split-K for the 128-column tiles: when the tiles occupy less than half of the CUs and K is long, each tile's k range
// is cut into `splits` pieces of *kt_per_split k-tiles (at least 8 each), one workgroup per piece, fp32 partial sums
// in the workspace.  Returns 1 when it does not pay; the partial sums are capped at 32 MB.
static int tileN128_splits(int64_t M, int64_t N, int64_t K, int* kt_per_split) {
  *kt_per_split = 0;
  const int bm = tileN128_rows(M, N, K);
  if (bm == 0 || K % T256_BK != 0 || M <= 16 || (M <= 32 && K <= 8192)) return 1;  // other kernels take those
  const int bn = tileN128_pitch(M, N);
  const int64_t tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn), nk = K / T256_BK;
  int64_t s = 256 / tiles;
  if (s > nk / 8) s = nk / 8;
  while (s > 1 && s * M * N * 4 > (32LL << 20)) --s;
  if (s < 2) return 1;
  const int64_t per = (nk + s - 1) / s;
  *kt_per_split = (int)per;
  return (int)((nk + per - 1) / per);
}

// 0 general, 1 tile256, 2 skinny, 3 tile256 with edge tiles (M or N not a multiple of 256, K not of 128),
// 5 tileN128 (too few 256x256 tiles to occupy the chip)
static int gemm_path_kmajor(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, const void* a, const void* b,
                            const void* c) {
  const bool ok = (lda % 16 == 0) && (ldb % 16 == 0) && (K % 16 == 0) && aligned(a, 16) && aligned(b, 16) && K >= 16;
  if (!ok) return 0;
  const bool ktail = K % 128 != 0;  // only the edge instantiation of the tile kernel pads a partial last k-tile
  if (!ktail && (M <= 16 || (M <= 32 && K <= 8192)) && lda >= K && ldb >= K) return 2;
  if (lda >= (1LL << 27) || ldb >= (1LL << 27)) return 0;
  // 128-column tiles or 256x256 tiles: whichever tileN128_rows estimates to finish first
  if (!ktail && M * lda < (1LL << 32) && N * ldb < (1LL << 32) && tileN128_rows(M, N, K) != 0) return 5;
  if (!ktail && (M % 256 == 0) && (N % 256 == 0) && (ldc % 8 == 0) && aligned(c, 16)) return 1;  // 16-byte row-aligned stores
  if (M * lda < (1LL << 32) && N * ldb < (1LL << 32)) return 3;
  return 0;
}

// row-major B (N contiguous) on the tile kernel's transposing-read mode
static bool gemm_path_rowmajor_ok(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, const void* a, const void* b) {
  return M > 16 && (lda % 16 == 0) && (ldb_k % 16 == 0) && (K % 16 == 0) && K >= 16 && (N % 16 == 0) && ldb_k >= N && aligned(a, 16) &&
         aligned(b, 16) && lda < (1LL << 27) && ldb_k < (1LL << 27) && M * lda < (1LL << 32) && K * ldb_k < (1LL << 32);
}

// Any K / any alignment through the MFMA kernels (opt-in: HX_FEATURE_FP8_GEMM_ANY_K): which operands are copied into the
// workspace as zero-padded K-contiguous rows, where, and the kernel path the copies then take.
struct Repack {
  bool copy_a;
  int copy_b;  // 0 no, 1 pad rows of a K-contiguous B, 2 transpose a row-major B
  int64_t K16;
  size_t b_off, bytes;
  int path;
};
static size_t repack_bytes(int64_t M, int64_t N, int64_t K16, bool copy_a, bool copy_b, size_t* b_off) {
  size_t ab = copy_a ? (((size_t)(M * K16) + 255) & ~(size_t)255) : 0;
  *b_off = ab;
  return ab + (copy_b ? (size_t)(N * K16) : 0);
}
static bool repack_plan(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc, const void* a,
                        const void* b, const void* c, void* ws, size_t ws_bytes, Repack* rp) {
  if (!hx_feature(HX_FEATURE_FP8_GEMM_ANY_K) || !ws || !aligned(ws, 16) || K < 1) return false;
  rp->K16 = (K + 15) & ~(int64_t)15;
  rp->copy_a = !(K % 16 == 0 && lda % 16 == 0 && aligned(a, 16));
  if (ldb_k == 1) rp->copy_b = (K % 16 == 0 && ldb_n % 16 == 0 && aligned(b, 16)) ? 0 : 1;
  else if (ldb_n == 1 && ldb_k >= N) rp->copy_b = 2;
  else return false;  // B strided in both dimensions: the plain kernel
  if (!rp->copy_a && !rp->copy_b) return false;
  rp->bytes = repack_bytes(M, N, rp->K16, rp->copy_a, rp->copy_b != 0, &rp->b_off);
  if (ws_bytes < rp->bytes) return false;
  const void* a2 = rp->copy_a ? (const void*)ws : a;
  const void* b2 = rp->copy_b ? (const void*)((const uint8_t*)ws + rp->b_off) : b;
  rp->path = gemm_path_kmajor(M, N, rp->K16, rp->copy_a ? rp->K16 : lda, rp->copy_b ? rp->K16 : ldb_n, ldc, a2, b2, c);
  return rp->path != 0;
}

// Row-major B for a decode batch, streamed in place by hx_fp8_gemm_skinny_rm (opt-in: HX_FEATURE_SKINNY_ROWMAJOR).  The
// shape part of the test is what the workspace query can evaluate; the call adds strides and alignment.
static bool skinny_rm_shape_ok(int64_t M, int64_t N, int64_t K, int64_t ldb_k) {
  return hx_feature(HX_FEATURE_SKINNY_ROWMAJOR) && M >= 1 && M <= 32 && K >= 1024 && K % 1024 == 0 && N % 16 == 0 && ldb_k % 16 == 0 &&
         ldb_k >= N && 8 * ldb_k < (1LL << 32);
}
static bool skinny_rm_ok(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, const void* a, const void* b) {
  return skinny_rm_shape_ok(M, N, K, ldb_k) && lda % 8 == 0 && lda >= K && aligned(a, 8) && aligned(b, 16);
}
// k per workgroup (8192, 4096 or 1024: the kernel's instantiations) and the number of k splits: the largest piece with
// which column groups x splits still come to half the chip's CUs, else the smallest piece
static int skinny_rm_plan(int64_t N, int64_t K, int* kwg) {
  const int64_t ngroups = (N + SKR_COLS - 1) / SKR_COLS;
  for (int64_t k : {8192, 4096, 1024}) {
    if (K % k != 0) continue;
    *kwg = (int)k;
    if (ngroups * (K / k) >= 128) break;
  }
  return (int)(K / *kwg);
}

// The persistent form of the 256x256 kernel (opt-in, HX_FEATURE_FP8_GEMM_PERSISTENT) takes a problem the plain one would
// (path 1) when every workgroup gets at least two tiles and the k-tiles pair up; 16-bit outputs only (the launcher checks).
static bool tile256p_ok(int64_t M, int64_t N, int64_t K) {
  const int64_t tiles = (M / 256) * (N / 256), grid = (hx_cu_count() / 8) * 8;
  return hx_feature(HX_FEATURE_FP8_GEMM_PERSISTENT) && K % 256 == 0 && K >= 512 && grid >= 8 && tiles >= 2 * grid;
}

// decode batches of 33..256 rows on the kernel with separate A / B rings (opt-in: HX_FEATURE_FP8_GEMM_DECODE_RING), where
// hx_fp8_gemm_tileN128 runs otherwise (path 5 becomes 8)
static bool decode_ring_ok(int64_t M, int64_t N, int64_t K) {
  return hx_feature(HX_FEATURE_FP8_GEMM_DECODE_RING) && M > 32 && M <= 256 && tileN128_rows(M, N, K) != 0;
}
// its row tile: 64, 128, 192 or 256 rows
static int decode_ring_rows(int64_t M) { return M <= 64 ? 64 : M <= 128 ? 128 : M <= 192 ? 192 : 256; }

extern "C" int hx_fp8_gemm_path(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                                const void* a, const void* b, const void* c) {
  if (ldb_k == 1) {
    const int p = gemm_path_kmajor(M, N, K, lda, ldb_n, ldc, a, b, c);
    if (p == 5 && decode_ring_ok(M, N, K)) return 8;
    return p == 1 && tile256p_ok(M, N, K) ? 7 : p;
  }
  if (ldb_n == 1 && skinny_rm_ok(M, N, K, lda, ldb_k, a, b)) return 6;
  if (ldb_n == 1 && gemm_path_rowmajor_ok(M, N, K, lda, ldb_k, a, b)) return 4;
  return 0;
}

template <int OUT, int MB, int NSTEP, typename... Args>
static void launch_skinny_rm_n(bool nt, dim3 grid, hipStream_t stream, Args... args) {
  if (nt) hx_launch((hx_fp8_gemm_skinny_rm<OUT, MB, NSTEP, true>), grid, dim3(256), 0, stream, args...);
  else hx_launch((hx_fp8_gemm_skinny_rm<OUT, MB, NSTEP, false>), grid, dim3(256), 0, stream, args...);
}
template <int OUT, typename... Args>
static void launch_skinny_rm(int mb, int kwg, bool nt, dim3 grid, hipStream_t stream, Args... args) {
  if (mb == 1) {
    if (kwg == 8192) launch_skinny_rm_n<OUT, 1, 64>(nt, grid, stream, args...);
    else if (kwg == 4096) launch_skinny_rm_n<OUT, 1, 32>(nt, grid, stream, args...);
    else launch_skinny_rm_n<OUT, 1, 8>(nt, grid, stream, args...);
  } else {
    if (kwg == 8192) launch_skinny_rm_n<OUT, 2, 64>(nt, grid, stream, args...);
    else if (kwg == 4096) launch_skinny_rm_n<OUT, 2, 32>(nt, grid, stream, args...);
    else launch_skinny_rm_n<OUT, 2, 8>(nt, grid, stream, args...);
  }
}

// b_read_once: non-temporal DMA for B
template <int OUT, int BM, bool PAIR, typename... Args>
static void launch_tileN128(bool b_read_once, dim3 grid, hipStream_t stream, Args... args) {
  if (b_read_once) hx_launch((hx_fp8_gemm_tileN128<OUT, BM, PAIR, true>), grid, dim3(256), 0, stream, args...);
  else hx_launch((hx_fp8_gemm_tileN128<OUT, BM, PAIR, false>), grid, dim3(256), 0, stream, args...);
}

template <int OUT, typename... Args>
static void launch_decode_ring(int bm, bool b_read_once, dim3 grid, hipStream_t stream, Args... args) {
  if (bm == 64) {
    if (b_read_once) hx_launch((hx_fp8_gemm_decode_ring<OUT, 64, true, true>), grid, dim3(256), 0, stream, args...);
    else hx_launch((hx_fp8_gemm_decode_ring<OUT, 64, true, false>), grid, dim3(256), 0, stream, args...);
  } else if (bm == 128) {
    if (b_read_once) hx_launch((hx_fp8_gemm_decode_ring<OUT, 128, false, true>), grid, dim3(256), 0, stream, args...);
    else hx_launch((hx_fp8_gemm_decode_ring<OUT, 128, false, false>), grid, dim3(256), 0, stream, args...);
  } else if (bm == 192) {
    if (b_read_once) hx_launch((hx_fp8_gemm_decode_ring<OUT, 192, false, true>), grid, dim3(256), 0, stream, args...);
    else hx_launch((hx_fp8_gemm_decode_ring<OUT, 192, false, false>), grid, dim3(256), 0, stream, args...);
  } else {
    if (b_read_once) hx_launch((hx_fp8_gemm_decode_ring<OUT, 256, false, true>), grid, dim3(256), 0, stream, args...);
    else hx_launch((hx_fp8_gemm_decode_ring<OUT, 256, false, false>), grid, dim3(256), 0, stream, args...);
  }
}

static std::atomic<unsigned long long> g_skd_launches{0};
// The ticket tag of a decode launch: a counter scrambled together with a per-process value, so that whatever an
// uninitialised (or recycled) workspace word holds matches a launch's tag with probability 2^-40 instead of "whenever it
// holds a small integer"; never zero.
static unsigned long long skd_next_tag() {
  static const unsigned long long salt = [] {
    unsigned long long x = (unsigned long long)(uintptr_t)&g_skd_launches ^ (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count();
    return x * 0x9E3779B97F4A7C15ull;
  }();
  unsigned long long z = (g_skd_launches.fetch_add(1, std::memory_order_relaxed) + 1) * 0x9E3779B97F4A7C15ull + salt;  // splitmix64
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = (z ^ (z >> 31)) & ((1ull << 40) - 1);
  return z ? z : 1;
}

template <int OUT, int MB, typename... Args>
static void launch_skinny_direct(int ns, int grid, hipStream_t stream, Args... args) {
  switch (ns) {  // k-steps per wave as a compile-time constant where K allows it
#define HX_SKD_CASE(NS) \
  case NS:              \
    hx_launch((hx_fp8_gemm_skinny_direct<OUT, NS, MB>), dim3(grid), dim3(512), 0, stream, args...); \
    break;
    HX_SKD_CASE(1) HX_SKD_CASE(2) HX_SKD_CASE(3) HX_SKD_CASE(4) HX_SKD_CASE(5) HX_SKD_CASE(6) HX_SKD_CASE(7) HX_SKD_CASE(8)
#undef HX_SKD_CASE
    default:
      hx_launch((hx_fp8_gemm_skinny_direct<OUT, 0, MB>), dim3(grid), dim3(512), 0, stream, args...);
  }
}

template <int OUT>
static void launch_kmajor(int path, const void* a, const void* bt, void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                          int64_t ldc, const float* sa, const float* sb, void* ws, size_t ws_bytes, hipStream_t stream) {
  typedef typename OutT<OUT>::T out_t;
  if (path == 4) {  // row-major B; ldb is its row stride
    const int tiles_m = (int)((M + 255) / 256), tiles_n = (int)((N + 255) / 256);
    const bool edge = (M % 256 != 0) || (N % 256 != 0) || (K % 128 != 0) || (ldc % 8 != 0) || !aligned(c, 16);
    if (!edge)
      hx_launch((hx_fp8_gemm_tile256<OUT, false, true>), dim3(tiles_m * tiles_n), dim3(256), 0, stream, (const uint8_t*)a,
                         (const uint8_t*)bt, (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m,
                         tiles_n);
    else
      hx_launch((hx_fp8_gemm_tile256<OUT, true, true>), dim3(tiles_m * tiles_n), dim3(256), 0, stream, (const uint8_t*)a,
                         (const uint8_t*)bt, (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m,
                         tiles_n);
  } else if (path == 5 || path == 8) {  // (8: the same plan on hx_fp8_gemm_decode_ring, chosen below)
    const int bm = tileN128_rows(M, N, K), bn = tileN128_pitch(M, N);
    const int tiles_m = (int)((M + bm - 1) / bm), tiles_n = (int)((N + bn - 1) / bn);
    int ktps = 0;
    const int splits = tileN128_splits(M, N, K, &ktps);
    const bool split = splits > 1 && ws && aligned(ws, 16) && ws_bytes >= (size_t)splits * M * N * 4;
    if (!split) ktps = 0;
    const dim3 grid((unsigned)(tiles_m * tiles_n), split ? splits : 1);
    // B read exactly once by the launch, and too large to stay in the 256 MB memory-side cache between calls
    const bool b_once = tiles_m == 1 && N * K >= (192LL << 20);
    // split-K launches write unscaled fp32 slabs into the workspace; hx_fp8_gemm_split_reduce sums, scales and casts them
    if (split) {
      float* part = (float*)ws;
      if (decode_ring_ok(M, N, K))
        launch_decode_ring<HX_F32>(decode_ring_rows(M), b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt, part, (int)M, (int)N, (int)K, (long)lda,
                                   (long)ldb, (long)N, (const float*)nullptr, (const float*)nullptr, bn, ktps);
      else if (bm == 64)
        launch_tileN128<HX_F32, 64, true>(b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt,
                           part, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)N, nullptr, nullptr, tiles_m, bn, ktps);
      else if (bm == 256)
        launch_tileN128<HX_F32, 256, false>(b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt, part,
                           (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)N, nullptr, nullptr, tiles_m, bn, ktps);
      else
        launch_tileN128<HX_F32, 128, false>(b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt, part,
                           (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)N, nullptr, nullptr, tiles_m, bn, ktps);
      const long quads = (long)M * ((N + 3) / 4);
      hx_launch((hx_fp8_gemm_split_reduce<OUT>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream,
                         (const float*)part, (out_t*)c, (int)M, (int)N, (long)ldc, splits, sa, sb);
    } else if (decode_ring_ok(M, N, K)) {
      launch_decode_ring<OUT>(decode_ring_rows(M), b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt, (out_t*)c, (int)M, (int)N, (int)K, (long)lda,
                              (long)ldb, (long)ldc, sa, sb, bn, 0);
    } else if (bm == 64) {
      launch_tileN128<OUT, 64, true>(b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt,
                         (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m, bn, 0);
    } else if (bm == 256) {
      launch_tileN128<OUT, 256, false>(b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt,
                         (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m, bn, 0);
    } else {
      launch_tileN128<OUT, 128, false>(b_once, grid, stream, (const uint8_t*)a, (const uint8_t*)bt,
                         (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m, bn, 0);
    }
  } else if (path == 7 && OUT != HX_F32) {
    const int tiles_m = (int)(M / 256), tiles_n = (int)(N / 256), grid = (hx_cu_count() / 8) * 8;
    hx_launch((hx_fp8_gemm_tile256p<OUT == HX_F32 ? HX_BF16 : OUT>), dim3(grid), dim3(256), 0, stream, (const uint8_t*)a, (const uint8_t*)bt,
              (typename OutT<OUT == HX_F32 ? HX_BF16 : OUT>::T*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m,
              tiles_n);
  } else if (path == 1 || path == 3 || path == 7) {
    const int tiles_m = (int)((M + 255) / 256), tiles_n = (int)((N + 255) / 256);
    if (path != 3)
      hx_launch((hx_fp8_gemm_tile256<OUT, false, false>), dim3(tiles_m * tiles_n), dim3(256), 0, stream, (const uint8_t*)a,
                         (const uint8_t*)bt, (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m,
                         tiles_n);
    else
      hx_launch((hx_fp8_gemm_tile256<OUT, true, false>), dim3(tiles_m * tiles_n), dim3(256), 0, stream, (const uint8_t*)a,
                         (const uint8_t*)bt, (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb, tiles_m,
                         tiles_n);
  } else {  // path == 2
    const int cus = hx_cu_count();
    const int ncg = (int)((N + 15) / 16);
    const int grid = ncg < cus ? ncg : cus;
    // a ticket word for the dynamic hand-out of column groups (8 bytes of the workspace, any content)
    unsigned long long* tickets = nullptr;
    unsigned long long tag = 0;
    // (worth it from about 12 groups per workgroup: a ticket is a whole group, 4 us of work, and the spread between the
    // XCDs is 8-10 %; at 7 groups per workgroup tickets measured 0.9 us slower to 0.3 us faster than strided shares, at
    // 14 groups 3 % faster)
    if (ws && ws_bytes >= 16 && aligned(ws, 8) && ncg >= 12 * grid && ncg < (1 << 24)) {
      tickets = (unsigned long long*)ws;  // word 0: {tag, count}; word 1: the give-up record
      tag = skd_next_tag();
    }
    if (K <= 8192) {
      const int ns = K % 1024 == 0 ? (int)(K / 1024) : 0;
      if (M <= 16)
        launch_skinny_direct<OUT, 1>(ns, grid, stream, (const uint8_t*)a, (const uint8_t*)bt, (out_t*)c, (int)M, (int)N, (int)K,
                                     (long)lda, (long)ldb, (long)ldc, sa, sb, tickets, tag);
      else
        launch_skinny_direct<OUT, 2>(ns, grid, stream, (const uint8_t*)a, (const uint8_t*)bt, (out_t*)c, (int)M, (int)N, (int)K,
                                     (long)lda, (long)ldb, (long)ldc, sa, sb, tickets, tag);
    } else
      hx_launch(hx_fp8_gemm_skinny<OUT>, dim3(grid), dim3(512), 0, stream, (const uint8_t*)a, (const uint8_t*)bt,
                         (out_t*)c, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, sa, sb);
  }
}

template <int OUT>
static int launch_fp8_gemm(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                           int64_t ldb_n, int64_t ldc, const float* sa, const float* sb, void* ws, size_t ws_bytes,
                           hipStream_t stream) {
  typedef typename OutT<OUT>::T out_t;
  int path = hx_fp8_gemm_path(M, N, K, lda, ldb_k, ldb_n, ldc, a, b, c);
  if (path == 6) {
    int kwg = 1024;
    const int splits = skinny_rm_plan(N, K, &kwg);
    const int ngroups = (int)((N + SKR_COLS - 1) / SKR_COLS), cus = hx_cu_count();
    const bool nt = N * K >= (192LL << 20);
    const int mb = M <= 16 ? 1 : 2;
    if (splits == 1) {
      launch_skinny_rm<OUT>(mb, kwg, nt, dim3((unsigned)(ngroups < cus ? ngroups : cus), 1), stream, (const uint8_t*)a,
                            (const uint8_t*)b, (out_t*)c, (int)M, (int)N, (long)lda, (long)ldb_k, (long)ldc, sa, sb, ngroups, 0L);
    } else if (ws && aligned(ws, 16) && ws_bytes >= (size_t)splits * M * N * 4) {
      // every split writes an unscaled fp32 slab; hx_fp8_gemm_split_reduce sums them in a fixed order, scales and casts
      float* part = (float*)ws;
      launch_skinny_rm<HX_F32>(mb, kwg, nt, dim3((unsigned)(ngroups < cus ? ngroups : cus), (unsigned)splits), stream,
                               (const uint8_t*)a, (const uint8_t*)b, part, (int)M, (int)N, (long)lda, (long)ldb_k, (long)N,
                               (const float*)nullptr, (const float*)nullptr, ngroups, (long)(M * N));
      const long quads = (long)M * ((N + 3) / 4);
      hx_launch((hx_fp8_gemm_split_reduce<OUT>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream, (const float*)part,
                (out_t*)c, (int)M, (int)N, (long)ldc, splits, sa, sb);
    } else {
      path = gemm_path_rowmajor_ok(M, N, K, lda, ldb_k, a, b) ? 4 : 0;  // no room for the partial sums: the paths without them
    }
  }
  if (path == 6) {
  } else if (path != 0) {
    launch_kmajor<OUT>(path, a, b, c, M, N, K, lda, path == 4 ? ldb_k : ldb_n, ldc, sa, sb, ws, ws_bytes, stream);
  } else {
    // row-major B with a workspace: transpose it once into K-contiguous form, then take a fast path
    int tpath = 0;
    Repack rp;
    if (ldb_n == 1 && ldb_k >= N && ws && ws_bytes >= (size_t)(N * K) && aligned(ws, 16))
      tpath = gemm_path_kmajor(M, N, K, lda, K, ldc, a, ws, c);
    if (tpath != 0) {
      dim3 tg((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
      hx_launch(hx_transpose_u8, tg, dim3(256), 0, stream, (const uint8_t*)b, (uint8_t*)ws, (int)K, (int)N, (long)ldb_k, (int)K);
      launch_kmajor<OUT>(tpath, a, ws, c, M, N, K, lda, K, ldc, sa, sb, nullptr, 0, stream);
    } else if (repack_plan(M, N, K, lda, ldb_k, ldb_n, ldc, a, b, c, ws, ws_bytes, &rp)) {
      // Any K, any alignment (opt-in): A and / or B are copied once into the workspace as K-contiguous rows padded with
      // zeros to K16 = the next multiple of 16 - zeros add nothing to a dot product - and the MFMA kernels run on the copies.
      uint8_t* wa = (uint8_t*)ws;
      uint8_t* wb = (uint8_t*)ws + rp.b_off;
      if (rp.copy_a)
        hx_launch(hx_pad_rows_u8, dim3((unsigned)((M * (rp.K16 / 16) + 255) / 256)), dim3(256), 0, stream, (const uint8_t*)a, wa, (int)M,
                  (int)K, (long)lda, (int)rp.K16);
      if (rp.copy_b == 1)
        hx_launch(hx_pad_rows_u8, dim3((unsigned)((N * (rp.K16 / 16) + 255) / 256)), dim3(256), 0, stream, (const uint8_t*)b, wb, (int)N,
                  (int)K, (long)ldb_n, (int)rp.K16);
      else if (rp.copy_b == 2)
        hx_launch(hx_transpose_u8, dim3((unsigned)((N + 63) / 64), (unsigned)((rp.K16 + 63) / 64)), dim3(256), 0, stream, (const uint8_t*)b,
                  wb, (int)K, (int)N, (long)ldb_k, (int)rp.K16);
      launch_kmajor<OUT>(rp.path, rp.copy_a ? (const void*)wa : a, rp.copy_b ? (const void*)wb : b, c, M, N, rp.K16,
                         rp.copy_a ? rp.K16 : lda, rp.copy_b ? rp.K16 : ldb_n, ldc, sa, sb, nullptr, 0, stream);
    } else {
      dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
      hx_launch(hx_fp8_gemm_general<OUT>, grid, dim3(256), 0, stream, (const uint8_t*)a, (const uint8_t*)b, (out_t*)c,
                         (int)M, (int)N, (int)K, (long)lda, (long)ldb_k, (long)ldb_n, (long)ldc, sa, sb);
    }
  }
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_fp8_gemm: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

extern "C" size_t hx_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t ldb_k, int64_t ldb_n) {
  // A row-major B (N contiguous) that the tile kernel cannot read in place (M <= 16: the skinny kernel wants K
  // contiguous; N or the row stride not a multiple of 16) but that could take a fast path after a transpose needs
  // N*K bytes of scratch; a column-major B needs scratch only for split-K partial sums.
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  if (hx_feature(HX_FEATURE_FP8_GEMM_ANY_K) && K % 16 != 0 && (ldb_k == 1 || ldb_n == 1)) {  // both operands repacked, K padded
    size_t off;
    return repack_bytes(M, N, (K + 15) & ~(int64_t)15, true, true, &off);
  }
  if (ldb_k == 1) {  // column-major B: fp32 partial sums when the 128-column tile kernel would split K
    int ktps = 0;
    const int splits = tileN128_splits(M, N, K, &ktps);
    if (splits > 1) return (size_t)splits * M * N * 4;
    // the decode kernel's ticket word (dynamic hand-out of column groups), used from 12 groups per CU of an MI355X
    return M <= 16 && K <= 8192 && (N + 15) / 16 >= 12 * 256 ? 16 : 0;
  }
  if (ldb_n != 1 || K % 16 != 0) return 0;
  if (skinny_rm_shape_ok(M, N, K, ldb_k)) {  // streamed in place: fp32 partial sums only when K is split over workgroups
    int kwg = 1024;
    const int splits = skinny_rm_plan(N, K, &kwg);
    return splits > 1 ? (size_t)splits * M * N * 4 : 0;
  }
  if (M > 16 && N % 16 == 0 && ldb_k % 16 == 0) return 0;
  return (size_t)(N * K);
}

extern "C" int hx_fp8_gemm(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                           int64_t ldb_n, int64_t ldc, const float* scale_a, const float* scale_b, int out_dtype,
                           void* workspace, size_t workspace_bytes, void* stream) {
  if (M < 0 || N < 0 || K < 0) {
    hx_set_error("hx_fp8_gemm: negative size M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    return HX_ERR_BAD_ARG;
  }
  if (M == 0 || N == 0) return 0;
  if (!c || (K > 0 && (!a || !b))) {
    hx_set_error("hx_fp8_gemm: null operand pointer");
    return HX_ERR_BAD_ARG;
  }
  if (M >= (1LL << 31) || N >= (1LL << 31) || K >= (1LL << 31)) {
    hx_set_error("hx_fp8_gemm: dimension exceeds int32");
    return HX_ERR_UNSUPPORTED;
  }
  if (lda < K || ldc < N) {
    hx_set_error("hx_fp8_gemm: leading dimension smaller than row length (lda=%lld K=%lld ldc=%lld N=%lld)",
                 (long long)lda, (long long)K, (long long)ldc, (long long)N);
    return HX_ERR_BAD_ARG;
  }
  hipStream_t s = (hipStream_t)stream;
  switch (out_dtype) {
    case HX_F16: return launch_fp8_gemm<HX_F16>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, scale_a, scale_b, workspace, workspace_bytes, s);
    case HX_BF16: return launch_fp8_gemm<HX_BF16>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, scale_a, scale_b, workspace, workspace_bytes, s);
    case HX_F32: return launch_fp8_gemm<HX_F32>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, scale_a, scale_b, workspace, workspace_bytes, s);
    default:
      hx_set_error("hx_fp8_gemm: unknown out_dtype tag %d", out_dtype);
      return HX_ERR_BAD_ARG;
  }
}
