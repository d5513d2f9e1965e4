// hx_fp8_gemm_decode_ring: the FP8 GEMM for a decode batch of 33..256 rows against a wide column-major weight matrix
// (B^T rows of K): one row tile, so the kernel is a weight-streaming loop bound by HBM, and what decides its speed is how
// many weight bytes every CU keeps in flight.
//
// Same BM x 128 x 128 workgroup tile, LDS tile layout, fragment assignment and MFMA order as hx_fp8_gemm_tileN128 (its
// results are the same bit for bit), but A and B have rings of their own in the LDS and wave streams of their own:
//   * waves 0 and 1 issue all DMA of A (BM x 128 bytes per k-tile; the same few rows for every workgroup, so L2 hits with
//     a short latency): a ring of 3 stages is enough;
//   * waves 2 and 3 issue all DMA of B (128 columns x 128 bytes per k-tile, from HBM): a ring of 8 / 7 / 5 / 4 stages of
//     16 KB for BM = 64 / 128 / 192 / 256 (whatever the A ring leaves of the 160 KB), so that six / five / three / two of
//     them are in flight while one is consumed and one is being refilled.
// A wave's vmcnt counts only its own instructions and they complete in order, so a single stream carrying both operands
// would tie B's depth to A's: waiting for a recently issued A tile would also wait for every B tile issued before it.
// With one stage ring for both (tileN128) the 128-row tile has two to three B stages in flight (32 - 48 KB per CU) and the
// 256-row tile one to two.  BM = 192 exists only here: 129..192 rows do three quarters of the 256-row tile's MFMAs.
// PAIR (BM = 64): the B waves issue two consecutive k-tiles together at every other step, row piece by row piece, so
// that memory sees 256 contiguous bytes of a weight row back to back.
// All four waves multiply; the barrier at the top of a step makes both streams' landed tiles visible to everybody.
#pragma once
#include <type_traits>

#include "hx_common.h"

// bn: column pitch of the tiles (a multiple of 16, 64..128: about one tile per CU); kt_per_split != 0: workgroup row
// blockIdx.y multiplies k-tiles [kt0, kt0 + nk) into its own M x N slab of C_.
// BNT: B is read exactly once by the launch and is too large to stay cached between calls: its DMA is non-temporal.
template <int OUT, int BM, bool PAIR, bool BNT>
__global__ __launch_bounds__(256) void hx_fp8_gemm_decode_ring(const uint8_t* __restrict__ A_, const uint8_t* __restrict__ Bt_,
                                                              typename OutT<OUT>::T* __restrict__ C_, int M, int N, int K, long lda,
                                                              long ldb, long ldc, const float* __restrict__ scale_a,
                                                              const float* __restrict__ scale_b, int bn, int kt_per_split) {
  typedef typename OutT<OUT>::T out_t;
  static_assert(BM == 64 || BM == 128 || BM == 192 || BM == 256, "one row tile of 64, 128, 192 or 256 rows");
  constexpr int BK = 128;
  constexpr int NA = 3, NB = BM == 64 ? 8 : BM == 128 ? 7 : BM == 192 ? 5 : 4;
  static_assert(!PAIR || NB % 2 == 0, "pairs of k-tiles need an even ring");
  constexpr int ASTAGE = BM * 128, BSTAGE = 128 * 128;
  constexpr int WMB = BM / 32;  // 16-row blocks per wave
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NA * ASTAGE + NB * BSTAGE];  // 152 / 160 / 152 / 160 KB
  const int kt0 = kt_per_split * (int)blockIdx.y;
  const int nk = kt_per_split ? min(kt_per_split, K / BK - kt0) : K / BK;
  const uint8_t* A = A_ + (long)kt0 * BK;
  const uint8_t* Bt = Bt_ + (long)kt0 * BK;
  out_t* C = C_ + (kt_per_split ? (long)blockIdx.y * M * ldc : 0);

  const long n0 = (long)blockIdx.x * bn;
  const int nlast = (int)min(n0 + bn, (long)N) - 1;  // last column this tile owns
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;

  // ---- DMA: instruction j of a tile covers rows 8j .. 8j+7 (1 KB); of its operand's tile, wave wr = w % 2 issues
  // j = wr, wr + 2, ...  The swizzle of a lane's row, ((8j + lrow) >> 1) & 7 = (4 wr + (lrow >> 1)) & 7, is the same for all.
  // Rows past M (columns past the tile's last) re-read the last valid one and are never stored.
  const int wr = w & 1;
  const int lrow = lane >> 3, lpos = lane & 7;
  const uint32_t chunk = (uint32_t)((lpos ^ ((4 * wr + (lrow >> 1)) & 7)) * 16);
  const uint32_t lds0 = hx_lds_addr(&smem[0]);

  // ---- MFMA operands (as in tileN128): lane (r16, gq) reads chunks 2kq, 2kq + 1 of its row
  const int r16 = lane & 15, gq = lane >> 4;
  const int kq = (gq >> 1) ^ ((gq & 1) * 3);
  const int x16 = ((2 * kq) ^ ((r16 >> 1) & 7)) * 16;
  const int a_base = (wm * (BM / 2) + r16) * 128;
  const int b_base = NA * ASTAGE + (wn * 64 + r16) * 128;
  v8i fa[WMB], fb[4];
  auto load_a = [&](int f, int kt) {
    const uint8_t* st = &smem[0] + (kt % NA) * ASTAGE + a_base + f * 2048;
    const v4i lo = *(const v4i*)(st + x16), hi = *(const v4i*)(st + (x16 ^ 16));
    fa[f] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  auto load_b = [&](int f, int kt) {
    const uint8_t* st = &smem[0] + (kt % NB) * BSTAGE + b_base + f * 2048;
    const v4i lo = *(const v4i*)(st + x16), hi = *(const v4i*)(st + (x16 ^ 16));
    fb[f] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  // acc[bj][bi][r] is C[wm*BM/2 + 16 bi + lane%16][n0 + wn*64 + 16 bj + 4*(lane/16) + r]
  v4f acc[4][WMB];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < WMB; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  // The whole k-loop, once for each kind of wave (a wave runs one of the two copies from start to end, so the
  // accumulators meet only once, after the loop).  RA: this wave streams A; otherwise B.
  auto run = [&](auto role) {
    constexpr bool RA = decltype(role)::value;
    constexpr int IP = RA ? BM / 16 : 8;  // DMA instructions per wave per k-tile
    constexpr int NR = RA ? NA : NB;      // this stream's ring
    constexpr int STG = RA ? ASTAGE : BSTAGE;
    constexpr bool PR = PAIR && !RA;
    const uint8_t* src = RA ? A : Bt;
    const uint32_t ring0 = lds0 + (RA ? 0 : NA * ASTAGE);
    uint32_t vo[IP];
#pragma unroll
    for (int i = 0; i < IP; ++i) {
      const int row = 8 * (wr + 2 * i) + lrow;
      vo[i] = RA ? (uint32_t)min(row, M - 1) * (uint32_t)lda + chunk : (uint32_t)min((int)n0 + row, nlast) * (uint32_t)ldb + chunk;
    }
    // instruction i of this wave for k-tile kt; past the end: the last tile again, into the stage of a tile nobody reads
    // any more, so that every step issues the same number of instructions and the counted waits stay exact
    auto issue_one = [&](int kt, int i) {
      const int t = min(kt, nk - 1);
      const uint32_t dst = ring0 + (uint32_t)(kt % NR) * STG + (wr + 2 * i) * 1024;
      if (!RA && BNT) hx_g2l16_s_nt(hx_uniform_ptr(src + (long)t * BK), vo[i], dst);
      else hx_g2l16_s(hx_uniform_ptr(src + (long)t * BK), vo[i], dst);
    };
    constexpr int NMF = 4 * WMB;                       // MFMAs per step
    constexpr int EVERY = NMF >= 2 * IP ? 2 : 1;       // plain steps: one DMA instruction after every EVERY-th MFMA
    constexpr int PER = (2 * IP + NMF - 1) / NMF;      // pair steps: DMA instructions after each MFMA
    static_assert(NMF >= EVERY * IP, "every DMA instruction of a k-tile has an MFMA to follow");
    // Pair steps: pairs go out at even steps as tiles (kt + NR - 1, kt + NR), interleaved, into the stages of tiles kt - 1
    // and kt.  NR is even, so the tile needed next (kt + 1) is the first of its pair at even steps - the pair's last
    // instruction is not its own and may be outstanding, with the (NR - 4) / 2 pairs issued since - and the second of its
    // pair at odd steps, followed by (NR - 2) / 2 pairs.
    constexpr int W_EVEN = IP * (NR - 4) + 1, W_ODD = IP * (NR - 2);

    constexpr int PRO = PR ? NR - 1 : NR;  // tiles in flight before the first step
    for (int t = 0; t < PRO; ++t)
#pragma unroll
      for (int i = 0; i < IP; ++i) issue_one(t, i);
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((PRO - 1) * IP));  // this wave's part of tile 0 has landed
    __syncthreads();
#pragma unroll
    for (int f = 0; f < WMB; ++f) load_a(f, 0);
#pragma unroll
    for (int f = 0; f < 4; ++f) load_b(f, 0);

    // step kt: the fragments hold tile kt; tile kt+1 must have landed (the refills read it); the stage of tile kt is free.
    for (int kt = 0; kt < nk; ++kt) {
      const bool even = (kt & 1) == 0;
      if (!PR) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((NR - 2) * IP));
      else if (even) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(PR ? W_EVEN : 0));
      else __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(PR ? W_ODD : 0));
      __syncthreads();  // both streams' tile kt+1 is visible to everybody, and everybody has read tile kt out of its stages
#pragma unroll
      for (int i = 0; i < NMF; ++i) {
        const int bj = i & 3, bi = i >> 2;
        acc[bj][bi] = hx_mfma_16x16x128_e4m3(fb[bj], fa[bi], acc[bj][bi]);
        if (!PR) {
          if (i % EVERY == EVERY - 1 && i / EVERY < IP) issue_one(kt + NR, i / EVERY);
        } else if (even) {  // row piece by row piece: (first, 0), (second, 0), (first, 1), ...; the counted waits rely on that order
#pragma unroll
          for (int q = PER * i; q < PER * (i + 1) && q < 2 * IP; ++q) issue_one((q & 1) ? kt + NR : kt + NR - 1, q >> 1);
        }
        if (bj == 3) load_a(bi, kt + 1);
        if (bi == WMB - 1) load_b(bj, kt + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  if (w < 2) run(std::true_type{});
  else run(std::false_type{});
  HX_WAIT_VM0();  // no DMA may still be writing this workgroup's LDS when it ends

  float alpha = 1.f;
  if (scale_a) alpha = *scale_a;
  if (scale_b) alpha = alpha * *scale_b;
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
  const bool vec_ok = (ldc % 4 == 0) && (((uintptr_t)C & (4 * sizeof(out_t) - 1)) == 0);
#pragma unroll
  for (int bi = 0; bi < WMB; ++bi) {
    const long m = wm * (BM / 2) + 16 * bi + r16;
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
