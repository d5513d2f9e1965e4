// Dense matmul with a fused epilogue for gfx950 — device side of the reference's examples/matmul.py:25-56 and
// examples/matmul_split_k.py:30-68:
//   C = cast( act( fp32(A) @ fp32(B) + bias[None, :] ) ),   act = identity | relu,  fp32 accumulation.
// A [M,K], B [K,N] row-major or column-major, bias [N] or absent.  bf16 / fp16 operands run the 256x256x64 MFMA tile kernel that the grouped
// (MoE) GEMM uses; K can be split over workgroups (blockIdx.y), the fp32 partial sums then go through the workspace and
// a second kernel adds them up, applies the epilogue and casts.  The reference's split-K accumulates with atomics in
// the output type and applies the epilogue to the first split only; its result for one split — which is what its eager
// mode computes — is the formula above, and that is what every split count gives here.
// Anything the tile kernel does not cover (fp32 operands, odd sizes, strided B) runs a plain fp32-FMA kernel.
#include "gemm16_tile128.h"
#include "gemm16_tile256p.h"

template <typename T>
__device__ __forceinline__ float mm_ld(const T* p) { return (float)*p; }

// 64x64 outputs per workgroup, 16 k per step, fp32 FMAs; any sizes and strides
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void hx_matmul_general(const TI* __restrict__ A, const TI* __restrict__ B, TO* __restrict__ C, int M,
                                                        int N, int K, long lda, long ldb_k, long ldb_n, long ldc,
                                                        const void* __restrict__ bias, int bias_f32, int relu) {
  __shared__ float sa[16][64 + 1];
  __shared__ float sb[16][64 + 1];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const long m0 = (long)blockIdx.x * 64, n0 = (long)blockIdx.y * 64;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int e = tid; e < 64 * 16; e += 256) {
      const int kk = e & 15, r = e >> 4;
      const long m = m0 + r, k = k0 + kk;
      sa[kk][r] = (m < M && k < K) ? mm_ld(A + m * lda + k) : 0.f;
    }
    for (int e = tid; e < 64 * 16; e += 256) {
      const int c = ldb_n == 1 ? (e & 63) : (e >> 4), kk = ldb_n == 1 ? (e >> 6) : (e & 15);
      const long k = k0 + kk, n = n0 + c;
      sb[kk][c] = (n < N && k < K) ? mm_ld(B + k * ldb_k + n * ldb_n) : 0.f;
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
    const long m = m0 + ty * 4 + i;
    if (m >= M) continue;
    for (int j = 0; j < 4; ++j) {
      const long n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias_f32 ? ((const float*)bias)[n] : (float)((const TI*)bias)[n];
      if (relu) v = fmaxf(v, 0.f);
      C[m * ldc + n] = (TO)v;
    }
  }
}

// C[m, n..n+3] = cast(act(sum_s part[s][m][n..] + bias[n..])); part is [S][M][N] fp32, N % 4 == 0.
// A workgroup covers 16 groups of 4 columns; 16 threads share each group's splits (s = lane, lane + 16, ...: many
// splits of a small output would otherwise be one long chain of loads per thread) and are summed through LDS in a
// fixed order, so the result does not depend on the launch.
template <typename TB, typename TO>
__global__ __launch_bounds__(256) void hx_matmul16_reduce(const float* __restrict__ part, int S, int M, int N, TO* __restrict__ C,
                                                         long ldc, const void* __restrict__ bias, int bias_f32, int relu) {
  __shared__ v4f red[16][16];
  const int gl = threadIdx.x & 15, sl = threadIdx.x >> 4;
  const long q = (long)blockIdx.x * 16 + gl;  // group of 4 columns
  const int nq = N >> 2;
  const bool live = q < (long)M * nq;
  const long m = live ? q / nq : 0, n = live ? (q % nq) * 4 : 0;
  const long plane = (long)M * N;
  v4f v = {0.f, 0.f, 0.f, 0.f};
  if (live)
    for (int s = sl; s < S; s += 16) v += *(const v4f*)(part + s * plane + m * N + n);
  red[sl][gl] = v;
  __syncthreads();
  if (sl != 0 || !live) return;
#pragma unroll
  for (int i = 1; i < 16; ++i) v += red[i][gl];
  if (bias) {
#pragma unroll
    for (int b = 0; b < 4; ++b) v[b] += bias_f32 ? ((const float*)bias)[n + b] : (float)((const TB*)bias)[n + b];
  }
  if (relu) {
#pragma unroll
    for (int b = 0; b < 4; ++b) v[b] = fmaxf(v[b], 0.f);
  }
#pragma unroll
  for (int b = 0; b < 4; ++b) C[m * ldc + n + b] = (TO)v[b];
}

// ------------------------------------------------------------------------------------------
static bool mm_fast_ok(const void* a, const void* b, const void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                       int64_t ldb_n, int64_t ldc, const void* bias, int in_dtype) {
  if (in_dtype != HX_BF16 && in_dtype != HX_F16) return false;
  if (K < MOE_BK || K % MOE_BK || N % 8 || lda % 8 || ldc % 8) return false;  // 16-byte row pieces in and out
  if ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)bias) & 15) != 0) return false;
  if (M * lda * 2 >= (1LL << 32)) return false;
  if (ldb_n == 1) return ldb_k % 8 == 0 && ldb_k * 4 < (1LL << 31);               // row-major B
  if (ldb_k == 1) return ldb_n % 8 == 0 && ldb_n >= K && N * ldb_n * 2 < (1LL << 32);  // column-major B (B^T rows of K)
  return false;
}

// Tile size and K split for a problem the tile kernels take.  256x256 tiles unless they would leave most of the chip
// idle; an automatic split (split_k <= 0) only while the workgroups do not fill the chip, every split keeps at least
// eight k-tiles (a split costs a second launch) and the fp32 partial sums, which are written and read again, stay below
// half the operand bytes.
struct MmPlan {
  int tile, splits;
};
static MmPlan mm_plan(int64_t M, int64_t N, int64_t K, int split_k) {
  const int64_t nkt = K / MOE_BK;
  const int64_t t256 = ((M + 255) / 256) * ((N + 255) / 256);
  MmPlan p;
  p.tile = t256 > 128 ? 256 : 128;  // (measured: at 112-128 tiles of 256x256 the small tile is 15-40 % faster, at 160 it is 25 % slower)
  const int64_t tiles = ((M + p.tile - 1) / p.tile) * ((N + p.tile - 1) / p.tile);
  // resident workgroups to aim for: one per CU (with 128x128 tiles a deep LDS ring then keeps several k-tiles in flight;
  // two workgroups per CU with a shallow ring are for problems that have the tiles anyway)
  const int64_t room = 256;
  int64_t s = split_k;
  if (s <= 0) {
    s = 1;
    const int64_t cap = (M + N) * K;  // half the operand bytes
    while (tiles * s * 2 <= room && nkt / (s * 2) >= 8 && (s * 2) * M * N * 4 <= cap) s *= 2;
  }
  if (s > nkt) s = nkt;
  if (s > 65535) s = 65535;
  if (s < 1) s = 1;
  const int64_t per = (nkt + s - 1) / s;
  p.splits = (int)((nkt + per - 1) / per);
  return p;
}

extern "C" int hx_matmul_splits(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc, int in_dtype,
                                int split_k) {
  if (M <= 0 || N <= 0 || K <= 0) return 1;
  // alignment of the pointers is not known here; the launcher re-checks and falls back to one split
  if (!mm_fast_ok(nullptr, nullptr, nullptr, M, N, K, lda, ldb_k, ldb_n, ldc, nullptr, in_dtype)) return 1;
  return mm_plan(M, N, K, split_k).splits;
}

extern "C" size_t hx_matmul_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                                            int in_dtype, int out_dtype, int has_epilogue, int split_k) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  if (!mm_fast_ok(nullptr, nullptr, nullptr, M, N, K, lda, ldb_k, ldb_n, ldc, nullptr, in_dtype)) return 0;
  const int s = mm_plan(M, N, K, split_k).splits;
  const bool partial = s > 1 || (out_dtype == HX_F32 && has_epilogue);
  return partial ? (size_t)s * M * N * 4 : 0;
}

template <typename TI, typename TO>
static void mm_launch_general(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                              int64_t ldb_n, int64_t ldc, const void* bias, int bias_f32, int relu, hipStream_t s) {
  dim3 grid((unsigned)((M + 63) / 64), (unsigned)((N + 63) / 64));
  hx_launch((hx_matmul_general<TI, TO>), grid, dim3(256), 0, s, (const TI*)a, (const TI*)b, (TO*)c, (int)M, (int)N, (int)K,
                     (long)lda, (long)ldb_k, (long)ldb_n, (long)ldc, bias, bias_f32, relu);
}

// The dense 256x256 kernel in persistent workgroups (opt-in, HX_FEATURE_MATMUL_PERSISTENT): a row-major B, no epilogue, a
// 16-bit output, whole tiles, an even number (at least four) of k-tiles, and at least two tiles for every workgroup.
static bool mm_persistent_ok(int64_t M, int64_t N, int64_t K, int64_t ldb_n, const void* bias, int relu, int out_dtype, int tile, int splits) {
  const int64_t grid = (hx_cu_count() / 8) * 8;
  return hx_feature(HX_FEATURE_MATMUL_PERSISTENT) && tile == 256 && splits == 1 && ldb_n == 1 && !bias && !relu && out_dtype != HX_F32 &&
         M % MOE_BM == 0 && N % MOE_BN == 0 && K % (2 * MOE_BK) == 0 && K >= 4 * MOE_BK && grid >= 8 && (M / MOE_BM) * (N / MOE_BN) >= 2 * grid;
}

template <bool BF, bool BCOL>
static void mm_launch_fast(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                           int64_t ldc, const void* bias, int bias_f32, int relu, int out_dtype, int tile, int splits, void* ws,
                           hipStream_t s) {
  typedef typename Mfma16<BF>::T T16;
  const int tiles_m = (int)((M + tile - 1) / tile), tiles_n = (int)((N + tile - 1) / tile);
  G16Dense d = {};
  d.lda = lda; d.ldb = ldb_k; d.bias = bias; d.bias_f32 = bias_f32; d.relu = relu;
  // one row tile and a weight matrix too large to stay in the 256 MB memory-side cache between calls: stream it
  d.w_once = tiles_m == 1 && K * N * 2 >= (192LL << 20);
  const bool partial = splits > 1 || (out_dtype == HX_F32 && (bias || relu));
  if (!partial && out_dtype != HX_F32) {
    d.ldc = ldc;
    if (!BCOL && mm_persistent_ok(M, N, K, 1, bias, relu, out_dtype, tile, splits))
      hx_launch((hx_gemm16_tile256p<BF, true>), dim3((hx_cu_count() / 8) * 8), dim3(256), 0, s, (const uint8_t*)a, (const uint8_t*)b, c,
                (const int*)nullptr, (const MoeTile*)nullptr, (const int32_t*)nullptr, (int)M, (int)K, (int)N, tiles_n, 1, (uint8_t*)c, (long)lda,
                (long)ldb_k, (long)ldc, tiles_m);
    else if (tile == 256)
      hx_launch((hx_gemm16_tile256<BF, 1, BCOL>), dim3(tiles_m * tiles_n), dim3(256), 0, s, (const uint8_t*)a, (const uint8_t*)b, c,
                         (const int*)nullptr, (const MoeTile*)nullptr, (const int32_t*)nullptr, (int)M, (int)K, (int)N, tiles_m, tiles_n, 1, d);
    else if (tiles_m * tiles_n <= 256)
      hx_launch((hx_gemm16_tile128<BF, 1, BCOL, 4>), dim3(tiles_m * tiles_n), dim3(256), 0, s, (const uint8_t*)a, (const uint8_t*)b,
                         c, (const int*)nullptr, (const MoeTile*)nullptr, (const int32_t*)nullptr, (int)M, (int)K, (int)N, tiles_m, tiles_n, 1,
                         d);
    else
      hx_launch((hx_gemm16_tile128<BF, 1, BCOL, 2>), dim3(tiles_m * tiles_n), dim3(256), 0, s, (const uint8_t*)a, (const uint8_t*)b,
                         c, (const int*)nullptr, (const MoeTile*)nullptr, (const int32_t*)nullptr, (int)M, (int)K, (int)N, tiles_m, tiles_n, 1,
                         d);
    return;
  }
  const int nkt = (int)(K / MOE_BK);
  d.kt_per_split = (nkt + splits - 1) / splits;
  d.ldc = partial ? N : ldc;
  if (tile == 256)
    hx_launch((hx_gemm16_tile256<BF, 2, BCOL>), dim3(tiles_m * tiles_n, splits), dim3(256), 0, s, (const uint8_t*)a,
                       (const uint8_t*)b, partial ? ws : c, (const int*)nullptr, (const MoeTile*)nullptr, (const int32_t*)nullptr, (int)M,
                       (int)K, (int)N, tiles_m, tiles_n, 1, d);
  else if ((long)tiles_m * tiles_n * splits <= 256)
    hx_launch((hx_gemm16_tile128<BF, 2, BCOL, 4>), dim3(tiles_m * tiles_n, splits), dim3(256), 0, s, (const uint8_t*)a,
                       (const uint8_t*)b, partial ? ws : c, (const int*)nullptr, (const MoeTile*)nullptr, (const int32_t*)nullptr, (int)M,
                       (int)K, (int)N, tiles_m, tiles_n, 1, d);
  else
    hx_launch((hx_gemm16_tile128<BF, 2, BCOL, 2>), dim3(tiles_m * tiles_n, splits), dim3(256), 0, s, (const uint8_t*)a,
                       (const uint8_t*)b, partial ? ws : c, (const int*)nullptr, (const MoeTile*)nullptr, (const int32_t*)nullptr, (int)M,
                       (int)K, (int)N, tiles_m, tiles_n, 1, d);
  if (!partial) return;
  const long groups = M * (N / 4);
  const dim3 grid((unsigned)((groups + 15) / 16));
  if (out_dtype == HX_F32)
    hx_launch((hx_matmul16_reduce<T16, float>), grid, dim3(256), 0, s, (const float*)ws, splits, (int)M, (int)N, (float*)c, (long)ldc,
                       bias, bias_f32, relu);
  else
    hx_launch((hx_matmul16_reduce<T16, T16>), grid, dim3(256), 0, s, (const float*)ws, splits, (int)M, (int)N, (T16*)c, (long)ldc,
                       bias, bias_f32, relu);
}

extern "C" int hx_matmul_path(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc, int in_dtype,
                              const void* a, const void* b, const void* c, const void* bias) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  if (!mm_fast_ok(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, bias, in_dtype)) return 0;
  // 2: the persistent form of the 256x256 kernel (for a call without epilogue, a 16-bit output and the library's own split)
  const MmPlan plan = mm_plan(M, N, K, 0);
  return mm_persistent_ok(M, N, K, ldb_n, bias, 0, in_dtype, plan.tile, plan.splits) ? 2 : 1;
}

extern "C" int hx_matmul(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                         int64_t ldb_n, int64_t ldc, const void* bias, int bias_dtype, int relu, int in_dtype, int out_dtype, int split_k,
                         void* workspace, size_t workspace_bytes, void* stream) {
  if (M < 0 || N < 0 || K < 0) {
    hx_set_error("hx_matmul: negative size");
    return HX_ERR_BAD_ARG;
  }
  if (in_dtype != HX_BF16 && in_dtype != HX_F16 && in_dtype != HX_F32) {
    hx_set_error("hx_matmul: operand dtype must be HX_BF16, HX_F16 or HX_F32, got %d", in_dtype);
    return HX_ERR_BAD_ARG;
  }
  if (out_dtype != in_dtype && out_dtype != HX_F32) {
    hx_set_error("hx_matmul: output dtype must be the operand dtype or HX_F32, got %d", out_dtype);
    return HX_ERR_BAD_ARG;
  }
  if (bias && bias_dtype != in_dtype && bias_dtype != HX_F32) {
    hx_set_error("hx_matmul: bias dtype must be the operand dtype or HX_F32, got %d", bias_dtype);
    return HX_ERR_BAD_ARG;
  }
  if (M == 0 || N == 0) return 0;
  if (!c || (K > 0 && (!a || !b))) {
    hx_set_error("hx_matmul: null pointer");
    return HX_ERR_BAD_ARG;
  }
  if (M >= (1LL << 31) || N >= (1LL << 31) || K >= (1LL << 31) || N > 65535LL * 64) {
    hx_set_error("hx_matmul: dimension too large");
    return HX_ERR_UNSUPPORTED;
  }
  if (lda < K || ldc < N) {
    hx_set_error("hx_matmul: lda (%lld) < K or ldc (%lld) < N", (long long)lda, (long long)ldc);
    return HX_ERR_BAD_ARG;
  }
  hipStream_t s = (hipStream_t)stream;
  const int bias_f32 = (bias_dtype == HX_F32 || in_dtype == HX_F32) ? 1 : 0;
  bool fast = mm_fast_ok(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, bias, in_dtype);
  if (fast) {
    const MmPlan plan = mm_plan(M, N, K, split_k);
    int splits = plan.splits;
    const bool partial = splits > 1 || (out_dtype == HX_F32 && (bias || relu));
    const size_t need = partial ? (size_t)splits * M * N * 4 : 0;
    if (need && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15))) {
      if (split_k > 1 || out_dtype == HX_F32) {
        hx_set_error("hx_matmul: workspace must be 16-byte aligned and at least %zu bytes (got %zu)", need, workspace_bytes);
        return HX_ERR_WORKSPACE;
      }
      splits = 1;  // automatic split without room for it: one pass
    }
    const bool bcol = ldb_n != 1;  // column-major B: its leading dimension is ldb_n
    const int64_t ldb = bcol ? ldb_n : ldb_k;
    if (in_dtype == HX_BF16) {
      if (bcol) mm_launch_fast<true, true>(a, b, c, M, N, K, lda, ldb, ldc, bias, bias_f32, relu, out_dtype, plan.tile, splits, workspace, s);
      else mm_launch_fast<true, false>(a, b, c, M, N, K, lda, ldb, ldc, bias, bias_f32, relu, out_dtype, plan.tile, splits, workspace, s);
    } else {
      if (bcol) mm_launch_fast<false, true>(a, b, c, M, N, K, lda, ldb, ldc, bias, bias_f32, relu, out_dtype, plan.tile, splits, workspace, s);
      else mm_launch_fast<false, false>(a, b, c, M, N, K, lda, ldb, ldc, bias, bias_f32, relu, out_dtype, plan.tile, splits, workspace, s);
    }
  } else if (in_dtype == HX_F32) {
    mm_launch_general<float, float>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, bias, 1, relu, s);
  } else if (in_dtype == HX_BF16) {
    if (out_dtype == HX_F32) mm_launch_general<__bf16, float>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, bias, bias_f32, relu, s);
    else mm_launch_general<__bf16, __bf16>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, bias, bias_f32, relu, s);
  } else {
    if (out_dtype == HX_F32) mm_launch_general<_Float16, float>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, bias, bias_f32, relu, s);
    else mm_launch_general<_Float16, _Float16>(a, b, c, M, N, K, lda, ldb_k, ldb_n, ldc, bias, bias_f32, relu, s);
  }
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_matmul: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}
