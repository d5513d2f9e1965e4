// Casts and per-tensor quantisation to OCP e4m3fn for gfx950 — the step in front of the FP8 kernels:
//   * hx_cast_e4m3 / hx_fp8_attention_preprocess: `x.to(torch.float8_e4m3fn)` for fp16 / bf16 / fp32 inputs, as
//     preprocess_fp8_attention_inputs does three times (examples/fp8_attention.py:110-133 of the reference); V needs no
//     transposing copy because the attention kernel reads the [S][D] memory order that function leaves it in.
//   * hx_fp8_quantize: amax -> scale -> cast, producing the (tensor, scale) pair that the scaled GEMM consumes
//     (the reference's baseline call hard-codes unit scales, examples/fp8_gemm.py:74-78):
//         amax = max|x|;  scale = amax / 448  (1 if amax == 0);  q = e4m3(x * (448 / amax))
// All of it is streaming, HBM-bound work: 16 elements per lane per step, whole-line loads and 16-byte stores,
// round-to-nearest-even in hardware (v_cvt_pk_fp8_f32: |v| <= 464 rounds to at most 448, larger or NaN gives NaN,
// which is what torch's cast does).
#include "hx_common.h"

#define QZ_THREADS 256
#define QZ_EPT 16  // elements per thread per step

template <int DT>
struct QzIn;
template <>
struct QzIn<HX_F16> {
  typedef _Float16 T;
};
template <>
struct QzIn<HX_BF16> {
  typedef __bf16 T;
};
template <>
struct QzIn<HX_F32> {
  typedef float T;
};

// 16 consecutive elements -> fp32
template <typename T>
__device__ __forceinline__ void qz_load16(const T* __restrict__ p, float (&f)[QZ_EPT]) {
  constexpr int NV = (int)(QZ_EPT * sizeof(T) / 16);  // 16-byte loads
  v4i raw[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) raw[i] = ((const v4i*)p)[i];
  const T* e = (const T*)raw;
#pragma unroll
  for (int i = 0; i < QZ_EPT; ++i) f[i] = (float)e[i];
}

__device__ __forceinline__ v4i qz_pack16(const float (&f)[QZ_EPT], float mul) {
  v4i out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int dw = HX_CVT_PK_E4M3(f[4 * i] * mul, f[4 * i + 1] * mul, 0, false);
    out[i] = HX_CVT_PK_E4M3(f[4 * i + 2] * mul, f[4 * i + 3] * mul, dw, true);
  }
  return out;
}

// dst[i] = e4m3(src[i] * mul), mul = *mul_ptr or 1.  Up to three (src, dst, n) jobs in one launch (blockIdx.y).
struct QzJobs {
  const void* src[3];
  void* dst[3];
  long long n[3];
};

template <int DT>
__global__ __launch_bounds__(QZ_THREADS) void hx_cast_e4m3_kernel(QzJobs jobs, const float* __restrict__ mul_ptr) {
  typedef typename QzIn<DT>::T T;
  const T* __restrict__ src = (const T*)jobs.src[blockIdx.y];
  uint8_t* __restrict__ dst = (uint8_t*)jobs.dst[blockIdx.y];
  const long long n = jobs.n[blockIdx.y];
  const float mul = mul_ptr ? *mul_ptr : 1.f;
  const long long nvec = n / QZ_EPT;
  const long long stride = (long long)gridDim.x * QZ_THREADS;
  for (long long v = (long long)blockIdx.x * QZ_THREADS + threadIdx.x; v < nvec; v += stride) {
    float f[QZ_EPT];
    qz_load16(src + v * QZ_EPT, f);
    // non-temporal store: the codes are written once and not read here (the three C4-sized casts -3 %); the loads stay
    // plain, so the second read of a quantisation still finds what the amax pass left in the caches
    __builtin_nontemporal_store(qz_pack16(f, mul), (v4i*)dst + v);
  }
  // ragged tail (fewer than 16 elements) by the first threads of block 0
  if (blockIdx.x == 0) {
    const long long i = nvec * QZ_EPT + threadIdx.x;
    if (i < n) {
      const int dw = HX_CVT_PK_E4M3((float)src[i] * mul, 0.f, 0, false);
      dst[i] = (uint8_t)(dw & 0xff);
    }
  }
}

// per-block max|x| -> partial[blockIdx.x]
template <int DT>
__global__ __launch_bounds__(QZ_THREADS) void hx_amax_partial_kernel(const void* __restrict__ src_, long long n, float* __restrict__ partial) {
  typedef typename QzIn<DT>::T T;
  const T* __restrict__ src = (const T*)src_;
  float m = 0.f;
  bool bad = false;  // NaN anywhere makes the amax NaN, as torch's amax does
  const long long nvec = n / QZ_EPT;
  const long long stride = (long long)gridDim.x * QZ_THREADS;
  for (long long v = (long long)blockIdx.x * QZ_THREADS + threadIdx.x; v < nvec; v += stride) {
    float f[QZ_EPT];
    qz_load16(src + v * QZ_EPT, f);
#pragma unroll
    for (int i = 0; i < QZ_EPT; ++i) {
      bad |= f[i] != f[i];
      m = fmaxf(m, fabsf(f[i]));
    }
  }
  if (blockIdx.x == 0) {
    const long long i = nvec * QZ_EPT + threadIdx.x;
    if (i < n) {
      const float x = (float)src[i];
      bad |= x != x;
      m = fmaxf(m, fabsf(x));
    }
  }
  if (bad) m = __builtin_nanf("");
  __shared__ float red[QZ_THREADS / 64];
  // NaN-propagating max across the block
  auto nmax = [](float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); };
  for (int off = 32; off > 0; off >>= 1) m = nmax(m, __shfl_xor(m, off));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = red[0];
    for (int i = 1; i < QZ_THREADS / 64; ++i) r = nmax(r, red[i]);
    partial[blockIdx.x] = r;
  }
}

// partial[0..np) -> *scale_out = amax / 448 (1 if amax == 0), out[1] = 448 / amax (1 if amax == 0), out[2] = amax
__global__ __launch_bounds__(QZ_THREADS) void hx_amax_final_kernel(const float* __restrict__ partial, int np, float* __restrict__ out,
                                                                  float* __restrict__ scale_out) {
  auto nmax = [](float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); };
  float m = 0.f;
  for (int i = threadIdx.x; i < np; i += QZ_THREADS) m = nmax(m, partial[i]);
  __shared__ float red[QZ_THREADS / 64];
  for (int off = 32; off > 0; off >>= 1) m = nmax(m, __shfl_xor(m, off));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = red[0];
    for (int i = 1; i < QZ_THREADS / 64; ++i) r = nmax(r, red[i]);
    const bool zero = r == 0.f;
    *scale_out = zero ? 1.f : r / 448.f;
    out[1] = zero ? 1.f : 448.f / r;
    out[2] = r;
  }
}

static int qz_grid(long long n) {
  const int cus = hx_cu_count();
  const long long need = (n / QZ_EPT + QZ_THREADS - 1) / QZ_THREADS;
  const long long cap = (long long)cus * 8;
  return (int)(need < 1 ? 1 : (need < cap ? need : cap));
}

static int qz_launch_cast(const QzJobs& jobs, int njobs, long long nmax_, int dt, const float* mul, hipStream_t s) {
  dim3 grid((unsigned)qz_grid(nmax_), (unsigned)njobs);
  if (dt == HX_F16) hx_launch(hx_cast_e4m3_kernel<HX_F16>, grid, dim3(QZ_THREADS), 0, s, jobs, mul);
  else if (dt == HX_BF16) hx_launch(hx_cast_e4m3_kernel<HX_BF16>, grid, dim3(QZ_THREADS), 0, s, jobs, mul);
  else hx_launch(hx_cast_e4m3_kernel<HX_F32>, grid, dim3(QZ_THREADS), 0, s, jobs, mul);
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("fp8 cast: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

static int qz_check(const char* who, const void* src, const void* dst, int64_t n, int dt) {
  if (n < 0) {
    hx_set_error("%s: negative size", who);
    return HX_ERR_BAD_ARG;
  }
  if (dt != HX_F16 && dt != HX_BF16 && dt != HX_F32) {
    hx_set_error("%s: source dtype must be HX_F16, HX_BF16 or HX_F32, got %d", who, dt);
    return HX_ERR_BAD_ARG;
  }
  if (n > 0 && (!src || !dst)) {
    hx_set_error("%s: null pointer", who);
    return HX_ERR_BAD_ARG;
  }
  if ((((uintptr_t)src | (uintptr_t)dst) & 15) != 0) {
    hx_set_error("%s: pointers must be 16-byte aligned", who);
    return HX_ERR_UNSUPPORTED;
  }
  return 0;
}

extern "C" int hx_cast_e4m3(const void* src, void* dst, int64_t n, int src_dtype, const float* multiplier, void* stream) {
  int rc = qz_check("hx_cast_e4m3", src, dst, n, src_dtype);
  if (rc != 0 || n == 0) return rc;
  QzJobs jobs = {{src, nullptr, nullptr}, {dst, nullptr, nullptr}, {n, 0, 0}};
  return qz_launch_cast(jobs, 1, n, src_dtype, multiplier, (hipStream_t)stream);
}

extern "C" int hx_fp8_attention_preprocess(const void* q, const void* k, const void* v, void* q8, void* k8, void* v8, int64_t n,
                                           int src_dtype, void* stream) {
  int rc = qz_check("hx_fp8_attention_preprocess", q, q8, n, src_dtype);
  if (rc == 0) rc = qz_check("hx_fp8_attention_preprocess", k, k8, n, src_dtype);
  if (rc == 0) rc = qz_check("hx_fp8_attention_preprocess", v, v8, n, src_dtype);
  if (rc != 0 || n == 0) return rc;
  QzJobs jobs = {{q, k, v}, {q8, k8, v8}, {n, n, n}};
  return qz_launch_cast(jobs, 3, n, src_dtype, nullptr, (hipStream_t)stream);
}

extern "C" size_t hx_fp8_quantize_workspace_bytes(int64_t n) {
  if (n < 0) return 0;
  return (size_t)qz_grid(n) * sizeof(float) + 16;
}

extern "C" int hx_fp8_quantize(const void* src, void* dst, int64_t n, int src_dtype, float* scale_out, void* workspace,
                               size_t workspace_bytes, void* stream) {
  int rc = qz_check("hx_fp8_quantize", src, dst, n, src_dtype);
  if (rc != 0) return rc;
  if (!scale_out) {
    hx_set_error("hx_fp8_quantize: null scale_out");
    return HX_ERR_BAD_ARG;
  }
  if (!workspace || workspace_bytes < hx_fp8_quantize_workspace_bytes(n) || ((uintptr_t)workspace & 15)) {
    hx_set_error("hx_fp8_quantize: workspace must be 16-byte aligned and at least %zu bytes (got %zu)",
                 hx_fp8_quantize_workspace_bytes(n), workspace_bytes);
    return HX_ERR_WORKSPACE;
  }
  hipStream_t s = (hipStream_t)stream;
  // workspace: [0] unused | [1] 448/amax | [2] amax | [3] pad | partial maxima
  float* triple = (float*)workspace;
  float* partial = triple + 4;
  const int blocks = qz_grid(n);
  if (src_dtype == HX_F16) hx_launch(hx_amax_partial_kernel<HX_F16>, dim3(blocks), dim3(QZ_THREADS), 0, s, src, (long long)n, partial);
  else if (src_dtype == HX_BF16) hx_launch(hx_amax_partial_kernel<HX_BF16>, dim3(blocks), dim3(QZ_THREADS), 0, s, src, (long long)n, partial);
  else hx_launch(hx_amax_partial_kernel<HX_F32>, dim3(blocks), dim3(QZ_THREADS), 0, s, src, (long long)n, partial);
  hx_launch(hx_amax_final_kernel, dim3(1), dim3(QZ_THREADS), 0, s, (const float*)partial, blocks, triple, scale_out);
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_fp8_quantize: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  if (n > 0) {
    QzJobs jobs = {{src, nullptr, nullptr}, {dst, nullptr, nullptr}, {n, 0, 0}};
    rc = qz_launch_cast(jobs, 1, n, src_dtype, triple + 1, s);
    if (rc != 0) return rc;
  }
  return 0;
}
