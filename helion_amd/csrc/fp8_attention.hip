// FP8 (e4m3fn) attention for gfx950 — device side of examples/fp8_attention.py:22-106 of the reference.
//   per (batch*head):  s = (q k^T) * c,  c = fp32(1/sqrt(D) * 1.44269504)
//                      p = exp2(s - m),  l = sum(p) (un-quantised),  o = (e4m3(p) v) / l
// exact_max: two passes over the keys — pass 1 finds the exact row max m (what the reference's
// single-tile ref-eager execution uses), pass 2 quantises p against it.  Otherwise one pass with
// the running max (online softmax; what the reference's compiled kernel does).
//
// Work decomposition: workgroup = 4 waves = 128 queries of one head; wave = 32 queries.
// Per 64-key tile a wave computes S^T = K Q^T as two 32x32 blocks (32x32x64 fp8 MFMA, D/64 k-steps),
// so lane (q = lane%32, G = lane/32) ends up holding 16 *consecutive* keys of query q per block (the
// K rows are fed to the MFMA in the permuted order key(i) = 16*((i>>2)&1) + 4*(i>>3) + (i&3)).
// Those 2x16 values, converted to e4m3, are exactly the B operand of the P.V MFMA
// (O^T[d][q] += V^T[d][key] P^T[key][q]) with k-slots 0..15 = keys 16G..16G+15 of block 0 and
// 16..31 = the same keys of block 1; the V^T operand reads the matching two 16-byte chunks.
// Row max / row sum need no cross-lane traffic inside the key loop: each lane reduces its own
// values and the two lanes of a query are combined once (exact_max) or once per tile (online).
#include "hx_common.h"

#define ATT_BN 64      // keys per tile
#define ATT_WAVES 4
#define ATT_BM (32 * ATT_WAVES)

// K tile: [64 keys][D bytes]; V tile: [D rows][64 bytes].  Rows are 16-byte chunks, swizzled:
//   row bytes 128: pos = chunk ^ ((row >> 1) & 7);   row bytes 64: pos = chunk ^ ((row >> 2) & 3)
template <int RB>
__device__ __forceinline__ int att_swz(int row) {
  return RB == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}

template <int D, int OUT, bool EXACT>
__global__ __launch_bounds__(256, 2) void hx_fp8_attention_kernel(const uint8_t* __restrict__ Q, const uint8_t* __restrict__ Kt,
                                                                  const uint8_t* __restrict__ Vt, void* __restrict__ Out, int S,
                                                                  int BH, int qtiles) {
  constexpr int KSTEPS = D / 64;  // MFMA k-steps for S = K Q^T
  constexpr int DB = D / 32;      // 32-row blocks of O^T
  constexpr int KROWS_PER_DMA = 1024 / D;
  constexpr int K_DMAS = ATT_BN / KROWS_PER_DMA;  // per tile
  constexpr int V_DMAS = D / 16;                  // 16 rows of 64 B per DMA
  __shared__ __attribute__((aligned(1024))) uint8_t sK0[ATT_BN * D];
  __shared__ __attribute__((aligned(1024))) uint8_t sK1[ATT_BN * D];
  __shared__ __attribute__((aligned(1024))) uint8_t sV0[D * ATT_BN];
  __shared__ __attribute__((aligned(1024))) uint8_t sV1[D * ATT_BN];

  // workgroup -> (head, query tile): XCD x (= id%8) takes heads x, x+8, ...; the query tiles of a head
  // are consecutive on that XCD so its K/V stay in that XCD's L2.
  int bh, qt;
  {
    const int id = blockIdx.x, xcd = id & 7, loc = id >> 3;
    const int hpx = (BH + 7) >> 3;  // heads per xcd (upper bound)
    const int hl = loc / qtiles;
    qt = loc % qtiles;
    bh = xcd + 8 * hl;
    if (hl >= hpx || bh >= BH) return;  // whole workgroup exits together
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q31 = lane & 31, G = lane >> 5;
  const int q0 = qt * ATT_BM + w * 32;
  const bool active = q0 < S;  // wave-uniform; inactive waves still help with DMA and barriers

  const uint8_t* Qh = Q + (long)bh * S * D;
  const uint8_t* Kh = Kt + (long)bh * S * D;
  const uint8_t* Vh = Vt + (long)bh * D * S;

  // ---- Q fragments (B operand of S^T): lane (q, G): Q[q][64t + 32G .. +31]
  v8i qf[KSTEPS];
  {
    const int qrow = min(q0 + q31, S - 1);
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) {
      const v4i* p = (const v4i*)(Qh + (long)qrow * D + 64 * t + 32 * G);
      v4i lo = p[0], hi = p[1];
      qf[t] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  }

  // ---- DMA addressing.  K: one instruction = KROWS_PER_DMA rows of D bytes.
  constexpr int KCPR = D / 16;  // chunks per K row
  const int k_lrow = lane / KCPR, k_lpos = lane % KCPR;
  auto issue_k = [&](int tile, uint8_t* sk) {
#pragma unroll
    for (int j = w; j < K_DMAS; j += ATT_WAVES) {
      const int row = j * KROWS_PER_DMA + k_lrow;
      const int chunk = k_lpos ^ att_swz<D>(row);
      hx_g2l16(Kh + (long)(tile * ATT_BN + row) * D + chunk * 16, sk + j * 1024);
    }
  };
  const int v_lrow = lane >> 2, v_lpos = lane & 3;
  auto issue_v = [&](int tile, uint8_t* sv) {
#pragma unroll
    for (int j = w; j < V_DMAS; j += ATT_WAVES) {
      const int row = j * 16 + v_lrow;
      const int chunk = v_lpos ^ att_swz<64>(row);
      hx_g2l16(Vh + (long)row * S + tile * ATT_BN + chunk * 16, sv + j * 1024);
    }
  };

  // ---- MFMA operand addressing
  // K operand (A of S^T): MFMA row i = lane%32 is key(i) within the 32-key block
  const int krow = 16 * ((q31 >> 2) & 1) + 4 * (q31 >> 3) + (q31 & 3);
  int k_off[2][KSTEPS][2];  // [block][t][half] byte offsets in the K tile
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = kb * 32 + krow;
        k_off[kb][t][h] = row * D + (((4 * t + 2 * G + h) ^ att_swz<D>(row)) * 16);
      }
  int v_off[2];  // [block] byte offsets in the V tile for d-row lane%32 (add db*32*64)
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) v_off[kb] = q31 * 64 + (((2 * kb + G) ^ att_swz<64>(q31)) * 16);

  const float c = (float)((1.0 / __builtin_sqrt((double)D)) * 1.44269504);
  const int ntiles = S / ATT_BN;

  auto scores = [&](const uint8_t* sk, v16f (&s)[2]) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
#pragma unroll
      for (int t = 0; t < KSTEPS; ++t) {
        v4i lo = *(const v4i*)(sk + k_off[kb][t][0]);
        v4i hi = *(const v4i*)(sk + k_off[kb][t][1]);
        v8i kf = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        s[kb] = hx_mfma_32x32x64_e4m3(kf, qf[t], s[kb]);
      }
    }
  };

  float m_run = -__builtin_inff();  // scaled-domain row max

  if (EXACT) {
    // ---------------- pass 1: exact row max of the raw scores
    float smax = -__builtin_inff();
    issue_k(0, sK0);
    for (int j = 0; j < ntiles; j += 2) {
      HX_WAIT_VM0();
      __syncthreads();
      if (j + 1 < ntiles) issue_k(j + 1, sK1);
      if (active) {
        v16f s[2];
        scores(sK0, s);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) smax = fmaxf(smax, s[kb][r]);
      }
      if (j + 1 < ntiles) {
        HX_WAIT_VM0();
        __syncthreads();
        if (j + 2 < ntiles) issue_k(j + 2, sK0);
        if (active) {
          v16f s[2];
          scores(sK1, s);
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) smax = fmaxf(smax, s[kb][r]);
        }
      }
    }
    smax = fmaxf(smax, __shfl_xor(smax, 32));
    m_run = smax * c;  // max(s*c) == max(s)*c for c > 0 (rounding is monotone)
    __syncthreads();   // all waves done with sK0/sK1 before pass 2 overwrites them
  }

  // ---------------- pass 2 (or the only pass)
  v16f o[DB];
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[d][r] = 0.f;
  float l_lane = 0.f;

  auto tile_step = [&](const uint8_t* sk, const uint8_t* sv) {
    v16f s[2];
    scores(sk, s);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kb][r] = __fmul_rn(s[kb][r], c);
    if (!EXACT) {
      float tmax = s[0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s[kb][r]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
      const float m_new = fmaxf(m_run, tmax);
      const float alpha = __builtin_amdgcn_exp2f(__fsub_rn(m_run, m_new));
      l_lane *= alpha;
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
      m_run = m_new;
    }
    v8i pf;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[r] = __builtin_amdgcn_exp2f(__fsub_rn(s[kb][r], m_run));
        l_lane += p[r];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int dw = HX_CVT_PK_E4M3(p[4 * j], p[4 * j + 1], 0, false);
        dw = HX_CVT_PK_E4M3(p[4 * j + 2], p[4 * j + 3], dw, true);
        pf[kb * 4 + j] = dw;
      }
    }
#pragma unroll
    for (int d = 0; d < DB; ++d) {
      v4i lo = *(const v4i*)(sv + d * 32 * 64 + v_off[0]);
      v4i hi = *(const v4i*)(sv + d * 32 * 64 + v_off[1]);
      v8i vf = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      o[d] = hx_mfma_32x32x64_e4m3(vf, pf, o[d]);
    }
  };

  issue_k(0, sK0);
  issue_v(0, sV0);
  for (int j = 0; j < ntiles; j += 2) {
    HX_WAIT_VM0();
    __syncthreads();
    if (j + 1 < ntiles) {
      issue_k(j + 1, sK1);
      issue_v(j + 1, sV1);
    }
    if (active) tile_step(sK0, sV0);
    if (j + 1 < ntiles) {
      HX_WAIT_VM0();
      __syncthreads();
      if (j + 2 < ntiles) {
        issue_k(j + 2, sK0);
        issue_v(j + 2, sV0);
      }
      if (active) tile_step(sK1, sV1);
    }
  }

  if (!active) return;
  // ---------------- epilogue: o[db][4a+b] is O[q0 + lane%32][32 db + 8a + 4G + b]
  const float l = l_lane + __shfl_xor(l_lane, 32);
  const int qrow = q0 + q31;
  if (qrow >= S) return;
  if (OUT == HX_F32) {
    float* orow = (float*)Out + ((long)bh * S + qrow) * D + 4 * G;
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        v4f v;
#pragma unroll
        for (int b = 0; b < 4; ++b) v[b] = o[d][4 * a + b] / l;
        *(v4f*)(orow + d * 32 + 8 * a) = v;
      }
  } else {
    uint8_t* orow = (uint8_t*)Out + ((long)bh * S + qrow) * D + 4 * G;
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        int dw = HX_CVT_PK_E4M3(o[d][4 * a] / l, o[d][4 * a + 1] / l, 0, false);
        dw = HX_CVT_PK_E4M3(o[d][4 * a + 2] / l, o[d][4 * a + 3] / l, dw, true);
        *(int*)(orow + d * 32 + 8 * a) = dw;
      }
  }
}

template <int D, int OUT>
static int launch_att(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, int exact, hipStream_t s) {
  const int qtiles = (int)((S + ATT_BM - 1) / ATT_BM);
  const int hpx = (int)((BH + 7) / 8);
  const int grid = 8 * hpx * qtiles;
  if (exact)
    hipLaunchKernelGGL((hx_fp8_attention_kernel<D, OUT, true>), dim3(grid), dim3(256), 0, s, (const uint8_t*)q, (const uint8_t*)k,
                       (const uint8_t*)v, out, (int)S, (int)BH, qtiles);
  else
    hipLaunchKernelGGL((hx_fp8_attention_kernel<D, OUT, false>), dim3(grid), dim3(256), 0, s, (const uint8_t*)q, (const uint8_t*)k,
                       (const uint8_t*)v, out, (int)S, (int)BH, qtiles);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    hx_set_error("hx_fp8_attention: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

extern "C" int hx_fp8_attention(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, int64_t D,
                                int out_dtype, int exact_max, void* stream) {
  if (BH < 0 || S < 0 || D < 0) {
    hx_set_error("hx_fp8_attention: negative size");
    return HX_ERR_BAD_ARG;
  }
  if (BH == 0 || S == 0) return 0;
  if (!q || !k || !v || !out) {
    hx_set_error("hx_fp8_attention: null pointer");
    return HX_ERR_BAD_ARG;
  }
  if (out_dtype != HX_F32 && out_dtype != HX_E4M3) {
    hx_set_error("hx_fp8_attention: out_dtype must be HX_E4M3 or HX_F32, got %d", out_dtype);
    return HX_ERR_BAD_ARG;
  }
  if ((D != 64 && D != 128) || (S % ATT_BN) != 0) {
    hx_set_error("hx_fp8_attention: unsupported shape S=%lld D=%lld (need D in {64,128}, S %% 64 == 0)", (long long)S,
                 (long long)D);
    return HX_ERR_UNSUPPORTED;
  }
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) {
    hx_set_error("hx_fp8_attention: pointers must be 16-byte aligned");
    return HX_ERR_UNSUPPORTED;
  }
  if (BH * S * D >= (1LL << 40)) {
    hx_set_error("hx_fp8_attention: problem too large");
    return HX_ERR_UNSUPPORTED;
  }
  hipStream_t s = (hipStream_t)stream;
  if (D == 128) {
    if (out_dtype == HX_F32) return launch_att<128, HX_F32>(q, k, v, out, BH, S, exact_max, s);
    return launch_att<128, HX_E4M3>(q, k, v, out, BH, S, exact_max, s);
  }
  if (out_dtype == HX_F32) return launch_att<64, HX_F32>(q, k, v, out, BH, S, exact_max, s);
  return launch_att<64, HX_E4M3>(q, k, v, out, BH, S, exact_max, s);
}
