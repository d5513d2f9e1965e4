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
//
// V comes in either of two physical layouts per head: [D][S] (VSD = false; "pre-transposed" and contiguous) or
// [S][D] (VSD = true; what examples/fp8_attention.py:110-133 really hands over: `v.permute(0,1,3,2).to(e4m3)`
// keeps the memory order of the [B,H,S,D] source and only the strides say [D,S]).  In the second case a V tile
// sits in LDS like a K tile, rows = keys, and the V^T operand is formed by transposing LDS reads
// (ds_read_b64_tr_b8: 8 keys x 16 columns per 16 lanes), so neither layout needs a copy.
#include "hx_common.h"

#include <cmath>

#define ATT_BN 64      // keys per tile
#define ATT_WAVES 4
#define ATT_BM (32 * ATT_WAVES)
#define ATT_NS 4       // LDS stages: tiles j .. j+2 are in flight while tile j is consumed
#define ATT_LEAD (ATT_NS - 1)

// K tile: [64 keys][D bytes]; V tile: [D rows][64 bytes].  Rows are 16-byte chunks, swizzled:
//   row bytes 128: pos = chunk ^ ((row >> 1) & 7);   row bytes 64: pos = chunk ^ ((row >> 2) & 3)
template <int RB>
__device__ __forceinline__ int att_swz(int row) {
  return RB == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}
// V tile in the [keys][D bytes] layout: one transposing read has 32 lanes fetch 8 consecutive key rows x two
// adjacent 16-byte chunks; the swizzle has to spread those over all banks and must leave bit 0 (which chunk of
// the pair) alone.  RB = 128: rows r, r+1 share a 256-byte bank window -> (r>>1)&3 into bits 2:1;  RB = 64: rows
// r, r+4 share a 64-byte quarter of it -> (r>>2)&1 into bit 1.
template <int RB>
__device__ __forceinline__ int att_vswz(int row) {
  return RB == 128 ? (((row >> 1) & 3) << 1) : (((row >> 2) & 1) << 1);
}

// wait until at most `newer` tiles' worth of this wave's DMA instructions (IPT per tile) are outstanding
template <int IPT>
__device__ __forceinline__ void att_wait_tiles(int newer) {
  if (newer >= 2) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(2 * IPT));
  else if (newer == 1) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(IPT));
  else __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(0));
}

template <int D, int OUT, bool EXACT, bool VSD>
__global__ __launch_bounds__(256, 2) void hx_fp8_attention_kernel(const uint8_t* __restrict__ Q, const uint8_t* __restrict__ Kt,
                                                                  const uint8_t* __restrict__ Vt, void* __restrict__ Out, int S,
                                                                  int BH, int qtiles, float c) {
  constexpr int KSTEPS = D / 64;  // MFMA k-steps for S = K Q^T
  constexpr int DB = D / 32;      // 32-row blocks of O^T
  constexpr int KROWS_PER_DMA = 1024 / D;
  constexpr int KPW = (ATT_BN / KROWS_PER_DMA) / ATT_WAVES;  // K DMA instructions per wave per tile
  constexpr int VPW = VSD ? KPW : (D / 16) / ATT_WAVES;      // V DMA instructions per wave per tile ([D][S]: 16 rows x 64 B each)
  constexpr int TILE = ATT_BN * D;                           // bytes of a K tile == bytes of a V tile
  __shared__ __attribute__((aligned(1024))) uint8_t smem[ATT_NS][2][TILE];

  // workgroup -> (head, query tile): XCD x (= id%8) takes heads x, x+8, ...; the query tiles of a head
  // are consecutive on that XCD so its K/V stay in that XCD's L2.
  int bh, qt;
  {
    const int id = blockIdx.x, xcd = id & 7, loc = id >> 3;
    const int hl = loc / qtiles;
    qt = loc % qtiles;
    bh = xcd + 8 * hl;
    if (bh >= BH) return;  // whole workgroup exits together
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q31 = lane & 31, G = lane >> 5;
  const int q0 = qt * ATT_BM + w * 32;
  const bool active = q0 < S;  // wave-uniform; inactive waves still help with DMA and barriers

  const uint8_t* Qh = Q + (long)bh * S * D;
  const uint8_t* Kh = Kt + (long)bh * S * D;
  const uint8_t* Vh = Vt + (long)bh * D * S;  // either layout: D*S bytes per head

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

  // ---- DMA addressing: wave w issues K instructions j = w, w+4, ... (KROWS_PER_DMA rows of D bytes each) and
  // V instructions j = w, w+4, ... (16 rows of 64 bytes each).  The swizzle of a lane's row does not depend on
  // which of the wave's instructions it is, so one per-lane offset serves all of them.
  constexpr int KCPR = D / 16;  // chunks per K row
  const int k_lrow = lane / KCPR, k_lpos = lane % KCPR;
  const uint32_t k_vo = (uint32_t)(k_lrow * D + ((k_lpos ^ att_swz<D>(w * KROWS_PER_DMA + k_lrow)) * 16));
  const int v_lrow = lane >> 2, v_lpos = lane & 3;
  const uint32_t v_vo = VSD ? (uint32_t)(k_lrow * D + ((k_lpos ^ att_vswz<D>(w * KROWS_PER_DMA + k_lrow)) * 16))
                            : (uint32_t)(v_lrow * S + ((v_lpos ^ att_swz<64>(v_lrow)) * 16));
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]);
  auto issue_k = [&](int tile, int stage) {
#pragma unroll
    for (int jj = 0; jj < KPW; ++jj) {
      const int j = w + ATT_WAVES * jj;
      hx_g2l16_s(Kh + ((long)tile * ATT_BN + j * KROWS_PER_DMA) * D, k_vo, lds0 + (uint32_t)stage * 2 * TILE + j * 1024);
    }
  };
  auto issue_v = [&](int tile, int stage) {
#pragma unroll
    for (int jj = 0; jj < VPW; ++jj) {
      const int j = w + ATT_WAVES * jj;
      if (VSD) hx_g2l16_s(Vh + ((long)tile * ATT_BN + j * KROWS_PER_DMA) * D, v_vo, lds0 + (uint32_t)stage * 2 * TILE + TILE + j * 1024);
      else hx_g2l16_s(Vh + (long)(j * 16) * S + (long)tile * ATT_BN, v_vo, lds0 + (uint32_t)stage * 2 * TILE + TILE + j * 1024);
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
  int v_off[2];  // [D][S] layout: [block] byte offsets in the V tile for d-row lane%32 (add db*32*64)
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) v_off[kb] = q31 * 64 + (((2 * kb + G) ^ att_swz<64>(q31)) * 16);
  // [S][D] layout: transposing read j (0..3) of a 32-row block of V^T fetches keys kr0..kr0+7,
  // kr0 = 32*(j>>1) + 16*G + 8*(j&1); this lane supplies 8 bytes of key row kr0 + (lane%16)/2, columns
  // 16*((lane>>4)&1) + 8*(lane&1) .. +7 of the block, and receives column lane%32, keys kr0..kr0+7.
  // Block db adds 2*db to the chunk index in bits the swizzle's xor commutes with: offset ^ (db*32).
  int vt_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 32 * (j >> 1) + 16 * G + 8 * (j & 1) + ((lane & 15) >> 1);
    vt_off[j] = row * D + (((((lane >> 4) & 1)) ^ att_vswz<D>(row)) * 16) + (lane & 1) * 8;
  }
  auto load_vfrag = [&](const uint8_t* sv, int d) -> v8i {
    if (VSD) {
      v8i f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v2i part = __builtin_amdgcn_ds_read_tr8_b64_v2i32((v2i __attribute__((address_space(3)))*)(sv + (vt_off[j] ^ (d * 32))));
        f[2 * j] = part[0];
        f[2 * j + 1] = part[1];
      }
      return f;
    }
    v4i lo = *(const v4i*)(sv + d * 32 * 64 + v_off[0]);
    v4i hi = *(const v4i*)(sv + d * 32 * 64 + v_off[1]);
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  const int ntiles = S / ATT_BN;

  auto scores = [&](const uint8_t* sk, v16f(&s)[2]) {
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

  // The Q loads above are the only memory operations the compiler tracks; retire them here so that it has no
  // reason to put a vmcnt wait (which would also wait for every DMA in flight) inside the key loops.
  HX_WAIT_VM0();

  float neg_m = __builtin_inff();  // minus the scaled-domain row max

  // Both key loops are software pipelined by one tile: the score MFMAs of tile j+1 are issued before the
  // VALU work on tile j's scores, so the matrix pipe runs under the softmax arithmetic.
  // LDS slots: tile t lives in slot t % 4.  At iteration j the wave reads K of tile j+1 and V of tile j while
  // tiles j+2 and j+3 are in flight; the barrier at the top of iteration j is what frees slot (j+3) % 4.
  if (EXACT) {
    // ---------------- pass 1: exact row max of the raw scores (K tiles only)
    float smax0 = -__builtin_inff(), smax1 = -__builtin_inff();
    for (int t = 0; t < ATT_LEAD && t < ntiles; ++t) issue_k(t, t % ATT_NS);
    att_wait_tiles<KPW>(min(ATT_LEAD - 1, ntiles - 1));
    __syncthreads();
    // one tile: sync, prefetch, issue the score MFMAs of tile j+1 into `next`, then reduce tile j's scores (`cur`)
    auto step1 = [&](v16f(&cur)[2], v16f(&next)[2], int j) {
      if (j + 2 < ntiles) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(KPW));  // tile j+1 landed, tile j+2 may be in flight
      else HX_WAIT_VM0();
      __syncthreads();  // tile j+1 visible to every wave; every wave is done with tile j-1
      if (active) {
        if (j + 1 < ntiles) scores(&smem[(j + 1) % ATT_NS][0][0], next);
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          smax0 = fmaxf(fmaxf(smax0, cur[0][r]), cur[0][r + 1]);
          smax1 = fmaxf(fmaxf(smax1, cur[1][r]), cur[1][r + 1]);
        }
      }
      if (j + ATT_LEAD < ntiles) issue_k(j + ATT_LEAD, (j + ATT_LEAD) % ATT_NS);  // (at the end of the step: see pass 2)
    };
    v16f sa[2], sb[2];
    if (active) scores(&smem[0][0][0], sa);
    int j = 0;
    for (; j + 1 < ntiles; j += 2) {
      step1(sa, sb, j);
      step1(sb, sa, j + 1);
    }
    if (j < ntiles) step1(sa, sb, j);
    float smax = fmaxf(smax0, smax1);
    smax = fmaxf(smax, __shfl_xor(smax, 32));
    neg_m = -(smax * c);  // max(s*c) == max(s)*c for c > 0 (rounding is monotone)
    __syncthreads();      // all waves done with the last K tiles before pass 2 overwrites the slots
  }

  // ---------------- pass 2 (or the only pass)
  v16f o[DB];
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[d][r] = 0.f;
  float l4[4] = {0.f, 0.f, 0.f, 0.f};  // four independent partial row sums per lane
  v8i pf = {0, 0, 0, 0, 0, 0, 0, 0};

  auto softmax_pv = [&](v16f(&s)[2], const uint8_t* sv) {
    if (!EXACT) {
      float t0 = s[0][0], t1 = s[1][0];
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        t0 = fmaxf(fmaxf(t0, s[0][r]), s[0][r + 1]);
        t1 = fmaxf(fmaxf(t1, s[1][r]), s[1][r + 1]);
      }
      float tmax = fmaxf(t0, t1);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
      const float neg_new = fminf(neg_m, -(tmax * c));
      const float alpha = __builtin_amdgcn_exp2f(neg_new - neg_m);  // exp2(m_old - m_new); first tile: exp2(-inf) = 0
      if (__builtin_amdgcn_ballot_w64(neg_new != neg_m)) {  // wave-uniform: most tiles leave every row max alone
#pragma unroll
        for (int i = 0; i < 4; ++i) l4[i] *= alpha;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
      }
      neg_m = neg_new;
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        // s*c - m fused into one rounding: the score already carries the fp8 MFMA's accumulation rounding,
        // three orders of magnitude above the difference between one and two roundings here
        p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][r], c, neg_m));
        l4[r & 3] += p[r];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // both halves of the dword are overwritten, so the previous tile's value serves as the tied operand
        int dw = HX_CVT_PK_E4M3(p[4 * j], p[4 * j + 1], pf[kb * 4 + j], false);
        pf[kb * 4 + j] = HX_CVT_PK_E4M3(p[4 * j + 2], p[4 * j + 3], dw, true);
      }
    }
#pragma unroll
    for (int d = 0; d < DB; ++d) o[d] = hx_mfma_32x32x64_e4m3(load_vfrag(sv, d), pf, o[d]);
  };

  for (int t = 0; t < ATT_LEAD && t < ntiles; ++t) {
    issue_k(t, t % ATT_NS);
    issue_v(t, t % ATT_NS);
  }
  att_wait_tiles<KPW + VPW>(min(ATT_LEAD - 1, ntiles - 1));
  __syncthreads();
  {
    auto step2 = [&](v16f(&cur)[2], v16f(&next)[2], int j) {
      if (j + 2 < ntiles) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(KPW + VPW));
      else HX_WAIT_VM0();
      __syncthreads();
      if (active) {
        if (j + 1 < ntiles) scores(&smem[(j + 1) % ATT_NS][0][0], next);
        softmax_pv(cur, &smem[j % ATT_NS][1][0]);
      }
      // the slot freed by this step's barrier is refilled at the end of the step: four DMA instructions in a row hold
      // the issuing wave up, and here nothing of this step is left to wait behind them (2 % against the top of the step)
      if (j + ATT_LEAD < ntiles) {
        issue_k(j + ATT_LEAD, (j + ATT_LEAD) % ATT_NS);
        issue_v(j + ATT_LEAD, (j + ATT_LEAD) % ATT_NS);
      }
    };
    v16f sa[2], sb[2];
    if (active) scores(&smem[0][0][0], sa);
    int j = 0;
    for (; j + 1 < ntiles; j += 2) {
      step2(sa, sb, j);
      step2(sb, sa, j + 1);
    }
    if (j < ntiles) step2(sa, sb, j);
  }
  const float l_lane = (l4[0] + l4[1]) + (l4[2] + l4[3]);

  __syncthreads();  // every wave is past its last K/V fragment read: the LDS ring can be reused
  if (!active) return;
  // ---------------- epilogue: o[db][4a+b] is O[q0 + lane%32][32 db + 8a + 4G + b]
  // A lane holds 4 consecutive columns of its row, so direct stores would write every output line in 16- or
  // 32-byte pieces.  Each wave instead passes its 32 rows through its own part of the LDS, PASS_COLS columns at a
  // time, and writes 16 bytes per lane with consecutive lanes on consecutive bytes of a row.
  const float l = l_lane + __shfl_xor(l_lane, 32);
  constexpr int ESZ = OUT == HX_F32 ? 4 : 1;
  constexpr int PASS_COLS = OUT == HX_F32 ? D / 2 : D;  // 256 or 128 bytes of a row per pass (128 or 64 for D = 64)
  constexpr int PASS_BYTES = PASS_COLS * ESZ;
  constexpr int RSTR = PASS_BYTES + 16;                 // padded row stride
  constexpr int LPR = PASS_BYTES / 16;                  // lanes per row on the way out
  constexpr int RPI = 64 / LPR;                         // rows per store instruction
  constexpr int NDB = PASS_COLS / 32;                   // 32-column accumulator blocks per pass
  static_assert(ATT_WAVES * 32 * RSTR <= ATT_NS * 2 * TILE, "output staging fits the K/V ring");
  uint8_t* st = &smem[0][0][0] + w * (32 * RSTR);
  uint8_t* out_rows = (uint8_t*)Out + ((long)bh * S + q0) * D * ESZ;
  const int rb_row = lane / LPR, rb_ch = lane % LPR;
#pragma unroll
  for (int h = 0; h < D / PASS_COLS; ++h) {
#pragma unroll
    for (int dd = 0; dd < NDB; ++dd)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int d = h * NDB + dd;
        if (OUT == HX_F32) {
          v4f v;
#pragma unroll
          for (int b = 0; b < 4; ++b) v[b] = o[d][4 * a + b] / l;
          *(v4f*)(st + q31 * RSTR + (dd * 32 + 8 * a + 4 * G) * 4) = v;
        } else {
          int dw = HX_CVT_PK_E4M3(o[d][4 * a] / l, o[d][4 * a + 1] / l, 0, false);
          dw = HX_CVT_PK_E4M3(o[d][4 * a + 2] / l, o[d][4 * a + 3] / l, dw, true);
          *(int*)(st + q31 * RSTR + dd * 32 + 8 * a + 4 * G) = dw;
        }
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // LDS operations of one wave execute in order
#pragma unroll
    for (int p = 0; p < 32 / RPI; ++p) {
      const int row = p * RPI + rb_row;
      const v4i v = *(const v4i*)(st + row * RSTR + rb_ch * 16);
      *(v4i*)(out_rows + ((long)row * D + h * PASS_COLS) * ESZ + rb_ch * 16) = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// ------------------------------------------------------------------------------------------
// general: any S, D <= 256, any V strides; one workgroup per query row, exact row max (two sweeps over the keys),
// p quantised to e4m3 against it, l from the un-quantised p.  Correctness path for the shapes the MFMA kernel does
// not take; it always computes the exact-max form.
// ------------------------------------------------------------------------------------------
template <int OUT>
__global__ __launch_bounds__(256) void hx_fp8_attention_general(const uint8_t* __restrict__ Q, const uint8_t* __restrict__ Kt,
                                                               const uint8_t* __restrict__ Vt, void* __restrict__ Out, int S, int D,
                                                               long vsd, long vss, float c) {
  constexpr int CH = 1024;
  __shared__ float sq[256];
  __shared__ float sp[CH];
  __shared__ float red[256];
  const int tid = threadIdx.x;
  const long bh = blockIdx.y, qi = blockIdx.x;
  const uint8_t* Kh = Kt + bh * (long)S * D;
  const uint8_t* Vh = Vt + bh * (long)S * D;
  if (tid < D) sq[tid] = hx_e4m3_to_f32(Q[(bh * S + qi) * D + tid]);
  __syncthreads();
  auto score = [&](int key) {
    const uint8_t* kr = Kh + (long)key * D;
    float s = 0.f;
    for (int d = 0; d < D; ++d) s = __builtin_fmaf(sq[d], hx_e4m3_to_f32(kr[d]), s);
    return s;
  };
  auto block_reduce = [&](float v, bool is_max) {
    red[tid] = v;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
      if (tid < st) red[tid] = is_max ? fmaxf(red[tid], red[tid + st]) : red[tid] + red[tid + st];
      __syncthreads();
    }
    const float r = red[0];
    __syncthreads();
    return r;
  };
  float smax = -__builtin_inff();
  for (int key = tid; key < S; key += 256) smax = fmaxf(smax, score(key));
  const float neg_m = -(block_reduce(smax, true) * c);
  float lsum = 0.f, acc = 0.f;
  for (int n0 = 0; n0 < S; n0 += CH) {
    const int cn = min(CH, S - n0);
    for (int i = tid; i < cn; i += 256) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(score(n0 + i), c, neg_m));
      lsum += p;
      sp[i] = hx_e4m3_to_f32((uint8_t)(HX_CVT_PK_E4M3(p, 0.f, 0, false) & 0xFF));
    }
    __syncthreads();
    if (tid < D)
      for (int i = 0; i < cn; ++i) acc = __builtin_fmaf(sp[i], hx_e4m3_to_f32(Vh[(long)tid * vsd + (long)(n0 + i) * vss]), acc);
    __syncthreads();
  }
  const float l = block_reduce(lsum, false);
  if (tid < D) {
    const float o = acc / l;
    const long at = (bh * S + qi) * D + tid;
    if (OUT == HX_F32) ((float*)Out)[at] = o;
    else ((uint8_t*)Out)[at] = (uint8_t)(HX_CVT_PK_E4M3(o, 0.f, 0, false) & 0xFF);
  }
}

template <int D, int OUT, bool EXACT, bool VSD>
static void launch_att_kernel(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, float c, hipStream_t s) {
  const int qtiles = (int)((S + ATT_BM - 1) / ATT_BM);
  const int hpx = (int)((BH + 7) / 8);
  const int grid = 8 * hpx * qtiles;
  hx_launch((hx_fp8_attention_kernel<D, OUT, EXACT, VSD>), dim3(grid), dim3(256), 0, s, (const uint8_t*)q, (const uint8_t*)k,
                     (const uint8_t*)v, out, (int)S, (int)BH, qtiles, c);
}

template <int D, int OUT>
static int launch_att(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, int exact, bool vsd, float c, hipStream_t s) {
  if (exact) {
    if (vsd) launch_att_kernel<D, OUT, true, true>(q, k, v, out, BH, S, c, s);
    else launch_att_kernel<D, OUT, true, false>(q, k, v, out, BH, S, c, s);
  } else {
    if (vsd) launch_att_kernel<D, OUT, false, true>(q, k, v, out, BH, S, c, s);
    else launch_att_kernel<D, OUT, false, false>(q, k, v, out, BH, S, c, s);
  }
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_fp8_attention: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

extern "C" int hx_fp8_attention(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, int64_t D,
                                int64_t scale_dim, int64_t v_stride_d, int64_t v_stride_s, int out_dtype, int exact_max,
                                void* stream) {
  if (BH < 0 || S < 0 || D < 0 || scale_dim < 0) {
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
  if (BH * S * D >= (1LL << 40) || S * D >= (1LL << 31)) {
    hx_set_error("hx_fp8_attention: problem too large");
    return HX_ERR_UNSUPPORTED;
  }
  hipStream_t s = (hipStream_t)stream;
  // the softmax scale in base 2, evaluated the way the reference does: double arithmetic, rounded to fp32 once
  const float c = (float)((1.0 / sqrt((double)(scale_dim > 0 ? scale_dim : (D > 0 ? D : 1)))) * 1.44269504);
  bool vsd = false, fast = (D == 64 || D == 128) && (S % ATT_BN) == 0 && ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) == 0);
  if (v_stride_s == 1 && (v_stride_d == S || D == 1)) vsd = false;       // [D][S] per head
  else if (v_stride_d == 1 && (v_stride_s == D || S == 1)) vsd = true;   // [S][D] per head
  else fast = false;
  if (!fast) {  // any other shape, alignment or V striding within a head (heads are D*S elements apart)
    if (D > 256 || D < 1 || BH >= 65536) {
      hx_set_error("hx_fp8_attention: unsupported shape S=%lld D=%lld BH=%lld (MFMA kernel: D in {64,128}, S %% 64 == 0; plain kernel: D <= 256, BH < 65536)",
                   (long long)S, (long long)D, (long long)BH);
      return HX_ERR_UNSUPPORTED;
    }
    const dim3 grid((unsigned)S, (unsigned)BH);
    if (out_dtype == HX_F32)
      hx_launch(hx_fp8_attention_general<HX_F32>, grid, dim3(256), 0, s, (const uint8_t*)q, (const uint8_t*)k, (const uint8_t*)v,
                         out, (int)S, (int)D, (long)v_stride_d, (long)v_stride_s, c);
    else
      hx_launch(hx_fp8_attention_general<HX_E4M3>, grid, dim3(256), 0, s, (const uint8_t*)q, (const uint8_t*)k,
                         (const uint8_t*)v, out, (int)S, (int)D, (long)v_stride_d, (long)v_stride_s, c);
    hipError_t e = hx_launch_status();
    if (e != hipSuccess) {
      hx_set_error("hx_fp8_attention: launch failed: %s", hipGetErrorString(e));
      return (int)e;
    }
    return 0;
  }
  if (D == 128) {
    if (out_dtype == HX_F32) return launch_att<128, HX_F32>(q, k, v, out, BH, S, exact_max, vsd, c, s);
    return launch_att<128, HX_E4M3>(q, k, v, out, BH, S, exact_max, vsd, c, s);
  }
  if (out_dtype == HX_F32) return launch_att<64, HX_F32>(q, k, v, out, BH, S, exact_max, vsd, c, s);
  return launch_att<64, HX_E4M3>(q, k, v, out, BH, S, exact_max, vsd, c, s);
}
