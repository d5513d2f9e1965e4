// 16-bit (bf16 / fp16) attention for gfx950 — device side of examples/attention.py:33-84 of the reference:
//   per (batch*head):  s = (q k^T) * c,  c = 1/sqrt(D) * 1.44269504;   online softmax in base 2 (m, l, acc in fp32);
//                      p = exp2(s - m) is cast to the value dtype for the P.V product, l sums the un-rounded p;
//                      out = cast(acc / l).
// q [BH, M, D], k [BH, N, D], v [BH, N, D], out [BH, M, D], all contiguous.
//
// MFMA kernel (D in {64, 128}): workgroup = 4 waves = 128 queries of one head, wave = 32 queries.
// Per 64-key tile a wave computes S^T = K Q^T as two 32x32 blocks (32x32x16 MFMA, D/16 k-steps), so lane
// (q = lane%32, G = lane/32) holds, per block, the scores of query q against keys 8*(r/4) + 4G + r%4, r = 0..15.
// Registers 8u' .. 8u'+7 of a block, cast to 16 bits, are exactly the B operand of one k-step (16 keys) of
// O^T[d][q] += V^T[d][key] P^T[key][q]; the matching V^T operand — for d = lane%32 the keys 16u + 8h + 4G + (0..3),
// h = 0, 1 — is formed by two transposing LDS reads (ds_read_b64_tr_b16: 4 keys x 16 columns per 16 lanes) of the V
// tile, which sits in LDS the way it sits in memory, rows = keys.  Row max and row sum need no cross-lane traffic
// beyond one exchange between the two lanes of a query per tile.  TAIL instantiations handle N % 64 != 0: the DMA of
// the last tile re-reads row N-1 for the missing keys and their scores are set to -inf before the softmax.
#include "hx_common.h"

#include <cmath>
#include <type_traits>

#define A16_BN 64
#define A16_WAVES 4
#define A16_BM (32 * A16_WAVES)
#define A16_SLACK 8.f  // log2 of how far a row's running max may exceed its softmax reference point

// K tile [64 keys][2D bytes], read as the A operand with 16-byte loads (16 lanes = 16 consecutive rows are served
// together): the 16-byte chunk index is xor-ed so that those rows land in 16 different bank groups.
template <int D>
__device__ __forceinline__ int a16_kswz(int row) {
  return D == 128 ? (row & 15) : ((row >> 1) & 7);
}
// V tile, same shape, read with transposing 8-byte loads: 32 lanes fetch 4 consecutive key rows x 64 contiguous
// bytes; the rows must land in different 64-byte quarters of the 256-byte bank window.
template <int D>
__device__ __forceinline__ int a16_vswz(int row) {
  return D == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2);
}

template <int D, bool BF, bool TAIL>
__global__ __launch_bounds__(64 * A16_WAVES, 2) void hx_attention16_kernel(const uint8_t* __restrict__ Q, const uint8_t* __restrict__ Kp,
                                                                const uint8_t* __restrict__ Vp, void* __restrict__ Out, int M, int N,
                                                                int BH, int qtiles, float c) {
  typedef typename Mfma16<BF>::T T16;
  typedef typename Mfma16<BF>::V8 V8;
  constexpr int RB = 2 * D;                                  // bytes of a row
  constexpr int KSTEPS = D / 16;                             // MFMA k-steps of S^T
  constexpr int DB = D / 32;                                 // 32-row blocks of O^T
  constexpr int RPD = 1024 / RB;                             // tile rows per DMA instruction
  constexpr int IPW = (A16_BN / RPD) / A16_WAVES;            // DMA instructions per wave per tile (K, and again V)
  constexpr int TILE = A16_BN * RB;                          // bytes of a K (or V) tile
  constexpr int NS = D == 128 ? 2 : 4;                       // ring slots for K and for V: 64 KB of LDS either way
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2][NS][TILE];  // [K | V][slot]

  // workgroup -> (head, query tile): XCD x (= id%8) takes heads x, x+8, ...; the query tiles of a head are
  // consecutive on that XCD so its K/V stay in that XCD's L2.
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
  const int q0 = qt * A16_BM + w * 32;
  const bool active = q0 < M;  // wave-uniform; inactive waves still help with DMA and barriers

  const uint8_t* Qh = Q + (long)bh * M * RB;
  const uint8_t* Kh = Kp + (long)bh * N * RB;
  const uint8_t* Vh = Vp + (long)bh * N * RB;

  // ---- Q fragments (B operand of S^T): lane (q, G): Q[q][16t + 8G .. +7]
  V8 qf[KSTEPS];
  {
    const int qrow = min(q0 + q31, M - 1);
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) qf[t] = *(const V8*)(Qh + (long)qrow * RB + 32 * t + 16 * G);
  }

  // ---- DMA addressing: wave w issues instructions j = w, w+4, ... of a tile (RPD rows each).  The swizzle of a
  // lane's row does not depend on which of the wave's instructions it is, so one per-lane offset serves all.
  constexpr int CPR = RB / 16;  // chunks per row
  const int lrow = lane / CPR, lpos = lane % CPR;
  const uint32_t k_vo = (uint32_t)(lrow * RB + ((lpos ^ a16_kswz<D>(w * RPD + lrow)) * 16));
  const uint32_t v_vo = (uint32_t)(lrow * RB + ((lpos ^ a16_vswz<D>(w * RPD + lrow)) * 16));
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]);
  // TAIL: rows past the end of K / V are replaced by row N-1 (valid, finite data; the scores are masked)
  auto tail_vo = [&](uint32_t vo, int tile, int j) {
    const int rit = min(j * RPD + lrow, N - 1 - tile * A16_BN);  // row in tile, clamped
    return (uint32_t)(rit * RB) + (vo - (uint32_t)(lrow * RB));
  };
  auto issue_k_one = [&](int tile, int jj) {
    const int j = w + A16_WAVES * jj;
    const uint32_t lds = lds0 + (uint32_t)(tile % NS) * TILE + j * 1024;
    if (TAIL) hx_g2l16_s(Kh + (long)tile * A16_BN * RB, tail_vo(k_vo, tile, j), lds);
    else hx_g2l16_s(Kh + ((long)tile * A16_BN + j * RPD) * RB, k_vo, lds);
  };
  auto issue_v_one = [&](int tile, int jj) {
    const int j = w + A16_WAVES * jj;
    const uint32_t lds = lds0 + (uint32_t)(NS + tile % NS) * TILE + j * 1024;
    if (TAIL) hx_g2l16_s(Vh + (long)tile * A16_BN * RB, tail_vo(v_vo, tile, j), lds);
    else hx_g2l16_s(Vh + ((long)tile * A16_BN + j * RPD) * RB, v_vo, lds);
  };
  auto issue_k = [&](int tile) {
#pragma unroll
    for (int jj = 0; jj < IPW; ++jj) issue_k_one(tile, jj);
  };
  auto issue_v = [&](int tile) {
#pragma unroll
    for (int jj = 0; jj < IPW; ++jj) issue_v_one(tile, jj);
  };

  // ---- MFMA operand addressing
  // K (A operand of S^T): lane (i = lane%32, G) reads row 32 kb + i, chunk 2t + G.  The chunk's xor with the swizzle
  // and the k-step's 2t act on disjoint bits of a row, so k-step t is an xor with 32 t on the byte offset.
  int k_off[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const int row = 32 * kb + q31;
    k_off[kb] = row * RB + ((G ^ a16_kswz<D>(row)) * 16);
  }
  // V (A operand of O^T): transposing read (u, h) fetches keys 16u + 8h + 4G + te, te = (lane>>2)&3; this lane supplies
  // 8 bytes = columns 32 db + 16*((lane>>4)&1) + 4*(lane&3) .. +3 of that key row and receives column 32 db + lane%32.
  // Block db adds 4 db to the chunk index, bits that the swizzle xors: an xor with 64 db on the byte offset.
  int v_off;
  {
    const int te = (lane >> 2) & 3, tq = lane & 3, row = 4 * G + te;
    const int chunk = 2 * ((lane >> 4) & 1) + (tq >> 1);
    v_off = row * RB + ((chunk ^ a16_vswz<D>(row)) * 16) + (tq & 1) * 8;
  }
  auto load_vfrag = [&](const uint8_t* sv, int u, int db) -> V8 {
    v4s part[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
      part[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (v4s __attribute__((address_space(3)))*)(sv + ((v_off + (16 * u + 8 * h) * RB) ^ (64 * db))));
    v8s both = (v8s){part[0][0], part[0][1], part[0][2], part[0][3], part[1][0], part[1][1], part[1][2], part[1][3]};
    return __builtin_bit_cast(V8, both);
  };

  const int ntiles = (N + A16_BN - 1) / A16_BN;

  auto load_kfrag = [&](const uint8_t* sk, int mi) -> V8 {  // A operand of score MFMA mi = kb * KSTEPS + t
    return *(const V8*)(sk + (k_off[mi / KSTEPS] ^ (32 * (mi % KSTEPS))));
  };
  const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  auto scores = [&](const uint8_t* sk, v16f(&s)[2]) {  // compiler-scheduled; used for the first tile only
#pragma unroll
    for (int mi = 0; mi < 2 * KSTEPS; ++mi)
      s[mi / KSTEPS] = Mfma16<BF>::run(load_kfrag(sk, mi), qf[mi % KSTEPS], mi % KSTEPS ? s[mi / KSTEPS] : zero16);
  };

  // The Q loads are the only memory operations the compiler tracks; retire them here so that it has no reason to put
  // a vmcnt wait (which would also wait for every DMA in flight) inside the key loop.
  HX_WAIT_VM0();

  float neg_m = __builtin_inff();  // minus the scaled-domain running row max
  v16f o[DB];
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[d][r] = 0.f;
  float l4[4] = {0.f, 0.f, 0.f, 0.f};  // four independent partial row sums per lane

  // Pipeline.  K(t) and V(t) live in slot t % NS of their rings; step j reads K(j+1) and V(j); its barrier frees the
  // slots of K(j) and V(j-1), which take K(j+NS) and V(j+NS-1) (past the end: the last tile again, so that every step
  // issues the same number of DMA instructions and the counted waits stay exact).
  //
  // Inside a step the instruction order is pinned by scheduling barriers, one slot per MFMA, because left to itself
  // the compiler emits the score MFMAs of the next tile, then the whole softmax, then the P.V MFMAs, and the matrix
  // pipe idles through the middle part:
  //   phase 0: row max of tile j's scores, new reference point, (rarely) rescaling of l and the accumulators;
  //   phase A: one slot per score MFMA of tile j+1, each followed by exp2 / row sum / 16-bit cast of a few of tile j's
  //            scores;
  //   phase B: one slot per P.V MFMA of tile j.
  // Fragments are read from LDS two slots ahead of the MFMA that consumes them; the step's DMA instructions go out one
  // after every fourth MFMA (a burst of them would hold the in-order instruction stream up).
  constexpr int NA = 2 * KSTEPS, NB = 4 * DB, EPS = 32 / NA;
  auto issue_step0 = [&](int t) {  // what "step t - NS" would have issued
    issue_k(min(t, ntiles - 1));
    if (t >= 1) issue_v(min(t - 1, ntiles - 1));
  };
  for (int t = 0; t < NS; ++t) issue_step0(t);
  __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((NS - 2) * 2 * IPW));
  __syncthreads();
  {
    auto step = [&](v16f(&cur)[2], v16f(&next)[2], int j, auto has_next_c) {
      constexpr bool HAS_NEXT = decltype(has_next_c)::value;
      __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm((NS - 2) * 2 * IPW));  // this wave's part of K(j+1) and V(j) has landed
      __syncthreads();
      const int dk = min(j + NS, ntiles - 1), dv = min(j + NS - 1, ntiles - 1);
      if (!active) {
        issue_k(dk);
        issue_v(dv);
        return;
      }
      const uint8_t* sk = &smem[0][(j + 1) % NS][0];
      const uint8_t* sv = &smem[1][j % NS][0];
      V8 kf[3], vf[3];
      if (HAS_NEXT) {
        kf[0] = load_kfrag(sk, 0);
        kf[1] = load_kfrag(sk, 1);
      }
      // ---- phase 0
      if (TAIL && j == ntiles - 1) {  // keys past the end: score -inf, p = 0
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (j * A16_BN + 32 * kb + 8 * (r >> 2) + 4 * G + (r & 3) >= N) cur[kb][r] = -__builtin_inff();
      }
      float t0 = cur[0][0], t1 = cur[1][0];
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        t0 = fmaxf(fmaxf(t0, cur[0][r]), cur[0][r + 1]);
        t1 = fmaxf(fmaxf(t1, cur[1][r]), cur[1][r + 1]);
      }
      float tmax = fmaxf(t0, t1);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
      // The reference point m of a row only moves when the tile's max exceeds it by more than 2^A16_SLACK: p, l and
      // the accumulators then run up to that factor above their usual range (p <= 256: exact in either 16-bit format,
      // and further from its underflow), the quotient acc / l is unchanged, and the rescaling pass below — 70
      // multiplies per lane — runs on a few tiles per row block instead of on most of them.
      const float cand = -(tmax * c);
      const float neg_new = cand < neg_m - A16_SLACK ? cand : neg_m;
      const float alpha = __builtin_amdgcn_exp2f(neg_new - neg_m);  // exp2(m_old - m_new); first tile: exp2(-inf) = 0
      if (__builtin_amdgcn_ballot_w64(neg_new != neg_m)) {         // wave-uniform
#pragma unroll
        for (int i = 0; i < 4; ++i) l4[i] *= alpha;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
      }
      neg_m = neg_new;
      __builtin_amdgcn_sched_barrier(0);
      // ---- phase A
      V8 pf[4];
#pragma unroll
      for (int mi = 0; mi < NA; ++mi) {
        if (HAS_NEXT) {
          if (mi + 2 < NA) kf[(mi + 2) % 3] = load_kfrag(sk, mi + 2);
          next[mi / KSTEPS] = Mfma16<BF>::run(kf[mi % 3], qf[mi % KSTEPS], mi % KSTEPS ? next[mi / KSTEPS] : zero16);
        }
#pragma unroll
        for (int e = mi * EPS; e < (mi + 1) * EPS; ++e) {
          const int kb = e >> 4, r = e & 15;
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(cur[kb][r], c, neg_m));
          l4[r & 3] += p;
          pf[2 * kb + (r >> 3)][r & 7] = (T16)p;
        }
        if ((mi & 3) == 1 && (mi >> 2) < IPW) issue_k_one(dk, mi >> 2);
        if (mi >= NA - 2) vf[mi - (NA - 2)] = load_vfrag(sv, 0, mi - (NA - 2));
        __builtin_amdgcn_sched_barrier(0);
      }
      // ---- phase B
#pragma unroll
      for (int mi = 0; mi < NB; ++mi) {
        if (mi + 2 < NB) vf[(mi + 2) % 3] = load_vfrag(sv, (mi + 2) / DB, (mi + 2) % DB);
        o[mi % DB] = Mfma16<BF>::run(vf[mi % 3], pf[mi / DB], o[mi % DB]);
        if ((mi & 3) == 1 && (mi >> 2) < IPW) issue_v_one(dv, mi >> 2);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    v16f sa[2], sb[2];
    if (active) scores(&smem[0][0][0], sa);
    int j = 0;
    for (; j + 2 < ntiles; j += 2) {
      step(sa, sb, j, std::true_type{});
      step(sb, sa, j + 1, std::true_type{});
    }
    if (j + 1 < ntiles) {
      step(sa, sb, j, std::true_type{});
      step(sb, sa, j + 1, std::false_type{});
    } else {
      step(sa, sb, j, std::false_type{});
    }
  }
  HX_WAIT_VM0();  // the trailing re-fetches have landed before the LDS is reused
  const float l_lane = (l4[0] + l4[1]) + (l4[2] + l4[3]);

  __syncthreads();  // every wave is past its last K/V fragment read: the LDS can be reused
  if (!active) return;
  // ---------------- epilogue: o[db][4a+b] is O[q0 + lane%32][32 db + 8a + 4G + b].  Each wave passes its 32 rows
  // through its own part of the LDS and writes 16 bytes per lane, consecutive lanes on consecutive bytes of a row.
  const float l = l_lane + __shfl_xor(l_lane, 32);
  constexpr int RSTR = RB + 16;  // padded row stride
  constexpr int LPR = RB / 16;   // lanes per row on the way out
  constexpr int RPI = 64 / LPR;  // rows per store instruction
  static_assert(A16_WAVES * 32 * RSTR <= 2 * NS * TILE, "output staging fits the K/V rings");
  uint8_t* st = &smem[0][0][0] + w * (32 * RSTR);
  uint8_t* out_rows = (uint8_t*)Out + ((long)bh * M + q0) * RB;
  typedef T16 ov4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      ov4 v;
#pragma unroll
      for (int b = 0; b < 4; ++b) v[b] = (T16)(o[d][4 * a + b] / l);
      *(ov4*)(st + q31 * RSTR + (32 * d + 8 * a + 4 * G) * 2) = v;
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // LDS operations of one wave execute in order
  const int rb_row = lane / LPR, rb_ch = lane % LPR;
#pragma unroll
  for (int p = 0; p < 32 / RPI; ++p) {
    const int row = p * RPI + rb_row;
    const v4i v = *(const v4i*)(st + row * RSTR + rb_ch * 16);
    if (q0 + row < M) *(v4i*)(out_rows + (long)row * RB + rb_ch * 16) = v;
  }
}

// ------------------------------------------------------------------------------------------
// general: any M, N, D <= 256, fp16 / bf16 / fp32; one workgroup per query row, keys in chunks of 1024
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void hx_attention_general(const T* __restrict__ Q, const T* __restrict__ Kp, const T* __restrict__ Vp,
                                                           T* __restrict__ Out, int M, int N, int D, float c) {
  constexpr int CH = 1024;
  __shared__ float sq[256];
  __shared__ float sp[CH];
  __shared__ float red[256];
  const int tid = threadIdx.x;
  const long bh = blockIdx.y, qi = blockIdx.x;
  const T* q = Q + (bh * M + qi) * D;
  const T* Kh = Kp + bh * (long)N * D;
  const T* Vh = Vp + bh * (long)N * D;
  if (tid < D) sq[tid] = (float)q[tid];
  __syncthreads();
  float m = -__builtin_inff(), l = 0.f, acc = 0.f;
  for (int n0 = 0; n0 < N; n0 += CH) {
    const int cn = min(CH, N - n0);
    float lmax = -__builtin_inff();
    for (int i = tid; i < cn; i += 256) {
      const T* kr = Kh + (long)(n0 + i) * D;
      float s = 0.f;
      for (int d = 0; d < D; ++d) s = __builtin_fmaf(sq[d], (float)kr[d], s);
      sp[i] = s;
      lmax = fmaxf(lmax, s);
    }
    red[tid] = lmax;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
      if (tid < st) red[tid] = fmaxf(red[tid], red[tid + st]);
      __syncthreads();
    }
    const float m_new = fmaxf(m, red[0] * c);
    __syncthreads();
    float lsum = 0.f;
    for (int i = tid; i < cn; i += 256) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sp[i], c, -m_new));
      lsum += p;
      sp[i] = (float)(T)p;  // the P.V product takes p in the value dtype
    }
    red[tid] = lsum;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
      if (tid < st) red[tid] += red[tid + st];
      __syncthreads();
    }
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    l = l * alpha + red[0];
    acc *= alpha;
    if (tid < D)
      for (int i = 0; i < cn; ++i) acc = __builtin_fmaf(sp[i], (float)Vh[(long)(n0 + i) * D + tid], acc);
    m = m_new;
    __syncthreads();
  }
  if (tid < D) Out[(bh * M + qi) * D + tid] = (T)(acc / l);
}

static bool att16_fast_ok(const void* q, const void* k, const void* v, const void* out, int64_t BH, int64_t M, int64_t N, int64_t D,
                          int dtype) {
  if (dtype != HX_BF16 && dtype != HX_F16) return false;
  if (D != 64 && D != 128) return false;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) return false;
  if (N * D * 2 >= (1LL << 31) || M * D * 2 >= (1LL << 31)) return false;
  return true;
}

extern "C" int hx_attention_path(int64_t BH, int64_t M, int64_t N, int64_t D, int dtype, const void* q, const void* k, const void* v,
                                 const void* out) {
  if (BH <= 0 || M <= 0 || N <= 0) return 0;
  return att16_fast_ok(q, k, v, out, BH, M, N, D, dtype) ? 1 : 0;
}

template <int D, bool BF>
static void launch_att16(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t M, int64_t N, float c, hipStream_t s) {
  const int qtiles = (int)((M + A16_BM - 1) / A16_BM);
  const int hpx = (int)((BH + 7) / 8);
  if (N % A16_BN)
    hx_launch((hx_attention16_kernel<D, BF, true>), dim3(8 * hpx * qtiles), dim3(64 * A16_WAVES), 0, s, (const uint8_t*)q,
                       (const uint8_t*)k, (const uint8_t*)v, out, (int)M, (int)N, (int)BH, qtiles, c);
  else
    hx_launch((hx_attention16_kernel<D, BF, false>), dim3(8 * hpx * qtiles), dim3(64 * A16_WAVES), 0, s, (const uint8_t*)q,
                       (const uint8_t*)k, (const uint8_t*)v, out, (int)M, (int)N, (int)BH, qtiles, c);
}

extern "C" int hx_attention(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t M, int64_t N, int64_t D,
                            int64_t scale_dim, int dtype, void* stream) {
  if (BH < 0 || M < 0 || N < 0 || D < 0) {
    hx_set_error("hx_attention: negative size");
    return HX_ERR_BAD_ARG;
  }
  if (dtype != HX_BF16 && dtype != HX_F16 && dtype != HX_F32) {
    hx_set_error("hx_attention: dtype must be HX_BF16, HX_F16 or HX_F32, got %d", dtype);
    return HX_ERR_BAD_ARG;
  }
  if (scale_dim < 0) {
    hx_set_error("hx_attention: negative scale_dim");
    return HX_ERR_BAD_ARG;
  }
  if (BH == 0 || M == 0 || D == 0) return 0;
  if (N == 0) {
    hx_set_error("hx_attention: no keys (softmax over an empty set)");
    return HX_ERR_BAD_ARG;
  }
  if (!q || !k || !v || !out) {
    hx_set_error("hx_attention: null pointer");
    return HX_ERR_BAD_ARG;
  }
  if (M >= (1LL << 31) || N >= (1LL << 31) || BH * M * D >= (1LL << 40) || BH * N * D >= (1LL << 40)) {
    hx_set_error("hx_attention: problem too large");
    return HX_ERR_UNSUPPORTED;
  }
  hipStream_t s = (hipStream_t)stream;
  // the softmax scale in base 2, evaluated the way the reference does: double arithmetic, rounded to fp32 once
  const float c = (float)((1.0 / sqrt((double)(scale_dim > 0 ? scale_dim : D))) * 1.44269504);
  if (att16_fast_ok(q, k, v, out, BH, M, N, D, dtype)) {
    if (D == 128) {
      if (dtype == HX_BF16) launch_att16<128, true>(q, k, v, out, BH, M, N, c, s);
      else launch_att16<128, false>(q, k, v, out, BH, M, N, c, s);
    } else {
      if (dtype == HX_BF16) launch_att16<64, true>(q, k, v, out, BH, M, N, c, s);
      else launch_att16<64, false>(q, k, v, out, BH, M, N, c, s);
    }
  } else {
    if (D > 256 || BH >= 65536) {
      hx_set_error("hx_attention: unsupported shape D=%lld BH=%lld (plain kernel: head dimension <= 256, batch*heads < 65536)",
                   (long long)D, (long long)BH);
      return HX_ERR_UNSUPPORTED;
    }
    const dim3 grid((unsigned)M, (unsigned)BH);
    if (dtype == HX_BF16)
      hx_launch(hx_attention_general<__bf16>, grid, dim3(256), 0, s, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v,
                         (__bf16*)out, (int)M, (int)N, (int)D, c);
    else if (dtype == HX_F16)
      hx_launch(hx_attention_general<_Float16>, grid, dim3(256), 0, s, (const _Float16*)q, (const _Float16*)k,
                         (const _Float16*)v, (_Float16*)out, (int)M, (int)N, (int)D, c);
    else
      hx_launch(hx_attention_general<float>, grid, dim3(256), 0, s, (const float*)q, (const float*)k, (const float*)v,
                         (float*)out, (int)M, (int)N, (int)D, c);
  }
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_attention: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}
