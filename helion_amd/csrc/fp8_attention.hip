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
#include <type_traits>

#define ATT_BN 64      // keys per tile
#define ATT_WAVES 4
#define ATT_BM (32 * ATT_WAVES)
#define ATT_NS 4       // LDS stages: tiles j .. j+2 are in flight while tile j is consumed
#define ATT_LEAD (ATT_NS - 1)

// K tile: [64 keys][D bytes]; V tile: [D rows][64 bytes].  Rows are 16-byte chunks, swizzled:
//   row bytes 128: pos = chunk ^ ((row >> 1) & 7);   row bytes 64: pos = chunk ^ ((row >> 2) & 3);   row bytes 256
//   (a row fills the 256-byte bank window): pos = chunk ^ (row & 15)
template <int RB>
__device__ __forceinline__ int att_swz(int row) {
  return RB == 256 ? (row & 15) : RB == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}
// V tile in the [keys][D bytes] layout: one transposing read has 32 lanes fetch 8 consecutive key rows x two
// adjacent 16-byte chunks; the swizzle has to spread those over all banks and must leave bit 0 (which chunk of
// the pair) alone.  RB = 128: rows r, r+1 share a 256-byte bank window -> (r>>1)&3 into bits 2:1;  RB = 64: rows
// r, r+4 share a 64-byte quarter of it -> (r>>2)&1 into bit 1.
template <int RB>
__device__ __forceinline__ int att_vswz(int row) {
  return RB == 256 ? ((row & 7) << 1) : RB == 128 ? (((row >> 1) & 3) << 1) : (((row >> 2) & 1) << 1);
}

// ------------------------------------------------------------------------------------------
// The MFMA kernel, software-pipelined three tiles deep.  MODE 1: exact row max (two passes); MODE 0: online softmax.
//
// What was measured on gfx950 and shapes this kernel:
//   * a SIMD issues one VALU-class instruction at a time and an fp8 MFMA holds that port for most of its 64 cycles:
//     on this kernel's instruction mix each 32x32x64 MFMA leaves room for about eight other VALU instructions of any
//     kind in its shadow, and what does not fit is paid in full.  So no wave may ever wait on the LDS, and the VALU
//     work has to be spread evenly between the MFMAs;
//   * step j of the key loop therefore issues the score MFMAs of tile j+1, the softmax arithmetic of tile j and the
//     P.V MFMAs of tile j-1: eight MFMAs that do not depend on the step's VALU work, one per micro-step, each followed
//     by its share of the fma / exp2 / convert instructions; fragments are read from the LDS two MFMAs ahead;
//   * the key loop is unrolled four times so that the LDS slot of every fragment read is an immediate offset, and every
//     step issues the same DMA instructions (past the last tile it re-fetches the last tile into a slot nobody reads
//     any more), so its body has no branch and one constant vmcnt wait;
//   * pass 1 (MODE 1) streams K through all eight tile slots of the ring and synchronises once per two tiles.
// LDS: K(t) lives in the K half of slot t % 4 from step t-4 to step t-1, V(t) in the V half of the same slot from
// step t-2 to step t+1.
// Any sequence length: the last key tile may be partial (keys past S are masked to -inf before the max and the
// exponential; their K / V rows are re-reads of valid rows), and so may the last query rows of a wave.
// ------------------------------------------------------------------------------------------
template <int IPT>
__device__ __forceinline__ void att_wait_outstanding(int n) {  // n tiles' worth of this wave's DMA may stay in flight
  switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(0)); break;
    case 1: __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(IPT)); break;
    case 2: __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(2 * IPT)); break;
    case 3: __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(3 * IPT)); break;
    case 4: __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(4 * IPT)); break;
    default: __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(5 * IPT)); break;
  }
}

// v_max3_f32 as one instruction (fmaxf(fmaxf(a, b), c) first canonicalises every operand that comes out of an MFMA,
// which doubles the instruction count of a max reduction)
__device__ __forceinline__ float att_max3(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}

// max over the two halves of the wave: lane l and lane l ^ 32 both receive max(x[l], x[l ^ 32])
__device__ __forceinline__ float att_max_across_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// D = 256 (opt-in, HX_FEATURE_ATTENTION_D256): the same code with 16 KB tiles - the ring is then 128 KB and the O^T
// accumulators 128 registers, so one workgroup per CU and one wave per SIMD.
template <int D, int OUT, int MODE, bool VSD>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void hx_fp8_attention_pipe(const uint8_t* __restrict__ Q, const uint8_t* __restrict__ Kt,
                                                                const uint8_t* __restrict__ Vt, void* __restrict__ Out, int S, int BH,
                                                                int qtiles, float c) {
  constexpr int KSTEPS = D / 64;  // MFMA k-steps for S = K Q^T
  constexpr int DB = D / 32;      // 32-row blocks of O^T == score MFMAs per tile (2 key blocks x KSTEPS)
  constexpr int KROWS_PER_DMA = 1024 / D;
  constexpr int KPW = (ATT_BN / KROWS_PER_DMA) / ATT_WAVES;
  constexpr int VPW = VSD ? KPW : (D / 16) / ATT_WAVES;
  constexpr int TILE = ATT_BN * D;
  constexpr int NM = 2 * DB;      // MFMA micro-steps per key tile in pass 2
  constexpr int GPM = 8 / NM < 1 ? 1 : 8 / NM;  // softmax groups (4 scores each) per micro-step
  __shared__ __attribute__((aligned(1024))) uint8_t smem[ATT_NS][2][TILE];
  __shared__ float xch[ATT_WAVES * 32];  // pass 1: the partial row maxima a wave pair exchanges
  uint8_t* const sm = &smem[0][0][0];

  int bh, qt;
  {
    const int id = blockIdx.x, xcd = id & 7, loc = id >> 3;
    const int hl = loc / qtiles;
    qt = loc % qtiles;
    bh = xcd + 8 * hl;
    if (bh >= BH) return;
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q31 = lane & 31, G = lane >> 5;
  const int q0 = qt * ATT_BM + w * 32;
  const bool active = q0 < S;
  const int ntiles = (S + ATT_BN - 1) / ATT_BN;
  const int last = ntiles - 1;
  const bool ragged = (S % ATT_BN) != 0;  // the last key tile is partial

  const uint8_t* Qh = Q + (long)bh * S * D;
  const uint8_t* Kh = Kt + (long)bh * S * D;
  const uint8_t* Vh = Vt + (long)bh * D * S;

  v8i qf[KSTEPS];
  if (MODE == 0) {  // (MODE 1: pass 1 holds the Q fragments of the wave pair; this wave's are among them)
    const int qrow = min(q0 + q31, S - 1);
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) {
      const v4i* p = (const v4i*)(Qh + (long)qrow * D + 64 * t + 32 * G);
      v4i lo = p[0], hi = p[1];
      qf[t] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  }

  // ---- DMA addressing (as in hx_fp8_attention_general's tiles: see att_swz); the destination is a byte offset into the ring
  constexpr int KCPR = D / 16;
  const int k_lrow = lane / KCPR, k_lpos = lane % KCPR;
  const int k_chunk = (k_lpos ^ att_swz<D>(w * KROWS_PER_DMA + k_lrow)) * 16;
  const uint32_t k_vo = (uint32_t)(k_lrow * D + k_chunk);
  const int v_lrow = lane >> 2, v_lpos = lane & 3;
  const int v_chunk = VSD ? (k_lpos ^ att_vswz<D>(w * KROWS_PER_DMA + k_lrow)) * 16 : (v_lpos ^ att_swz<64>(v_lrow)) * 16;
  const uint32_t v_vo = VSD ? (uint32_t)(k_lrow * D + v_chunk) : (uint32_t)(v_lrow * S + v_chunk);
  const uint32_t lds0 = hx_lds_addr(sm);
  // Two forms of every DMA instruction.  Plain: wave-uniform 64-bit base of the tile + a constant per-lane offset
  // (scalar arithmetic only; for the branch-free steps, which never touch a partial tile).  Clamped: the head's base +
  // a per-lane offset computed from the tile index (three vector instructions, no branch); rows (keys) past S re-read
  // row S-1 and, in the [D][S] layout of V, 16-byte column chunks past S re-read the last chunk of the same row
  // (S % 16 == 0 there), so a partial last tile is fetched by the same code as any other.
  auto issue_k_one = [&](int tile, uint32_t dst, int jj, auto clamped) {
    const int j = w + ATT_WAVES * jj;
    if (decltype(clamped)::value) {
      const int row = min(tile * ATT_BN + j * KROWS_PER_DMA + k_lrow, S - 1);
      hx_g2l16_s(Kh, (uint32_t)(row * D + k_chunk), lds0 + dst + j * 1024);
    } else {
      hx_g2l16_s(Kh + ((long)tile * ATT_BN + j * KROWS_PER_DMA) * D, k_vo, lds0 + dst + j * 1024);
    }
  };
  auto issue_v_one = [&](int tile, uint32_t dst, int jj, auto clamped) {
    const int j = w + ATT_WAVES * jj;
    if (decltype(clamped)::value) {
      if (VSD) {
        const int row = min(tile * ATT_BN + j * KROWS_PER_DMA + k_lrow, S - 1);
        hx_g2l16_s(Vh, (uint32_t)(row * D + v_chunk), lds0 + dst + j * 1024);
      } else {
        const int col = min(tile * ATT_BN + v_chunk, S - 16);
        hx_g2l16_s(Vh, (uint32_t)((j * 16 + v_lrow) * S + col), lds0 + dst + j * 1024);
      }
    } else if (VSD) {
      hx_g2l16_s(Vh + ((long)tile * ATT_BN + j * KROWS_PER_DMA) * D, v_vo, lds0 + dst + j * 1024);
    } else {
      hx_g2l16_s(Vh + (long)(j * 16) * S + (long)tile * ATT_BN, v_vo, lds0 + dst + j * 1024);
    }
  };
  auto issue_k = [&](int tile, uint32_t dst) {
#pragma unroll
    for (int jj = 0; jj < KPW; ++jj) issue_k_one(tile, dst, jj, std::true_type{});
  };
  auto issue_v = [&](int tile, uint32_t dst) {
#pragma unroll
    for (int jj = 0; jj < VPW; ++jj) issue_v_one(tile, dst, jj, std::true_type{});
  };

  // pass 2's first tiles, as "virtual steps" -4 .. -1: K(0) | K(1) | K(2), V(0) | K(3), V(1)   (tile indices clamped
  // like in the steps).  Issued as early as the ring is free: at kernel start (MODE 0), or under pass 1's last round.
  auto issue_pass2_prologue = [&]() {
    issue_k(0, 0);
    issue_k(min(1, last), 1 * 2 * TILE);
    issue_k(min(2, last), 2 * 2 * TILE);
    issue_v(0, TILE);
    issue_k(min(3, last), 3 * 2 * TILE);
    issue_v(min(1, last), 1 * 2 * TILE + TILE);
  };

  // ---- fragment addressing: per-lane parts in registers, slot / block parts as immediates
  const int krow = 16 * ((q31 >> 2) & 1) + 4 * (q31 >> 3) + (q31 & 3);
  int k_off[KSTEPS][2];  // key block 0; block 1 is 32 rows further (its swizzle is the same)
#pragma unroll
  for (int t = 0; t < KSTEPS; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) k_off[t][h] = krow * D + (((4 * t + 2 * G + h) ^ att_swz<D>(krow)) * 16);
  int v_off[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) v_off[kb] = q31 * 64 + (((2 * kb + G) ^ att_swz<64>(q31)) * 16);
  int vt_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 32 * (j >> 1) + 16 * G + 8 * (j & 1) + ((lane & 15) >> 1);
    vt_off[j] = row * D + (((((lane >> 4) & 1)) ^ att_vswz<D>(row)) * 16) + (lane & 1) * 8;
  }
  // n-th score MFMA of a tile: key block n % 2, k-step n / 2 (the two MFMAs of a block are never back to back)
  auto load_kfrag = [&](const uint8_t* sk, int n) -> v8i {
    const int kb = n & 1, t = n >> 1;
    v4i lo = *(const v4i*)(sk + kb * 32 * D + k_off[t][0]);
    v4i hi = *(const v4i*)(sk + kb * 32 * D + k_off[t][1]);
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
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
  const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  auto scores_plain = [&](const uint8_t* sk, v16f(&s)[2]) {
    v8i kf[2 * KSTEPS];
#pragma unroll
    for (int n = 0; n < 2 * KSTEPS; ++n) kf[n] = load_kfrag(sk, n);
#pragma unroll
    for (int n = 0; n < 2 * KSTEPS; ++n) s[n & 1] = hx_mfma_32x32x64_e4m3(kf[n], qf[n >> 1], (n >> 1) ? s[n & 1] : zero16);
  };
  // scores of the partial last tile: s[kb][r] belongs to key 64*last + 32*kb + 16*G + r; keys past S -> -inf
  auto mask_last = [&](v16f(&s)[2]) {
    int nv = S - last * ATT_BN - 16 * G;  // this lane's keys 32*kb + r of the tile are valid below nv
    asm volatile("" : "+v"(nv));          // keep the 32 comparisons here, in the one step that needs them
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (32 * kb + r >= nv) s[kb][r] = -__builtin_inff();
  };

  HX_WAIT_VM0();  // the Q loads: the only memory operations the compiler tracks with vmcnt

  float neg_m = __builtin_inff();  // minus the row max in the scaled domain (MODE 0: of the keys seen so far)
  // ================= pass 1 (MODE 1): exact row max of the raw scores.
  // The waves work in pairs: waves 2p and 2p+1 together own 64 queries, and each of them multiplies every other key
  // tile (parity = w & 1) by BOTH query blocks, so a K fragment read from the LDS feeds two MFMAs and the pass reads
  // half the LDS bytes per MFMA of a wave-owns-its-queries scheme (it was bound by those reads, not by the matrix pipe).
  // At the end the two waves of a pair exchange their partial maxima through the LDS.  A score is the same MFMA dot
  // product, k-step order included, whichever wave computes it, so pass 2 reproduces the maximum bit for bit.
  // Tile t sits in slot t % 8 of the ring viewed as eight K slots; one barrier per round of two tiles, with the four
  // tiles of the next two rounds in flight.
  if (MODE == 1) {
    const int pair = w >> 1, par = w & 1;
    const int qp0 = qt * ATT_BM + pair * 64;
    const bool pair_active = qp0 < S;  // wave-uniform
    v8i qp[2][KSTEPS];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int qrow = min(qp0 + 32 * qb + q31, S - 1);
#pragma unroll
      for (int t = 0; t < KSTEPS; ++t) {
        const v4i* pq = (const v4i*)(Qh + (long)qrow * D + 64 * t + 32 * G);
        v4i lo = pq[0], hi = pq[1];
        qp[qb][t] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
    }
    HX_WAIT_VM0();
    float smx[2] = {-__builtin_inff(), -__builtin_inff()};  // per query block: max of this lane's scores so far
    auto kslot = [&](int t) { return (uint32_t)((t & 7) * TILE); };
    const int npro = min(6, ntiles);
    for (int t = 0; t < npro; ++t) issue_k(t, kslot(t));
    constexpr int NF = 2 * KSTEPS;     // K fragments (= MFMAs per query block) per tile
    constexpr int RPF = 32 / NF;       // scores of each query block reduced per fragment step
    // max reduction of part `part` (of NF) of a finished tile's scores, both query blocks
    auto reduce_part = [&](v16f(&cur)[2][2], int part) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int e = part * RPF; e < (part + 1) * RPF; e += 2) smx[qb] = att_max3(smx[qb], cur[qb][e >> 4][e & 15], cur[qb][e >> 4][(e & 15) + 1]);
    };
    // One round: scores of tile `t` (if it exists) into `next` under the max reduction of `cur` (tile tc, if any).
    // A fragment read takes several hundred cycles when the LDS is busy, more than a pair of MFMAs covers, so the
    // four fragments of a tile live in registers and each is refilled with the NEXT round's fragment (tile t + 2) as
    // soon as its two MFMAs are out: by then that tile has landed for every wave (the round's barrier waits for the
    // tiles of two rounds), and the refill has the rest of the round and the barrier to arrive.
    v8i kf[NF];
    // FULL: a round of the steady state - its tile, the tile two ahead and a finished previous tile all exist - so the
    // body has no branch besides the one on pair_active.  (With the guards evaluated at run time a round was two dozen
    // scalar branches, and the pass spent more time fetching instructions than multiplying.)
    auto round = [&](auto full_c, v16f(&cur)[2][2], v16f(&next)[2][2], int t, int tc) __attribute__((always_inline)) {
      constexpr bool FULL = decltype(full_c)::value;
      if (!pair_active) return;
      // (a partial last tile needs no masking here: its rows past S are re-reads of key S-1, whose score is a
      // valid one, so they cannot change the maximum)
      if (FULL || t < ntiles) {
        const bool more = FULL || t + 2 < ntiles;
        const uint8_t* sk2 = sm + kslot(more ? t + 2 : t);  // (no next tile: re-read this one, the values are not used)
#pragma unroll
        for (int n = 0; n < NF; ++n) {
          const int kb = n & 1, ks = n >> 1;
          next[0][kb] = hx_mfma_32x32x64_e4m3(kf[n], qp[0][ks], ks ? next[0][kb] : zero16);
          next[1][kb] = hx_mfma_32x32x64_e4m3(kf[n], qp[1][ks], ks ? next[1][kb] : zero16);
          kf[n] = load_kfrag(sk2, n);
          if (FULL || tc >= 0) reduce_part(cur, n);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else if (tc >= 0) {
#pragma unroll
        for (int n = 0; n < NF; ++n) reduce_part(cur, n);
      }
    };
    v16f ca[2][2], cb[2][2];
    int tc = -1;  // the tile whose scores `cur` holds (-1: none)
    // tiles 0 .. 3 (two rounds' worth) have landed before the first fragments are read
    att_wait_outstanding<KPW>(max(npro - 4, 0));
    __syncthreads();
    if (pair_active) {
#pragma unroll
      for (int n = 0; n < NF; ++n) kf[n] = load_kfrag(sm + kslot(min(par, last)), n);
    }
    const int nrounds = (ntiles + 1) / 2;  // round r: tiles 2r and 2r+1
    // FULL rounds: 1 <= r, tiles 2r+6 and 2r+7 exist and are whole tiles (plain DMA form), so every guard is known
    auto do_round = [&](auto full_c, v16f(&cur)[2][2], v16f(&next)[2][2], int r) __attribute__((always_inline)) {
      constexpr bool FULL = decltype(full_c)::value;
      const int jj = 2 * r;
      // tiles jj .. jj+3 must have landed (this round's and the next round's, whose fragments this round
      // prefetches); tiles jj+4, jj+5 may still be in flight
      if (FULL || jj + 5 <= last) __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(2 * KPW));
      else HX_WAIT_VM0();
      __syncthreads();  // ... for every wave; and every wave is done with tiles jj-2 and jj-1: their slots are free
      if (FULL) {
#pragma unroll
        for (int i = 0; i < KPW; ++i) issue_k_one(jj + 6, kslot(jj + 6), i, std::false_type{});
#pragma unroll
        for (int i = 0; i < KPW; ++i) issue_k_one(jj + 7, kslot(jj + 7), i, std::false_type{});
      } else {
        if (jj + 6 < ntiles) issue_k(jj + 6, kslot(jj + 6));
        if (jj + 7 < ntiles) issue_k(jj + 7, kslot(jj + 7));
        // The last round multiplies out of registers (what its refills read is not used), and every wave has finished
        // its real fragment reads before this round's barrier: the whole ring is free, and pass 2's first tiles go out
        // now instead of after the pass.
        if (r == nrounds - 1) issue_pass2_prologue();
      }
      const int t = jj + par;
      round(full_c, cur, next, t, tc);
      tc = (FULL || t < ntiles) ? t : -1;
    };
    // Even rounds read ca and write cb, odd rounds the other way round, so rounds come in pairs; three loops one after
    // the other, each with its two rounds written out (a run-time choice between the guarded and the branch-free pair
    // inside one loop makes the compiler shuffle the 128 accumulator registers where the two paths meet, through scratch).
    const int r_full = last >= 8 ? (last - 8) / 2 : -1;  // the last round whose tiles 2r+6, 2r+7 lie before the last tile
    int r = 0;
    for (; r < 2 && r < nrounds; r += 2) {  // the first pair: no finished tile yet
      do_round(std::false_type{}, ca, cb, r);
      if (r + 1 < nrounds) do_round(std::false_type{}, cb, ca, r + 1);
    }
    for (; r + 1 <= r_full; r += 2) {
      do_round(std::true_type{}, ca, cb, r);
      do_round(std::true_type{}, cb, ca, r + 1);
    }
    for (; r < nrounds; r += 2) {
      do_round(std::false_type{}, ca, cb, r);
      if (r + 1 < nrounds) do_round(std::false_type{}, cb, ca, r + 1);
    }
    if (pair_active && tc >= 0) {  // the last tile's scores: round r wrote cb when r is even, ca when it is odd
      if ((nrounds - 1) & 1) {
#pragma unroll
        for (int n = 0; n < NF; ++n) reduce_part(ca, n);
      } else {
#pragma unroll
        for (int n = 0; n < NF; ++n) reduce_part(cb, n);
      }
    }
    const float m_own = att_max_across_halves(smx[par]);        // this wave's queries, its parity's tiles
    const float m_give = att_max_across_halves(smx[par ^ 1]);   // the partner's queries, this wave's tiles
    if (lane < 32) xch[w * 32 + lane] = m_give;
    __syncthreads();
    const float smax = fmaxf(m_own, xch[(w ^ 1) * 32 + q31]);
    neg_m = -(smax * c);  // max(s*c) == max(s)*c for c > 0 (rounding is monotone)
    // this wave's own 32 queries are block `par` of the pair's 64
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[t][e] = par ? qp[1][t][e] : qp[0][t][e];
  }

  // ================= pass 2 (MODE 0: the only pass)
  v16f o[DB];
#pragma unroll
  for (int d = 0; d < DB; ++d) o[d] = zero16;
  float l4[4] = {0.f, 0.f, 0.f, 0.f};  // four independent partial sums of the un-quantised p per lane

  // softmax group g of a tile: scores cur[g / 4][4 * (g % 4) .. + 3] -> dword g of the P fragment
  auto softmax_group = [&](v16f(&cur)[2], v8i& pf_new, int g) {
    const int kb = g >> 2, r0 = 4 * (g & 3);
    float p[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      // s*c - m fused into one rounding: the score already carries the fp8 MFMA's accumulation rounding, three orders
      // of magnitude above the difference between one and two roundings here
      p[b] = __builtin_amdgcn_exp2f(__builtin_fmaf(cur[kb][r0 + b], c, neg_m));
      l4[b] += p[b];
    }
    const int dw = HX_CVT_PK_E4M3(p[0], p[1], pf_new[g], false);
    pf_new[g] = HX_CVT_PK_E4M3(p[2], p[3], dw, true);
  };

  // step j: scores of tile j+1 -> next; softmax of tile j (cur) -> pf_new; P.V of tile j-1 (pf_prev)
  auto step = [&](auto slot_c, auto full_c, v16f(&cur)[2], v16f(&next)[2], v8i& pf_prev, v8i& pf_new, int j) {
    constexpr int SL = decltype(slot_c)::value;    // == j % 4
    constexpr bool FULL = decltype(full_c)::value;  // all three parts present, no partial tile involved: no branches
    const bool has_s = FULL || j + 1 < ntiles, has_sm = FULL || j < ntiles, has_pv = FULL || j >= 1;
    // DMA issued in steps j-2 and j-1 may stay in flight; everything older (K(j+1), V(j-1) included) has landed.
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(2 * (KPW + VPW)));
    __syncthreads();
    const int tk = min(j + 4, last), tv = min(j + 2, last);
    const uint8_t* sk = sm + ((SL + 1) & 3) * 2 * TILE;         // K(j+1)
    const uint8_t* sv = sm + ((SL + 3) & 3) * 2 * TILE + TILE;  // V(j-1)
    constexpr uint32_t kdst = SL * 2 * TILE;                    // K(j+4) replaces K(j)
    constexpr uint32_t vdst = ((SL + 2) & 3) * 2 * TILE + TILE;  // V(j+2) replaces V(j-2)
    if (active) {
      v8i kf[2], vf[2];
      if (has_pv) {
        vf[0] = load_vfrag(sv, 0);
        vf[1] = load_vfrag(sv, 1);
      }
      if (has_s) {
        kf[0] = load_kfrag(sk, 0);
        kf[1] = load_kfrag(sk, 1);
      }
      __builtin_amdgcn_sched_barrier(0);
      float alpha = 1.f;
      bool rescale = false;
      if (!FULL && ragged && j == last) mask_last(cur);
      float t0 = -__builtin_inff(), t1 = -__builtin_inff();  // MODE 0: the tile's row max, one chain per key block
      auto tile_max_half = [&](int kb) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          if (kb == 0) t0 = att_max3(t0, cur[0][r], cur[0][r + 1]);
          else t1 = att_max3(t1, cur[1][r], cur[1][r + 1]);
        }
      };
      // MODE 0: new reference point and the factor the older sums shrink by (first tile: exp2(-inf) = 0 on zeros)
      auto new_reference = [&]() {
        const float tmax = att_max_across_halves(fmaxf(t0, t1));
        const float neg_new = fminf(neg_m, -(tmax * c));
        alpha = __builtin_amdgcn_exp2f(neg_new - neg_m);
        rescale = __builtin_amdgcn_ballot_w64(neg_new != neg_m) != 0;  // wave-uniform: most tiles leave every row max alone
        neg_m = neg_new;
#pragma unroll
        for (int i = 0; i < 4; ++i) l4[i] *= alpha;
      };
      // MODE 1: the first softmax groups cover the latency of the fragment reads above.  MODE 0: the first half of
      // the max reduction does; the second half and the new reference follow the first MFMA, the groups start one
      // micro-step later and the last micro-step takes what is left.
      constexpr int GSH = MODE == 0 ? 1 : 0;  // micro-steps the groups are delayed by
      if (has_sm) {
        if (MODE == 0) {
          tile_max_half(0);
        } else {
#pragma unroll
          for (int g = 0; g < GPM; ++g) softmax_group(cur, pf_new, g);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < NM; ++i) {
        const int h = i >> 1;
        if ((i & 1) == 0) {
          if (has_pv) {
            o[h] = hx_mfma_32x32x64_e4m3(vf[h & 1], pf_prev, o[h]);
            if (h + 2 < DB) vf[h & 1] = load_vfrag(sv, h + 2);
          }
        } else {
          if (has_s) {
            next[h & 1] = hx_mfma_32x32x64_e4m3(kf[h & 1], qf[h >> 1], (h >> 1) ? next[h & 1] : zero16);
            if (h + 2 < DB) kf[h & 1] = load_kfrag(sk, h + 2);
          }
        }
        if (has_sm) {
          if (MODE == 0 && i == 0) {
            tile_max_half(1);
            new_reference();
          } else {
            const int g_lo = MODE == 0 ? (i - GSH) * GPM : (i + 1) * GPM;
            const int g_hi = (MODE == 0 && i == NM - 1) ? 8 : g_lo + GPM;
#pragma unroll
            for (int g = g_lo; g < g_hi && g < 8; ++g) softmax_group(cur, pf_new, g);
          }
        }
        // this step's DMA, one instruction per micro-step
        if (i < KPW) issue_k_one(tk, kdst, i, std::bool_constant<!FULL>{});
        else if (i < KPW + VPW) issue_v_one(tv, vdst, i - KPW, std::bool_constant<!FULL>{});
        __builtin_amdgcn_sched_barrier(0);
      }
      // MODE 0: the sums of the older tiles (P.V of tile j-1 included: it was quantised against the old reference)
      // shrink by alpha before tile j's P.V is added in the next step
      if (MODE == 0 && rescale) {
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
      }
    } else {
      issue_k(tk, kdst);
      issue_v(tv, vdst);
    }
  };

  if (MODE == 0) issue_pass2_prologue();  // (MODE 1: went out under pass 1's last round)
  __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(3 * KPW + 2 * VPW));  // K(0) has landed
  __syncthreads();
  v16f sa[2], sb[2];
  v8i pfA = {0, 0, 0, 0, 0, 0, 0, 0}, pfB = {0, 0, 0, 0, 0, 0, 0, 0};
  if (active) scores_plain(sm, sa);
  {
    using std::integral_constant;
    const integral_constant<int, 0> s0;
    const integral_constant<int, 1> s1;
    const integral_constant<int, 2> s2;
    const integral_constant<int, 3> s3;
    // Steps 0 .. ntiles.  Steps 1 .. ntiles-2 have all three parts and run the branch-free body, four at a time
    // (slots 1, 2, 3, 0) -- with a partial last tile only up to step ntiles-6, so that neither its masking nor its
    // DMA ever comes up there; the first step and whatever is left at the end run the guarded body.
    const int full_to = ragged ? ntiles - 6 : ntiles - 2;
    step(s0, std::false_type{}, sa, sb, pfA, pfB, 0);
    int j = 1;
    for (; j + 3 <= full_to; j += 4) {
      step(s1, std::true_type{}, sb, sa, pfB, pfA, j);
      step(s2, std::true_type{}, sa, sb, pfA, pfB, j + 1);
      step(s3, std::true_type{}, sb, sa, pfB, pfA, j + 2);
      step(s0, std::true_type{}, sa, sb, pfA, pfB, j + 3);
    }
    for (; j <= ntiles; j += 4) {  // j % 4 == 1 here
      step(s1, std::false_type{}, sb, sa, pfB, pfA, j);
      if (j + 1 <= ntiles) step(s2, std::false_type{}, sa, sb, pfA, pfB, j + 1);
      if (j + 2 <= ntiles) step(s3, std::false_type{}, sb, sa, pfB, pfA, j + 2);
      if (j + 3 <= ntiles) step(s0, std::false_type{}, sa, sb, pfA, pfB, j + 3);
    }
  }
  const float l_lane = (l4[0] + l4[1]) + (l4[2] + l4[3]);
  const float l = l_lane + __shfl_xor(l_lane, 32);

  HX_WAIT_VM0();     // the trailing re-fetches have landed ...
  __syncthreads();  // ... and every wave is past its last fragment read: the ring can be reused
  if (!active) return;
  // ---------------- epilogue: o[db][4a+b] is O[q0 + lane%32][32 db + 8a + 4G + b]
  // A lane holds 4 consecutive columns of its row, so direct stores would write every output line in 16- or
  // 32-byte pieces.  Each wave instead passes its 32 rows through its own part of the LDS, PASS_COLS columns at a
  // time, and writes 16 bytes per lane with consecutive lanes on consecutive bytes of a row.
  constexpr int ESZ = OUT == HX_F32 ? 4 : 1;
  constexpr int PASS_COLS = OUT == HX_F32 ? D / 2 : D;  // 256 or 128 bytes of a row per pass (128 or 64 for D = 64)
  constexpr int PASS_BYTES = PASS_COLS * ESZ;
  constexpr int RSTR = PASS_BYTES + 16;                 // padded row stride
  constexpr int LPR = PASS_BYTES / 16;                  // lanes per row on the way out
  constexpr int RPI = 64 / LPR;                         // rows per store instruction
  constexpr int NDB = PASS_COLS / 32;                   // 32-column accumulator blocks per pass
  static_assert(ATT_WAVES * 32 * RSTR <= ATT_NS * 2 * TILE, "output staging fits the K/V ring");
  uint8_t* st = sm + w * (32 * RSTR);
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
      // (non-temporal: at 256 MB of fp32 output per C4 launch, written once, the lines should not linger in the L2s that
      // hold the heads' K and V: online mode -3.5 %, exact mode +-0)
      if (q0 + row < S) __builtin_nontemporal_store(v, (v4i*)(out_rows + ((long)row * D + h * PASS_COLS) * ESZ + rb_ch * 16));
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

template <int D, int OUT, int MODE, bool VSD>
static void launch_att_pipe(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, float c, hipStream_t s) {
  const int qtiles = (int)((S + ATT_BM - 1) / ATT_BM);
  const int hpx = (int)((BH + 7) / 8);
  const int grid = 8 * hpx * qtiles;
  hx_launch((hx_fp8_attention_pipe<D, OUT, MODE, VSD>), dim3(grid), dim3(256), 0, s, (const uint8_t*)q, (const uint8_t*)k,
            (const uint8_t*)v, out, (int)S, (int)BH, qtiles, c);
}

template <int D, int OUT>
static int launch_att(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, int exact, bool vsd, float c, hipStream_t s) {
  if (exact) {
    if (vsd) launch_att_pipe<D, OUT, 1, true>(q, k, v, out, BH, S, c, s);
    else launch_att_pipe<D, OUT, 1, false>(q, k, v, out, BH, S, c, s);
  } else {
    if (vsd) launch_att_pipe<D, OUT, 0, true>(q, k, v, out, BH, S, c, s);
    else launch_att_pipe<D, OUT, 0, false>(q, k, v, out, BH, S, c, s);
  }
  hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_fp8_attention: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

// 1: the MFMA kernel takes these arguments; 0: the plain kernel does.  vsd: V is [S][D] per head.
static bool att_fast_path(const void* q, const void* k, const void* v, const void* out, int64_t S, int64_t D, int64_t v_stride_d,
                          int64_t v_stride_s, bool* vsd) {
  bool fast = (D == 64 || D == 128 || (D == 256 && hx_feature(HX_FEATURE_ATTENTION_D256))) && S >= 1 && ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) == 0);
  *vsd = false;
  if (v_stride_s == 1 && (v_stride_d == S || D == 1)) {
    *vsd = false;                                  // [D][S] per head: rows of S bytes, fetched in 16-byte pieces
    if (S % 16 != 0) fast = false;
  } else if (v_stride_d == 1 && (v_stride_s == D || S == 1)) {
    *vsd = true;                                   // [S][D] per head
  } else {
    fast = false;
  }
  return fast;
}

extern "C" int hx_fp8_attention_path(int64_t BH, int64_t S, int64_t D, int64_t v_stride_d, int64_t v_stride_s, const void* q,
                                     const void* k, const void* v, const void* out) {
  bool vsd;
  (void)BH;
  return att_fast_path(q, k, v, out, S, D, v_stride_d, v_stride_s, &vsd) ? 1 : 0;
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
  bool vsd = false;
  const bool fast = att_fast_path(q, k, v, out, S, D, v_stride_d, v_stride_s, &vsd);
  if (!fast) {  // any other shape, alignment or V striding within a head (heads are D*S elements apart)
    if (D > 256 || D < 1 || BH >= 65536) {
      hx_set_error("hx_fp8_attention: unsupported shape S=%lld D=%lld BH=%lld (MFMA kernel: D in {64,128}, 16-byte aligned pointers, v as [D][S] with S %% 16 == 0 or as [S][D]; plain kernel: D <= 256, BH < 65536)",
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
  if (D == 256) {
    if (out_dtype == HX_F32) return launch_att<256, HX_F32>(q, k, v, out, BH, S, exact_max, vsd, c, s);
    return launch_att<256, HX_E4M3>(q, k, v, out, BH, S, exact_max, vsd, c, s);
  }
  if (out_dtype == HX_F32) return launch_att<64, HX_F32>(q, k, v, out, BH, S, exact_max, vsd, c, s);
  return launch_att<64, HX_E4M3>(q, k, v, out, BH, S, exact_max, vsd, c, s);
}
