// hx_gemm16_tile256p: the 256x256x64 16-bit tile kernel - grouped (MoE) or dense - as a persistent workgroup (opt-in,
// HX_FEATURE_MOE_PERSISTENT / HX_FEATURE_MATMUL_PERSISTENT; not yet run on the hardware).  Same tile, LDS layout, fragment scheme, k-tile schedule and
// MFMA order per accumulator as hx_gemm16_tile256<BF, 0> (results bit-equal); what changes is what happens between two
// tiles of one workgroup, as in hx_fp8_gemm_tile256p:
//
//   * the k-tile pipeline does not stop at a tile's end: the last two k-tiles of a tile issue the DMA of the next tile's
//     first two (the number of k-tiles is even, so the stages keep their parity), and the refills of the last k-tile fetch
//     the next tile's first fragments.  The prologue - two k-tiles of DMA latency - is paid once per workgroup;
//   * the epilogue of tile T runs INSIDE the first half of tile T+1's first k-tile.  That half touches every accumulator
//     block exactly once (one 16x16x32 MFMA per block) and may do so in any order, with a zero C operand instead of the old
//     accumulator.  So the accumulators are handed over in eight groups of 16 rows: group g is converted and written to the
//     wave's staging block in the LDS, then the 8 MFMAs of the new tile that overwrite exactly those blocks are issued, then
//     the staged rows are read back as whole 256-byte row pieces and stored while the matrix pipe works;
//   * the row gather needs no global load inside the loop (a load the compiler waits for would also wait for every DMA in
//     flight): the rows of the NEXT tile come in by one 4-byte DMA instruction per wave at the start of a tile, into one of
//     three row tables in the LDS (previous tile: being stored; this tile; next tile), and the gather offsets are recomputed
//     from the table just before the next tile's first DMA;
//   * every wave issues the same number of vector-memory instructions per tile whatever the tile holds, because the waits
//     are counted: rows that are not stored (padding of an expert's last tile, malformed row ids) send their 16 bytes to a
//     per-lane slot of a 1 KB sink in the workspace instead of being skipped.
// Waits: the hand-over's half issues 16 DMA instructions and 32 stores after the ones the next wait is for, so that wait
// lets 48 fly; the one after lets 20 (16 DMA + the last group's 4 stores); all others are the plain kernel's 16.
// Tiles: at step s the workgroups process tiles s*G .. s*G + G-1 of the grouped raster (G = grid size, a multiple of 8),
// XCD x (= blockIdx % 8) the G/8 consecutive ones starting at s*G + x*G/8 - the order the plain kernel's launch gives.
#pragma once
#include "gemm16_tile256.h"

#define G16P_STG_BYTES (16 * 256)  // one wave's staging block: 16 rows x 128 columns of a 16-bit type
#define G16P_SINK_BYTES 1024       // 64 lanes x 16 bytes

// K % 128 == 0 and K >= 256 (an even number of k-tiles, at least four), N % 256 == 0 (the host checks).
// sink: G16P_SINK_BYTES of device memory, 16-byte aligned, written and never read.
// DENSE: C = A @ W without the tile table and the row list: row tile t covers rows 256 t .. of A and C, T % 256 == 0 (no row
// is ever left out, so the sink is not used), tiles_m row tiles; the row tables are filled by the waves themselves.
// lda, ldb, ldc: row strides of A, W and C in elements (grouped: K, N, N).
template <bool BF, bool DENSE>
__global__ __launch_bounds__(256) void hx_gemm16_tile256p(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                                                         void* __restrict__ Cv, const int* __restrict__ num_tiles,
                                                         const MoeTile* __restrict__ table, const int32_t* __restrict__ idx, int T,
                                                         int K, int N, int tiles_n, int a_div, uint8_t* __restrict__ sink, long lda,
                                                         long ldb, long ldc, int tiles_m) {
  typedef typename Mfma16<BF>::T out_t;
  typedef typename Mfma16<BF>::V8 V8;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2][2][MOE_TILE_BYTES];  // [stage][A|W][32 KB]
  __shared__ __attribute__((aligned(1024))) uint8_t stg[4][G16P_STG_BYTES];
  __shared__ __attribute__((aligned(1024))) int rowtab[3][256];  // matrix rows of a tile's 256 rows (as idx holds them)

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w >> 1, wn = w & 1;
  const int nk = K / MOE_BK;
  const long ldb2 = ldb * 2, lda2 = lda * 2, ldc2 = ldc * 2;  // row strides in bytes

  // ---- this workgroup's tiles
  const int nrt = DENSE ? tiles_m : *num_tiles, total = nrt * tiles_n;
  const int G = (int)gridDim.x, b = (int)blockIdx.x, cpx = G >> 3;
  auto tile_of = [&](int s) {  // tile of step s, or -1
    const int base = s * G, R = total - base;
    if (R >= G) return base + (b & 7) * cpx + (b >> 3);
    if (R <= 0) return -1;
    if ((R & 7) == 0) return (b >> 3) < (R >> 3) ? base + (b & 7) * (R >> 3) + (b >> 3) : -1;
    return b < R ? base + b : -1;
  };
  const int nfull = total / G;
  const int nt = nfull + (tile_of(nfull) >= 0 ? 1 : 0);
  if (nt == 0) return;  // (whole workgroup)
  // tile -> row tile's table entry and column tile (grouped raster, 4 row tiles tall, as the plain kernel)
  auto tile_info = [&](int tile, MoeTile& mt, int& tn) {
    const int GM = 4, group_size = GM * tiles_n, first_m = (tile / group_size) * GM;
    const int gm = min(nrt - first_m, GM);
    const int tm = first_m + (tile % group_size) % gm;
    if (DENSE) mt.expert = 0, mt.row_start = tm * MOE_BM, mt.rows = min(MOE_BM, T - tm * MOE_BM), mt.pad = 0;
    else mt = table[tm];
    tn = (tile % group_size) / gm;
  };

  // ---- A DMA: wave w owns tile rows [64w, 64w+64), 8 instructions of 8 rows, gathered: the per-lane offset carries the row
  const int lrow = lane >> 3, lpos = lane & 7;
  uint32_t a_vo[8];
  auto set_avo = [&](int slot, int rows) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      int lr = w * 64 + j * 8 + lrow;
      lr = lr < rows ? lr : 0;  // padded rows re-read row 0 of the tile; never stored
      int r = rowtab[slot][lr];
      r = (r >= 0 && r < T) ? r : 0;
      const int swz = ((j & 1) ? 4 + (lrow >> 1) : (lrow >> 1)) & 7;
      if (a_div != 1) r /= a_div;  // (wave-uniform; top-k routing without a replicated A: C row r is the product of A row r / a_div)
      a_vo[j] = (uint32_t)r * (uint32_t)lda2 + (uint32_t)((lpos ^ swz) * 16);
    }
  };
  // the rows of a tile -> row table `slot`, this wave's 64 of them by one 4-byte DMA instruction (entries past the end of
  // idx re-read its last one; they belong to rows past the tile's count, which are masked wherever the table is read)
  auto fetch_rows = [&](int row_start, int slot) {
    if (DENSE) rowtab[slot][w * 64 + lane] = row_start + w * 64 + lane;
    else hx_g2l4_s(idx, (uint32_t)min(row_start + w * 64 + lane, T - 1) * 4u, hx_lds_addr(&rowtab[slot][w * 64]));
  };
  // ---- W DMA: wave w owns k rows [16w, 16w+16), 8 instructions of 2 rows x 512 B (N % 256 == 0: no ragged column tile)
  const int wk_l = lane >> 5, wpos = lane & 31;
  uint32_t w_vo[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) w_vo[j] = (uint32_t)(wk_l * ldb2 + (wpos ^ (moe_wswz(2 * j + wk_l) << 1)) * 16);
  const uint32_t lds0 = hx_lds_addr(&smem[0][0][0]);
  // DMA instruction i (0..15) of the k-tile whose A bytes start at column ak of A and whose W rows start at wk (wave-uniform)
  auto issue_one = [&](long ak, const uint8_t* wk, int stage, int i) {
    const uint32_t la = lds0 + (uint32_t)stage * 2 * MOE_TILE_BYTES + (uint32_t)w * 64 * 128;
    const uint32_t lw = lds0 + (uint32_t)stage * 2 * MOE_TILE_BYTES + MOE_TILE_BYTES + (uint32_t)w * 16 * 512;
    if (i < 8) hx_g2l16_s(A + ak, a_vo[i], la + i * 1024);
    else hx_g2l16_s(wk + (long)(2 * (i - 8)) * ldb2, w_vo[i - 8], lw + (i - 8) * 1024);
  };
  // W rows of k-tile kt of the tile (expert e, column tile tn), this wave's part
  auto w_rows = [&](int e, int tn, int kt) {
    return hx_uniform_ptr(W + (long)e * K * ldb2 + (long)tn * (MOE_BN * 2) + ((long)kt * MOE_BK + w * 16) * ldb2);
  };

  // ---- operand addressing (as in hx_gemm16_tile256)
  const int r16 = lane & 15, g = lane >> 4;
  const int ax = (g ^ ((r16 >> 1) & 7)) * 16;
  const int a_base = (wm * 128 + r16) * 128;
  const int te = (lane >> 2) & 3, tq = lane & 3;
  const int tn_ = wn * 128 + 4 * tq;
  int w_off[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int k = 8 * g + te + 4 * half;
    w_off[half] = k * 512 + (((tn_ >> 3) ^ (moe_wswz(k) << 1)) * 16) + (tn_ & 7) * 2;
  }
  v4f acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  V8 fa[2][8], fw[2][8];  // [k-step][row block], [k-step][column block]
  auto load_frag = [&](int stage, int ks, int f) {
    if (f < 8) {
      fa[ks][f] = *(const V8*)(&smem[stage][0][0] + a_base + f * 2048 + (ax ^ (ks * 64)));
    } else {
      const uint8_t* sw = &smem[stage][1][0];
      v4s part[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int off = (w_off[half] ^ ((f - 8) * 32)) + ks * 16384;
        part[half] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3)))*)(sw + off));
      }
      v8s both = (v8s){part[0][0], part[0][1], part[0][2], part[0][3], part[1][0], part[1][1], part[1][2], part[1][3]};
      fw[ks][f - 8] = __builtin_bit_cast(V8, both);
    }
  };
  // second half of any k-tile: 64 MFMAs of k-step 1 and the refill of all 32 fragments from the other stage
  auto second_half = [&](int stage) {
    HX_OPAQUE_S(stage);  // (every k-tile computes its fragment addresses from the stage it is given, at run time)
#pragma unroll
    for (int i = 0; i < 64; ++i) {
      Mfma16<BF>::acc16(acc[i >> 3][i & 7], fw[1][i >> 3], fa[1][i & 7]);
      if (i < 32 && !(i & 1)) load_frag(stage ^ 1, 0, i >> 1);
      if ((i & 7) == 7) load_frag(stage ^ 1, 1, 8 + (i >> 3));
      if (i >= 56) load_frag(stage ^ 1, 1, i - 56);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();  // every wave has read the next k-tile's fragments out of the other stage: it is free
  };
  // one ordinary k-tile: 64 MFMAs of k-step 0 with the 16 DMA instructions of the k-tile two ahead (at ak / wk, which may
  // belong to the next tile) into this k-tile's own stage, the counted wait for the k-tile one ahead, a barrier, the second half
  auto ktile = [&](int stage, long ak, const uint8_t* wk, auto keep_c) {
    HX_OPAQUE_S(stage);
#pragma unroll
    for (int i = 0; i < 64; ++i) {
      Mfma16<BF>::acc16(acc[i >> 3][i & 7], fw[0][i >> 3], fa[0][i & 7]);
      if ((i & 3) == 3) issue_one(ak, wk, stage, i >> 2);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(decltype(keep_c)::value));
    __syncthreads();
    second_half(stage);
  };

  // ---- the epilogue's two halves for one group of 16 rows (accumulator blocks bi = grp, all bj).
  // Everything a lane needs for them hangs off six lane constants, re-derived from `lane` at the top of every tile behind
  // an empty instruction the compiler cannot see through (HX_OPAQUE_V): otherwise it computes the ~100 addresses and row numbers of the eight
  // groups once, before the tile loop, and keeps them in scratch memory - and a reload from scratch makes it wait for
  // every vector-memory operation in flight, the DMA included.
  out_t* C = (out_t*)Cv;
  typedef out_t ov4 __attribute__((ext_vector_type(4)));
  struct Lanes {
    uint32_t st_w;   // staging, on the way in: row r16, byte (g & 1) * 8 of chunk 0
    uint32_t x0;     // (g >> 1) ^ r16: chunk 2 bj + (g >> 1) of row r16 sits at position (x0 ^ 2 bj)
    uint32_t st_r;   // staging, on the way out: row rb_row (16 lanes per row, 4 rows per store instruction)
    uint32_t y0;     // rb_ch ^ rb_row: chunk rb_ch of row 4p + rb_row sits at position (y0 ^ 4p)
    uint32_t rb_row, rb16;  // lane / 16; (lane % 16) * 16 = byte of the lane's 8 columns in a 256-byte row piece
  };
  auto lanes_now = [&]() {
    int l = lane;
    HX_OPAQUE_V(l);
    const uint32_t r = l & 15, q = l >> 4, stb = (uint32_t)w * G16P_STG_BYTES;  // (byte offsets into stg)
    Lanes L;
    L.st_w = stb + r * 256 + (q & 1) * 8, L.x0 = (q >> 1) ^ r;
    L.st_r = stb + q * 256, L.y0 = r ^ q, L.rb_row = q, L.rb16 = r * 16;
    return L;
  };
  auto stage_rows = [&](const Lanes& L, int grp) {
#pragma unroll
    for (int bj = 0; bj < 8; ++bj) {
      ov4 o;
#pragma unroll
      for (int q = 0; q < 4; ++q) o[q] = (out_t)hx_acc_read(acc[bj][grp][q]);
      // row r16 of the group; columns 16 bj + 4 g .. + 3 = bytes 32 bj + 8 g .. + 7; chunk c of row r sits at c ^ r
      *(ov4*)(&stg[0][0] + L.st_w + ((L.x0 ^ (2 * bj)) * 16)) = o;
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // tab: this lane's entry of the row table of the tile being stored, &rowtab[slot][wm * 128 + rb_row]; rows: its row count
  auto drain = [&](const Lanes& L, int grp, const int* tab, int rows, const uint8_t* cbase) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int r = tab[grp * 16 + p * 4];
      const v4i v = *(const v4i*)(&stg[0][0] + L.st_r + p * 1024 + ((L.y0 ^ (4 * p)) * 16));
      const bool ok = (int)L.rb_row < rows - (wm * 128 + grp * 16 + p * 4) && r >= 0 && r < T;
      const uint8_t* dst = cbase + (long)r * ldc2 + L.rb16;
      // (non-temporal, as in the plain kernel; rows that are not stored go to the sink so that the instruction is issued anyway)
      __builtin_nontemporal_store(v, (v4i*)(ok ? dst : (const uint8_t*)sink + (L.rb_row * 16 + (L.rb16 >> 4)) * 16));
      if (p & 1) __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto tab_of = [&](const Lanes& L, int slot) { return (const int*)&rowtab[slot][wm * 128] + L.rb_row; };
  auto cbase_of = [&](long n0) { return (const uint8_t*)(C + n0 + wn * 128); };

  // ---- prologue, once per workgroup: the first tile's rows, its k-tiles 0 and 1, the fragments of k-tile 0
  MoeTile mt;
  int tn;
  tile_info(tile_of(0), mt, tn);
  fetch_rows(mt.row_start, 0);
  HX_WAIT_VM0();
  __syncthreads();
  set_avo(0, mt.rows);
#pragma unroll
  for (int i = 0; i < 16; ++i) issue_one(0, w_rows(mt.expert, tn, 0), 0, i);
#pragma unroll
  for (int i = 0; i < 16; ++i) issue_one(128, w_rows(mt.expert, tn, 1), 1, i);
  __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(16));
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int f = 0; f < 16; ++f) load_frag(0, ks, f);
  __syncthreads();

  // Every tile runs the same code, so that the accumulators keep their registers from one tile to the next: k-tile 0 as a
  // hand-over - of the previous tile's accumulators, or, for the workgroup's first tile, of the zeros the accumulators start
  // with, which go to the tile's own (not yet written) rows of C and are overwritten by its real values later - then
  // k-tiles 1 .. nk-1.
  int slot = 0;                                            // row table of this tile
  int pslot = 0, prows = mt.rows;                          // ... and of the tile whose accumulators the next hand-over stores
  long pn0 = (long)tn * MOE_BN;
  for (int ti = 0; ti < nt; ++ti) {
    // the next tile, or (last tile) this tile again: then the last two k-tiles re-fetch this tile's last k-tile into stages
    // nobody reads any more, so that every k-tile issues its 16 DMA instructions and the waits stay constant
    const bool has_next = ti + 1 < nt;
    MoeTile mn = mt;
    int tnn = tn;
    if (has_next) tile_info(tile_of(ti + 1), mn, tnn);
    const int nslot = slot == 2 ? 0 : slot + 1;
    fetch_rows(mn.row_start, nslot);
    const int e = mt.expert;

    // ---- hand-over = first half of k-tile 0 (its fragments are in registers; stage 0, which held them, takes k-tile 2)
    {
      const Lanes L = lanes_now();
      const int* tab = tab_of(L, pslot);
      const uint8_t* cb = cbase_of(pn0);
      const uint8_t* wk2 = w_rows(e, tn, 2);
#pragma unroll
      for (int grp = 0; grp < 8; ++grp) {
        stage_rows(L, grp);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
        for (int bj = 0; bj < 8; ++bj) {
          Mfma16<BF>::overwrite16(acc[bj][grp], fw[0][bj], fa[0][grp]);
          if ((bj & 3) == 3) issue_one(2L * 128, wk2, 0, 2 * grp + (bj >> 2));
          __builtin_amdgcn_sched_barrier(0);
        }
        drain(L, grp, tab, prows, cb);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
    }
    // k-tile 1 and the next tile's rows (issued before this half) have landed; this half's 16 DMA instructions and 32 stores may fly
    __builtin_amdgcn_s_waitcnt(hx_vmcnt_imm(48));
    __syncthreads();
    second_half(0);

    // ---- k-tiles 1 .. nk-1
    ktile(1, 3L * 128, w_rows(e, tn, 3), std::integral_constant<int, 20>{});  // (the last group's 4 stores are newer than k-tile 2's DMA)
    for (int kt = 2; kt + 2 < nk; ++kt) ktile(kt & 1, (long)(kt + 2) * 128, w_rows(e, tn, kt + 2), std::integral_constant<int, 16>{});
    // from here on the DMA belongs to the next tile: its gather offsets (this tile's again if there is none)
    set_avo(has_next ? nslot : slot, has_next ? mn.rows : mt.rows);
    const int k0 = has_next ? 0 : nk - 1, k1 = has_next ? 1 : nk - 1;
    ktile(0, (long)k0 * 128, w_rows(mn.expert, tnn, k0), std::integral_constant<int, 16>{});  // kt = nk - 2
    ktile(1, (long)k1 * 128, w_rows(mn.expert, tnn, k1), std::integral_constant<int, 16>{});  // kt = nk - 1
    pslot = slot, prows = mt.rows, pn0 = (long)tn * MOE_BN;
    if (has_next) slot = nslot;
    mt = mn, tn = tnn;
  }

  // ---- the workgroup's last tile: nothing left to overlap the epilogue with
  HX_WAIT_VM0();  // the trailing re-fetches
  const Lanes L = lanes_now();
#pragma unroll
  for (int grp = 0; grp < 8; ++grp) {
    stage_rows(L, grp);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    drain(L, grp, tab_of(L, pslot), prows, cbase_of(pn0));
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}
