// Routing tables for the MoE grouped GEMM, built on the device — replaces the torch ops of
// moe_matmul_ogs_helion_kernel_args_gen (examples/moe_matmul_ogs.py:84-121 of the reference):
//   idx     = argsort(expert_ids, stable=True)        (int32 [T])
//   counts  = bincount(expert_ids, minlength=E)       (int32 [E])
//   offsets = [0, cumsum(counts)]                     (int32 [E+1])
//   max_count = max(counts)                           (int32 [1], stays on the device: no host sync)
// Workgroups of 16 waves; every wave owns a contiguous block of rows, so a stable order is "by expert, then by
// (workgroup, wave), then by position in the wave's block".  A count pass finds the rows per (wave, expert); a
// scan over (expert-major, wave-minor) turns the counts into each wave's first output slot per expert; a scatter
// pass walks the rows again.  Up to 32768 rows one workgroup does all of it in one launch; above that the count
// pass, a one-workgroup scan over the per-workgroup counts and the scatter pass are three launches.  Inside a
// 64-row group the lanes that hold the same expert find each other with one ballot per bit of the expert id, so
// neither pass needs atomics and the result is deterministic.  Ids outside [0, E) are skipped (their rows appear in no expert's list).
#include "hx_common.h"

#define RT_WAVES 16
#define RT_MAX_E 512        // experts of the default instantiation (32 KB of per-wave counters)
#define RT_MAX_E_WIDE 2048  // opt-in (HX_FEATURE_ROUTING_WIDE): 128 KB of per-wave counters, two experts per work-item in the scans
#define RT_UNROLL 8

// lanes of this wave that hold the same in-range expert id as the calling lane (0 for out-of-range lanes)
__device__ __forceinline__ uint64_t rt_match(int e, bool in_range, int nbits) {
  uint64_t mask = __builtin_amdgcn_ballot_w64(in_range);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (e >> b) & 1;
    const uint64_t v = __builtin_amdgcn_ballot_w64(in_range && bit);
    mask &= bit ? v : ~v;
  }
  return in_range ? mask : 0;
}

// One pass over the rows [begin, end) of a wave: calls f(row, expert, lanes_with_same_expert) for every row whose
// expert id is in range, 64 rows at a time, RT_UNROLL loads in flight.
template <typename IdT, typename F>
__device__ __forceinline__ void rt_for_rows(const IdT* __restrict__ ids, int begin, int end, int E, int nbits, int lane, F f) {
  for (int base = begin; base < end; base += 64 * RT_UNROLL) {
    int e[RT_UNROLL];
#pragma unroll
    for (int u = 0; u < RT_UNROLL; ++u) {
      const int r = base + 64 * u + lane;
      e[u] = -1;
      if (r < end) {
        const IdT v = ids[r];
        e[u] = (v >= 0 && v < (IdT)E) ? (int)v : -1;  // also rejects 64-bit ids that do not fit an int
      }
    }
#pragma unroll
    for (int u = 0; u < RT_UNROLL; ++u) {
      if (base + 64 * u >= end) break;  // wave-uniform
      const bool ok = e[u] >= 0;
      const uint64_t m = rt_match(e[u], ok, nbits);
      if (ok) f(base + 64 * u + lane, e[u], m);
    }
  }
}

// MODE 0: the whole job in one workgroup.  MODE 1 (count): workgroup b writes its per-expert row counts to
// block_tab[b][E].  MODE 2 (scatter): block_tab[b][e] holds the first output slot of workgroup b's rows of expert e
// (hx_moe_routing_scan turned the counts into slots) and the workgroup scatters its rows.
// ME: experts the LDS tables hold (RT_MAX_E or RT_MAX_E_WIDE); a work-item owns experts tid, tid + 1024, ... below ME.
template <typename IdT, int MODE, int ME = RT_MAX_E>
__global__ __launch_bounds__(64 * RT_WAVES) void hx_moe_routing_kernel(const IdT* __restrict__ ids, int T, int E, int nbits,
                                                                      int block_rows, int32_t* __restrict__ counts,
                                                                      int32_t* __restrict__ offsets, int32_t* __restrict__ idx,
                                                                      int32_t* __restrict__ max_count, int32_t* __restrict__ block_tab) {
  __shared__ int hist[RT_WAVES][ME];  // count pass: rows per (wave, expert); afterwards: next output slot
  __shared__ int scan[2][ME];
  __shared__ int s_max;
  constexpr int NT = 64 * RT_WAVES, EPT = (ME + NT - 1) / NT;  // experts per work-item
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const uint64_t lt_mask = ((uint64_t)1 << lane) - 1;
  for (int i = tid; i < RT_WAVES * ME; i += 64 * RT_WAVES) (&hist[0][0])[i] = 0;
  if (tid == 0) s_max = 0;
  __syncthreads();

  // rows of this workgroup and of this wave (block_rows is a multiple of 64 * RT_WAVES: aligned, coalesced groups)
  const long long b0 = (long long)blockIdx.x * block_rows;
  const int chunk = block_rows / RT_WAVES;
  const int begin = (int)min((long long)T, b0 + (long long)w * chunk), end = (int)min((long long)T, (long long)begin + chunk);

  // Up to 2048 rows per wave (the one-workgroup form up to 32768 rows) the ids are read once, all loads in flight
  // together, and both passes walk the registers.
  constexpr int RT_CACHE = 32;
  const bool cached = MODE == 0 && chunk <= 64 * RT_CACHE;  // workgroup-uniform
  int ec[RT_CACHE];
  if (cached) {
#pragma unroll
    for (int u = 0; u < RT_CACHE; ++u) {
      const int r = begin + 64 * u + lane;
      ec[u] = -1;
      if (r < end) {
        const IdT v = ids[r];
        ec[u] = (v >= 0 && v < (IdT)E) ? (int)v : -1;
      }
    }
  }
  auto for_rows = [&](auto f) {
    if (cached) {
#pragma unroll
      for (int u = 0; u < RT_CACHE; ++u) {
        if (begin + 64 * u >= end) break;  // wave-uniform
        const bool ok = ec[u] >= 0;
        const uint64_t m = rt_match(ec[u], ok, nbits);
        if (ok) f(begin + 64 * u + lane, ec[u], m);
      }
    } else {
      rt_for_rows(ids, begin, end, E, nbits, lane, f);
    }
  };

  // ---- count pass: the first lane of every group of equal experts adds the group's size
  for_rows([&](int, int e, uint64_t m) {
    if ((m & lt_mask) == 0) hist[w][e] += __builtin_popcountll(m);
  });
  __syncthreads();

  // ---- per expert: prefix over the waves of this workgroup
  int total[EPT];
#pragma unroll
  for (int u = 0; u < EPT; ++u) {
    const int e = tid + u * NT;
    total[u] = 0;
    if (e < E) {
      for (int ww = 0; ww < RT_WAVES; ++ww) {
        const int v = hist[ww][e];
        hist[ww][e] = total[u];
        total[u] += v;
      }
    }
  }
  if (MODE == 1) {
#pragma unroll
    for (int u = 0; u < EPT; ++u)
      if (tid + u * NT < E) block_tab[(long long)blockIdx.x * E + tid + u * NT] = total[u];
    return;
  }
  int covered;
  if (MODE == 0) {
    // exclusive prefix over experts (inclusive Hillis-Steele scan over ME slots, minus the own count)
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
      const int e = tid + u * NT;
      if (e < E) {
        counts[e] = total[u];
        atomicMax(&s_max, total[u]);
      }
      if (e < ME) scan[0][e] = e < E ? total[u] : 0;
    }
    __syncthreads();
    int src = 0;
    for (int d = 1; d < ME; d <<= 1) {
#pragma unroll
      for (int u = 0; u < EPT; ++u) {
        const int e = tid + u * NT;
        if (e < ME) scan[src ^ 1][e] = scan[src][e] + (e >= d ? scan[src][e - d] : 0);
      }
      src ^= 1;
      __syncthreads();
    }
    covered = E > 0 ? scan[src][E - 1] : 0;
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
      const int e = tid + u * NT;
      if (e < E) {
        const int excl = scan[src][e] - total[u];
        offsets[e] = excl;
        for (int ww = 0; ww < RT_WAVES; ++ww) hist[ww][e] += excl;
      }
    }
    if (tid == 0) {
      offsets[E] = covered;
      *max_count = s_max;
    }
  } else {
    covered = offsets[E];
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
      const int e = tid + u * NT;
      if (e < E) {
        const int first = block_tab[(long long)blockIdx.x * E + e];
        for (int ww = 0; ww < RT_WAVES; ++ww) hist[ww][e] += first;
      }
    }
  }
  __syncthreads();

  // ---- scatter pass
  for_rows([&](int r, int e, uint64_t m) {
    const int slot = hist[w][e];  // every lane of the group reads before its first lane advances the slot
    const int rank = __builtin_popcountll(m & lt_mask);
    if (rank == 0) hist[w][e] = slot + __builtin_popcountll(m);
    idx[slot + rank] = r;
  });
  // rows with out-of-range ids leave the tail of idx unused: mark it
  for (long long i = (long long)covered + blockIdx.x * (64 * RT_WAVES) + tid; i < T; i += (long long)gridDim.x * 64 * RT_WAVES)
    idx[i] = -1;
}

// block_tab[b][e] (counts) -> first output slot of workgroup b's rows of expert e; also counts, offsets, max_count.
// One workgroup of min(ME, 1024) work-items.
template <int ME>
__global__ __launch_bounds__(ME < 1024 ? ME : 1024) void hx_moe_routing_scan(int32_t* __restrict__ block_tab, int B, int E,
                                                                             int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                                             int32_t* __restrict__ max_count) {
  __shared__ int scan[2][ME];
  __shared__ int s_max;
  constexpr int NT = ME < 1024 ? ME : 1024, EPT = ME / NT;
  const int tid = threadIdx.x;
  if (tid == 0) s_max = 0;
  __syncthreads();
  int total[EPT];
#pragma unroll
  for (int u = 0; u < EPT; ++u) {
    const int e = tid + u * NT;
    total[u] = 0;
    if (e < E) {
      for (int b = 0; b < B; ++b) {
        const int v = block_tab[(long long)b * E + e];
        block_tab[(long long)b * E + e] = total[u];
        total[u] += v;
      }
      counts[e] = total[u];
      atomicMax(&s_max, total[u]);
    }
    scan[0][e] = e < E ? total[u] : 0;
  }
  __syncthreads();
  int src = 0;
  for (int d = 1; d < ME; d <<= 1) {
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
      const int e = tid + u * NT;
      scan[src ^ 1][e] = scan[src][e] + (e >= d ? scan[src][e - d] : 0);
    }
    src ^= 1;
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < EPT; ++u) {
    const int e = tid + u * NT;
    if (e < E) {
      const int excl = scan[src][e] - total[u];
      offsets[e] = excl;
      for (int b = 0; b < B; ++b) block_tab[(long long)b * E + e] += excl;
    }
  }
  if (tid == 0) {
    offsets[E] = E > 0 ? scan[src][E - 1] : 0;
    *max_count = s_max;
  }
}

#define RT_SINGLE_MAX_T 32768  // up to here one workgroup (one launch) is faster than three launches
#define RT_MAX_BLOCKS 256

// rows per workgroup and number of workgroups of the multi-workgroup form
static inline void rt_blocks(int64_t T, int64_t* block_rows, int64_t* blocks) {
  int64_t br = 16384;
  while ((T + br - 1) / br > RT_MAX_BLOCKS) br *= 2;
  *block_rows = br;
  *blocks = (T + br - 1) / br;
}

// most experts a call may name: RT_MAX_E, or RT_MAX_E_WIDE with the opt-in instantiation
static int64_t rt_max_e() { return hx_feature(HX_FEATURE_ROUTING_WIDE) ? RT_MAX_E_WIDE : RT_MAX_E; }

extern "C" size_t hx_moe_routing_workspace_bytes(int64_t T, int64_t E) {
  if (T <= RT_SINGLE_MAX_T || E <= 0 || E > rt_max_e()) return 0;
  int64_t br, nb;
  rt_blocks(T, &br, &nb);
  return (size_t)nb * (size_t)E * 4;
}

template <typename IdT, int ME>
static void rt_launch(const IdT* ids, int64_t T, int64_t E, int nbits, int32_t* counts, int32_t* offsets, int32_t* idx,
                      int32_t* max_count, void* ws, size_t ws_bytes, hipStream_t s) {
  const size_t need = hx_moe_routing_workspace_bytes(T, E);
  if (need == 0 || !ws || ws_bytes < need) {
    const int block_rows = (int)((((T + RT_WAVES - 1) / RT_WAVES + 63) & ~(int64_t)63) * RT_WAVES);
    hx_launch((hx_moe_routing_kernel<IdT, 0, ME>), dim3(1), dim3(64 * RT_WAVES), 0, s, ids, (int)T, (int)E, nbits,
                       block_rows > 0 ? block_rows : 64 * RT_WAVES, counts, offsets, idx, max_count, (int32_t*)nullptr);
    return;
  }
  int64_t br, nb;
  rt_blocks(T, &br, &nb);
  int32_t* tab = (int32_t*)ws;
  hx_launch((hx_moe_routing_kernel<IdT, 1, ME>), dim3((unsigned)nb), dim3(64 * RT_WAVES), 0, s, ids, (int)T, (int)E, nbits, (int)br,
                     counts, offsets, idx, max_count, tab);
  hx_launch(hx_moe_routing_scan<ME>, dim3(1), dim3(ME < 1024 ? ME : 1024), 0, s, tab, (int)nb, (int)E, counts, offsets, max_count);
  hx_launch((hx_moe_routing_kernel<IdT, 2, ME>), dim3((unsigned)nb), dim3(64 * RT_WAVES), 0, s, ids, (int)T, (int)E, nbits, (int)br,
                     counts, offsets, idx, max_count, tab);
}

extern "C" int hx_moe_routing(const void* expert_ids, int ids_are_int64, int64_t T, int64_t E, int32_t* counts, int32_t* offsets,
                              int32_t* idx, int32_t* max_count, void* workspace, size_t workspace_bytes, void* stream) {
  if (T < 0 || E < 0) {
    hx_set_error("hx_moe_routing: negative size");
    return HX_ERR_BAD_ARG;
  }
  if (E > rt_max_e() || T >= (1LL << 31) - 64 * RT_WAVES * RT_UNROLL) {
    hx_set_error("hx_moe_routing: unsupported size T=%lld E=%lld (E <= %d)", (long long)T, (long long)E, (int)rt_max_e());
    return HX_ERR_UNSUPPORTED;
  }
  if (!offsets || !max_count || (E > 0 && !counts) || (T > 0 && (!expert_ids || !idx))) {
    hx_set_error("hx_moe_routing: null pointer");
    return HX_ERR_BAD_ARG;
  }
  if (workspace && ((uintptr_t)workspace & 3)) {
    hx_set_error("hx_moe_routing: workspace must be 4-byte aligned");
    return HX_ERR_WORKSPACE;
  }
  int nbits = 0;
  while ((1LL << nbits) < E) ++nbits;
  hipStream_t s = (hipStream_t)stream;
  if (E > RT_MAX_E) {
    if (ids_are_int64) rt_launch<long long, RT_MAX_E_WIDE>((const long long*)expert_ids, T, E, nbits, counts, offsets, idx, max_count, workspace, workspace_bytes, s);
    else rt_launch<int, RT_MAX_E_WIDE>((const int*)expert_ids, T, E, nbits, counts, offsets, idx, max_count, workspace, workspace_bytes, s);
  } else if (ids_are_int64) rt_launch<long long, RT_MAX_E>((const long long*)expert_ids, T, E, nbits, counts, offsets, idx, max_count, workspace, workspace_bytes, s);
  else rt_launch<int, RT_MAX_E>((const int*)expert_ids, T, E, nbits, counts, offsets, idx, max_count, workspace, workspace_bytes, s);
  hipError_t err = hx_launch_status();
  if (err != hipSuccess) {
    hx_set_error("hx_moe_routing: launch failed: %s", hipGetErrorString(err));
    return (int)err;
  }
  return 0;
}
