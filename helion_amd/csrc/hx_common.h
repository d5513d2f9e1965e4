// Shared device helpers for the gfx950 kernels: vector types, MFMA wrappers, global->LDS DMA,
// e4m3 conversion, output casts, error plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include <utility>

#include "../../include/hx_kernels.h"

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

#define HX_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define HX_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

// 16-byte global->LDS DMA: every lane supplies its own global address; the wave writes 1024
// contiguous bytes at lds_wave_base + lane*16 (lds_wave_base must be wave-uniform).
__device__ __forceinline__ void hx_g2l16(const void* gptr, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds(HX_GLB(gptr), HX_LDS(lds_wave_base), 16, 0, 0);
}

// Same DMA, spelled in assembly with a wave-uniform 64-bit base (SGPR pair) plus a per-lane 32-bit
// byte offset.  The compiler does not track this load: the caller orders it with HX_WAIT_VM0() and a
// barrier before any lane reads the destination.  (Keeping it out of the compiler's sight is the
// point: its own tracking waits for every outstanding DMA before *any* LDS read of an array it cannot
// tell apart from the destination, which would serialise the prefetch with the MFMA loop.)
__device__ __forceinline__ void hx_g2l16_s(const void* sbase, uint32_t voff, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_wave_base), "v"(voff), "s"(sbase) : "memory", "m0");
}
// The same with the non-temporal hint, for operands a launch reads exactly once (a weight matrix streamed past a single
// row tile): such lines then do not displace what is reused.  The 64-row decode GEMM at N 28672, K 8192: 51 -> 46.6 us.
__device__ __forceinline__ void hx_g2l16_s_nt(const void* sbase, uint32_t voff, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_wave_base), "v"(voff), "s"(sbase) : "memory", "m0");
}
// The 4-byte form: the wave writes 256 contiguous bytes at lds_wave_base + lane*4 (for rows that are only 4-byte aligned).
__device__ __forceinline__ void hx_g2l4_s(const void* sbase, uint32_t voff, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_wave_base), "v"(voff), "s"(sbase) : "memory", "m0");
}
// A wave-uniform pointer the compiler cannot prove uniform (the "s" constraint above needs SGPRs)
__device__ __forceinline__ const uint8_t* hx_uniform_ptr(const uint8_t* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const uint8_t*)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ uint32_t hx_lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)p;
}

// The value goes through an empty instruction the compiler cannot see through (in a vector / a scalar register): what is
// computed from it afterwards cannot be folded to a constant or moved out of the enclosing loop.  The persistent tile
// kernels use it to keep address arithmetic inside their tile loop: hoisted, the several hundred loop-invariant addresses
// are kept in scratch memory, and a reload from scratch makes the compiler wait for every vector-memory operation in
// flight, the hand-counted DMA included.
#define HX_OPAQUE_V(x) asm volatile("" : "+v"(x))
#define HX_OPAQUE_S(x) asm volatile("" : "+s"(x))

// s_waitcnt encodings (gfx9): vmcnt [3:0]+[15:14], expcnt [6:4], lgkmcnt [11:8]
#define HX_WAIT_VM0() __builtin_amdgcn_s_waitcnt(0x0F70)
#define HX_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)
__device__ __forceinline__ constexpr int hx_vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// D(32x32 f32) += A(32 rows x 64 k, e4m3) * B(64 k x 32 cols, e4m3).
// lane l supplies 32 bytes of row/col (l%32), k = (l/32)*32 .. +31; the result lane l holds
// column (l%32), rows 8*(r/4) + 4*(l/32) + (r%4) for r = 0..15.
__device__ __forceinline__ v16f hx_mfma_32x32x64_e4m3(v8i a, v8i b, v16f c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
// D(16x16 f32) += A(16 x 128 e4m3) * B(128 x 16 e4m3); lane l: row/col l%16, k = (l/16)*32 .. +31;
// result lane l: column l%16, rows 4*(l/16) + r, r = 0..3.
__device__ __forceinline__ v4f hx_mfma_16x16x128_e4m3(v8i a, v8i b, v4f c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// The matrix instructions of the persistent tile kernels, written as instructions rather than builtins so that the 256
// accumulators of a wave have one register class and one home each.  Left to the compiler's own accumulator handling, a
// kernel whose accumulators are carried around a tile loop, read out for conversion in one place and restarted from zero
// in another, has its live ranges split between accumulator and ordinary registers, with hundreds of copies and spills
// where the pieces meet - and a reload from scratch memory makes the compiler wait for every vector-memory operation in
// flight, the hand-counted DMA included.
//   *_acc:       D = A x B + D, the accumulator an in-and-out operand in an accumulator register;
//   *_overwrite: D = A x B, the accumulator an output only (its old value is dead: it has just been read out);
//   hx_acc_read: one element of an accumulator copied to an ordinary register at exactly this point.
// The operands come from LDS reads, which the compiler's own waits cover for inline assembly too.  What it does not know
// for inline assembly is the matrix pipe's result latency: the kernels never touch an accumulator within several MFMAs
// of the instruction that wrote it (an accumulator is used once per 64 MFMAs, and read out only after a barrier).
__device__ __forceinline__ void hx_mfma_16x16x128_e4m3_overwrite(v4f& acc, v8i a, v8i b) {
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void hx_mfma_16x16x128_e4m3_acc(v4f& acc, v8i a, v8i b) {
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

__device__ __forceinline__ float hx_acc_read(float e) {
  float t;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(e));
  return t;
}

// 16-bit MFMA (32x32x16, fp32 accumulate): lane l supplies 8 elements of row/col l%32, k = 8*(l/32) .. +7; the result
// layout is that of the 32x32 fp8 MFMA above.  run16 is the 16x16x32 shape: lane l supplies row/col l%16, k = 8*(l/16)
// .. +7, and receives D[4*(l/16) + r][l%16], r = 0..3.
template <bool BF>
struct Mfma16;
template <>
struct Mfma16<true> {
  typedef __bf16 T;
  typedef v8bf V8;
  static __device__ __forceinline__ v16f run(v8bf a, v8bf b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ v4f run16(v8bf a, v8bf b, v4f c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
  // (see hx_mfma_16x16x128_e4m3_overwrite)
  static __device__ __forceinline__ void overwrite16(v4f& acc, v8bf a, v8bf b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void acc16(v4f& acc, v8bf a, v8bf b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
};
template <>
struct Mfma16<false> {
  typedef _Float16 T;
  typedef v8h V8;
  static __device__ __forceinline__ v16f run(v8h a, v8h b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ v4f run16(v8h a, v8h b, v4f c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ void overwrite16(v4f& acc, v8h a, v8h b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void acc16(v4f& acc, v8h a, v8h b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
};

template <int OUT>
struct OutT;
template <>
struct OutT<HX_F16> {
  typedef _Float16 T;
};
template <>
struct OutT<HX_BF16> {
  typedef __bf16 T;
};
template <>
struct OutT<HX_F32> {
  typedef float T;
};

// pack two fp32 -> two e4m3 bytes in the low (hi=false) or high (hi=true) half of `old`
#define HX_CVT_PK_E4M3(a, b, old, hi) __builtin_amdgcn_cvt_pk_fp8_f32((a), (b), (old), (hi))

__device__ __forceinline__ float hx_e4m3_to_f32(uint8_t code) {
  return __builtin_amdgcn_cvt_f32_fp8((int)code, 0);
}

void hx_set_error(const char* fmt, ...);
int hx_cu_count();
bool hx_feature(unsigned bit);  // is this opt-in kernel path (HX_FEATURE_* of the C header) switched on  // compute units of the current device (looked up once per device, 256 if the query fails)

// Kernel launches go through hipLaunchKernel, whose own return code is the launch's status: the library never
// reads (and so never clears) the caller's sticky HIP error state, and a foreign earlier error is never
// attributed to one of its calls.  hx_launch records the first failure of the calling thread's current entry
// point; hx_launch_status() returns it and resets the record (every entry point ends with it).
inline thread_local hipError_t hx_tls_launch_err = hipSuccess;
template <typename... KArgs, typename... Args, size_t... I>
static inline hipError_t hx_launch_impl(void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned shmem, hipStream_t s,
                                        std::index_sequence<I...>, Args&&... args) {
  std::tuple<KArgs...> vals{static_cast<KArgs>(args)...};
  void* ptrs[] = {(void*)&std::get<I>(vals)..., nullptr};
  return hipLaunchKernel((const void*)kernel, grid, block, ptrs, shmem, s);
}
template <typename... KArgs, typename... Args>
static inline void hx_launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned shmem, hipStream_t s, Args&&... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "hx_launch: argument count does not match the kernel's");
  const hipError_t e = hx_launch_impl(kernel, grid, block, shmem, s, std::index_sequence_for<KArgs...>{}, std::forward<Args>(args)...);
  if (e != hipSuccess && hx_tls_launch_err == hipSuccess) hx_tls_launch_err = e;
}
static inline hipError_t hx_launch_status() {
  const hipError_t e = hx_tls_launch_err;
  hx_tls_launch_err = hipSuccess;
  return e;
}
