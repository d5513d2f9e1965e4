// Host execution model for the gfx950 kernels (test infrastructure; nothing under helion_amd/ includes or loads it).
//
// The kernel sources under helion_amd/csrc are compiled for the host CPU as they are, with this header included in
// front of them.  It supplies what the device compiler and the hardware supply on the GPU: the HIP keywords and launch
// geometry, and every gfx950 builtin the kernels use (matrix instructions, global->LDS DMA, transposing LDS reads,
// cross-lane moves, wait counters, fp8 conversion), each executed with the semantics of the instruction it stands for.
// One work-item is one fiber (its registers are its stack frame); the 64 fibers of a wave meet at every cross-lane
// instruction, which is then evaluated once for the whole wave; the waves of a workgroup meet at barriers.  DMA
// transfers land either at issue or as late as the wave's wait counter allows, and waves are scheduled in several
// orders, so a missing wait or barrier shows up as a wrong result.  Operand buffers sit between inaccessible pages, so
// an out-of-range global access stops the launch with the faulting address instead of going unnoticed.
//
// The arithmetic is what the instructions define (e4m3 / 16-bit products summed into fp32); the matrix pipe's internal
// summation order is not modelled, so results agree with the GPU's to accumulation rounding, not bit for bit.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <cmath>
#include <functional>
#include <tuple>
#include <type_traits>
#include <utility>

#define HX_SIM 1

// ---- HIP keywords ------------------------------------------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
// every __shared__ array of every kernel lives in one linker section, so the model knows where the LDS is, can give
// LDS pointers 32-bit addresses, refuse DMA and transposing reads that leave it, and poison it between workgroups
#define __shared__ static __attribute__((section("hx_lds")))
#define HIP_SYMBOL(x) x

struct dim3 {
  unsigned x, y, z;
  constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorLaunchFailure = 719 };
typedef void* hipStream_t;
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 63 };
const char* hipGetErrorString(hipError_t e);
hipError_t hipGetDevice(int* dev);
hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t attr, int dev);
template <typename T>
inline hipError_t hipGetSymbolAddress(void** p, T& sym) {
  *p = (void*)&sym;
  return hipSuccess;
}

namespace hxsim {

struct Lane;
extern Lane* cur;  // the work-item that is executing
struct Idx3 {
  unsigned x, y, z;
};
struct Geometry {
  Idx3 block_idx, block_dim, grid_dim;
};
extern Geometry geo;
const Idx3& thread_idx();

// ---- synchronisation and cross-lane instructions (each takes the source line as a site id: lanes that diverged to
// different sites are resolved as separate groups, like the hardware runs the sides of a branch one after the other)
void barrier();
int barrier_or(int pred);
void waitcnt(int imm);
void sleep(int n);
int readfirstlane(int v, int site);
void wave_sync(int site);
uint64_t ballot(bool p, int site);
uint32_t shfl_xor_u32(uint32_t v, int mask, int site);
uint32_t mov_dpp_u32(uint32_t v, int ctrl, int row_mask, int bank_mask, bool bound_ctrl, int site);
void permlane32_swap_u32(uint32_t a, uint32_t b, uint32_t out[2], int site);
void mfma(int kind, const void* a, const void* b, const void* c, void* d, int site);
void ds_read_tr(int elem_bytes, const void* lds_ptr, void* out8, int site);
void dma(const void* gptr, uint32_t lds_dst, int bytes);
uint32_t lds_addr(const void* p);
int cvt_pk_fp8(float a, float b, int old, bool hi);
float cvt_f32_fp8(int v, int sel);
uint64_t clock100mhz();

enum { MFMA_F8_32x32x64 = 0, MFMA_F8_16x16x128, MFMA_F8_16x16x32, MFMA_BF16_32x32x16, MFMA_F16_32x32x16, MFMA_BF16_16x16x32, MFMA_F16_16x16x32 };

// runs `fn` once per work-item of the grid; returns hipSuccess or hipErrorLaunchFailure (message: hx_sim_last_fault)
hipError_t run(dim3 grid, dim3 block, const std::function<void()>& fn, const void* kernel);

}  // namespace hxsim

#define threadIdx (hxsim::thread_idx())
#define blockIdx (hxsim::geo.block_idx)
#define blockDim (hxsim::geo.block_dim)
#define gridDim (hxsim::geo.grid_dim)

// ---- vector types the builtins below mention (the kernels' own header declares the same typedefs again)
typedef int hxs_v8i __attribute__((ext_vector_type(8)));
typedef int hxs_v2i __attribute__((ext_vector_type(2)));
typedef float hxs_v16f __attribute__((ext_vector_type(16)));
typedef float hxs_v4f __attribute__((ext_vector_type(4)));
typedef short hxs_v4s __attribute__((ext_vector_type(4)));
typedef __bf16 hxs_v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 hxs_v8h __attribute__((ext_vector_type(8)));
typedef unsigned hxs_v2u __attribute__((ext_vector_type(2)));

namespace hxsim {
template <int KIND, typename AB, typename CD>
inline CD mfma_t(AB a, AB b, CD c, int site) {
  CD d;
  mfma(KIND, &a, &b, &c, &d, site);
  return d;
}
inline hxs_v2i ds_read_tr8_b64(const void* p, int site) {
  hxs_v2i r;
  ds_read_tr(1, p, &r, site);
  return r;
}
inline hxs_v4s ds_read_tr16_b64(const void* p, int site) {
  hxs_v4s r;
  ds_read_tr(2, p, &r, site);
  return r;
}
inline hxs_v2u permlane32_swap(uint32_t a, uint32_t b, int site) {
  uint32_t o[2];
  permlane32_swap_u32(a, b, o, site);
  return (hxs_v2u){o[0], o[1]};
}
template <typename T>
inline T mov_dpp(T v, int ctrl, int rm, int bm, bool bc, int site) {
  static_assert(sizeof(T) == 4, "32-bit DPP only");
  uint32_t u;
  memcpy(&u, &v, 4);
  u = mov_dpp_u32(u, ctrl, rm, bm, bc, site);
  memcpy(&v, &u, 4);
  return v;
}
template <typename T>
inline T shfl_xor(T v, int mask, int site) {
  static_assert(sizeof(T) == 4, "32-bit shuffles only");
  uint32_t u;
  memcpy(&u, &v, 4);
  u = shfl_xor_u32(u, mask, site);
  memcpy(&v, &u, 4);
  return v;
}
}  // namespace hxsim

// ---- the gfx950 builtins the kernels use ------------------------------------------------------------------------------
#define __syncthreads() hxsim::barrier()
#define __syncthreads_or(p) hxsim::barrier_or(p)
#define __builtin_amdgcn_s_waitcnt(imm) hxsim::waitcnt(imm)
#define __builtin_amdgcn_s_sleep(n) hxsim::sleep(n)
#define __builtin_amdgcn_s_setprio(n) ((void)0)
#define __builtin_amdgcn_sched_barrier(m) ((void)0)
// a wavefront-scope fence orders one wave's LDS traffic: on the hardware the lanes of a wave move in lockstep, here
// they meet at it
#define __builtin_amdgcn_fence(...) hxsim::wave_sync(__LINE__)
#define __builtin_amdgcn_readfirstlane(v) hxsim::readfirstlane((int)(v), __LINE__)
#define __builtin_amdgcn_ballot_w64(p) hxsim::ballot((p), __LINE__)
#define __builtin_amdgcn_mov_dpp(v, ctrl, rm, bm, bc) hxsim::mov_dpp((v), (ctrl), (rm), (bm), (bc), __LINE__)
#define __builtin_amdgcn_permlane32_swap(a, b, fi, bc) hxsim::permlane32_swap((a), (b), __LINE__)
#define __shfl_xor(v, mask) hxsim::shfl_xor((v), (mask), __LINE__)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, cbsz, blgp, o0, s0, o1, s1) \
  hxsim::mfma_t<hxsim::MFMA_F8_32x32x64, hxs_v8i, hxs_v16f>((a), (b), (c), __LINE__)
#define __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, cbsz, blgp, o0, s0, o1, s1) \
  hxsim::mfma_t<hxsim::MFMA_F8_16x16x128, hxs_v8i, hxs_v4f>((a), (b), (c), __LINE__)
#define __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, b, c, x, y, z) hxsim::mfma_t<hxsim::MFMA_F8_16x16x32, long, hxs_v4f>((long)(a), (long)(b), (c), __LINE__)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) hxsim::mfma_t<hxsim::MFMA_BF16_32x32x16, hxs_v8bf, hxs_v16f>((a), (b), (c), __LINE__)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) hxsim::mfma_t<hxsim::MFMA_F16_32x32x16, hxs_v8h, hxs_v16f>((a), (b), (c), __LINE__)
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) hxsim::mfma_t<hxsim::MFMA_BF16_16x16x32, hxs_v8bf, hxs_v4f>((a), (b), (c), __LINE__)
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) hxsim::mfma_t<hxsim::MFMA_F16_16x16x32, hxs_v8h, hxs_v4f>((a), (b), (c), __LINE__)
#define __builtin_amdgcn_ds_read_tr8_b64_v2i32(p) hxsim::ds_read_tr8_b64((const void*)(uintptr_t)(p), __LINE__)
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) hxsim::ds_read_tr16_b64((const void*)(uintptr_t)(p), __LINE__)
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, hi) hxsim::cvt_pk_fp8((a), (b), (old), (hi))
#define __builtin_amdgcn_cvt_f32_fp8(v, sel) hxsim::cvt_f32_fp8((v), (sel))

// ---- HIP device library bits
#define __HIP_MEMORY_SCOPE_AGENT 4
#define __hip_atomic_fetch_add(p, v, order, scope) hxsim_fetch_add((p), (v))
#define __hip_atomic_load(p, order, scope) hxsim_atomic_load(p)
#define __hip_atomic_store(p, v, order, scope) hxsim_atomic_store((p), (v))
template <typename T>
__attribute__((noinline, no_sanitize("coverage"))) inline T hxsim_atomic_load(const T* p) {
  return *p;
}
template <typename T, typename V>
__attribute__((noinline, no_sanitize("coverage"))) inline void hxsim_atomic_store(T* p, V v) {
  *p = (T)v;
}
// (atomics are not plain loads and stores: kept out of the LDS access check)
#define HXSIM_UNTRACED __attribute__((noinline, no_sanitize("coverage")))
template <typename T, typename V>
HXSIM_UNTRACED inline T hxsim_fetch_add(T* p, V v) {  // work-items run one at a time
  const T old = *p;
  *p = old + (T)v;
  return old;
}
template <typename T>
HXSIM_UNTRACED inline T atomicMax(T* p, T v) {
  const T old = *p;
  if (v > old) *p = v;
  return old;
}
template <typename T>
HXSIM_UNTRACED inline T atomicAdd(T* p, T v) {
  const T old = *p;
  *p = old + v;
  return old;
}
inline uint64_t wall_clock64() { return hxsim::clock100mhz(); }
inline unsigned __float_as_uint(float f) {
  unsigned u;
  memcpy(&u, &f, 4);
  return u;
}
inline float __uint_as_float(unsigned u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
inline int __float_as_int(float f) {
  int u;
  memcpy(&u, &f, 4);
  return u;
}
inline float __int_as_float(int u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
// HIP's min / max take mixed integer types
template <typename A, typename B, typename = std::enable_if_t<std::is_arithmetic<A>::value && std::is_arithmetic<B>::value>>
inline constexpr std::common_type_t<A, B> min(A a, B b) {
  typedef std::common_type_t<A, B> T;
  return (T)b < (T)a ? (T)b : (T)a;
}
template <typename A, typename B, typename = std::enable_if_t<std::is_arithmetic<A>::value && std::is_arithmetic<B>::value>>
inline constexpr std::common_type_t<A, B> max(A a, B b) {
  typedef std::common_type_t<A, B> T;
  return (T)a < (T)b ? (T)b : (T)a;
}
