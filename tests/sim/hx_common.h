// Stand-in for helion_amd/csrc/hx_common.h in the host execution model (see hx_sim.h): the same names with the same
// meaning, the three pieces of inline assembly and the launch helper expressed through the model.  The kernel sources
// are compiled against this file unchanged otherwise.
#pragma once
#include <stdint.h>

#include <tuple>
#include <utility>

#include "hx_kernels.h"

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

#define HX_LDS(p) (p)
#define HX_GLB(p) (p)

// global->LDS DMA: lane `l` of the wave writes `bytes` at lds_wave_base + l * bytes
inline void hx_g2l16(const void* gptr, void* lds_wave_base) {
  hxsim::dma(gptr, hxsim::lds_addr(lds_wave_base) + (threadIdx.x & 63) * 16, 16);
}
inline void hx_g2l16_s(const void* sbase, uint32_t voff, uint32_t lds_wave_base) {
  hxsim::dma((const uint8_t*)sbase + voff, lds_wave_base + (threadIdx.x & 63) * 16, 16);
}
inline void hx_g2l16_s_nt(const void* sbase, uint32_t voff, uint32_t lds_wave_base) { hx_g2l16_s(sbase, voff, lds_wave_base); }
inline void hx_g2l4_s(const void* sbase, uint32_t voff, uint32_t lds_wave_base) {
  hxsim::dma((const uint8_t*)sbase + voff, lds_wave_base + (threadIdx.x & 63) * 4, 4);
}
inline const uint8_t* hx_uniform_ptr(const uint8_t* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const uint8_t*)(((uint64_t)hi << 32) | lo);
}
inline uint32_t hx_lds_addr(const void* p) { return hxsim::lds_addr(p); }

#define HX_OPAQUE_V(x) ((void)(x))
#define HX_OPAQUE_S(x) ((void)(x))

#define HX_WAIT_VM0() __builtin_amdgcn_s_waitcnt(0x0F70)
#define HX_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)
inline constexpr int hx_vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

inline v16f hx_mfma_32x32x64_e4m3(v8i a, v8i b, v16f c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
inline v4f hx_mfma_16x16x128_e4m3(v8i a, v8i b, v4f c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

inline float hx_acc_read(float e) { return e; }
inline void hx_mfma_16x16x128_e4m3_overwrite(v4f& acc, v8i a, v8i b) { acc = hx_mfma_16x16x128_e4m3(a, b, (v4f){0.f, 0.f, 0.f, 0.f}); }
inline void hx_mfma_16x16x128_e4m3_acc(v4f& acc, v8i a, v8i b) { acc = hx_mfma_16x16x128_e4m3(a, b, acc); }

template <bool BF>
struct Mfma16;
template <>
struct Mfma16<true> {
  typedef __bf16 T;
  typedef v8bf V8;
  static inline v16f run(v8bf a, v8bf b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static inline v4f run16(v8bf a, v8bf b, v4f c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
  static inline void overwrite16(v4f& acc, v8bf a, v8bf b) { acc = run16(a, b, (v4f){0.f, 0.f, 0.f, 0.f}); }
  static inline void acc16(v4f& acc, v8bf a, v8bf b) { acc = run16(a, b, acc); }
};
template <>
struct Mfma16<false> {
  typedef _Float16 T;
  typedef v8h V8;
  static inline v16f run(v8h a, v8h b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static inline v4f run16(v8h a, v8h b, v4f c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
  static inline void overwrite16(v4f& acc, v8h a, v8h b) { acc = run16(a, b, (v4f){0.f, 0.f, 0.f, 0.f}); }
  static inline void acc16(v4f& acc, v8h a, v8h b) { acc = run16(a, b, acc); }
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

#define HX_CVT_PK_E4M3(a, b, old, hi) __builtin_amdgcn_cvt_pk_fp8_f32((a), (b), (old), (hi))
inline float hx_e4m3_to_f32(uint8_t code) { return __builtin_amdgcn_cvt_f32_fp8((int)code, 0); }

void hx_set_error(const char* fmt, ...);
int hx_cu_count();
bool hx_feature(unsigned bit);

inline thread_local hipError_t hx_tls_launch_err = hipSuccess;
template <typename... KArgs, typename... Args>
static inline void hx_launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned shmem, hipStream_t, Args&&... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "hx_launch: argument count does not match the kernel's");
  (void)shmem;
  std::tuple<KArgs...> vals{static_cast<KArgs>(args)...};
  const hipError_t e = hxsim::run(grid, block, [&]() { std::apply(kernel, vals); }, (const void*)kernel);
  if (e != hipSuccess && hx_tls_launch_err == hipSuccess) hx_tls_launch_err = e;
}
static inline hipError_t hx_launch_status() {
  const hipError_t e = hx_tls_launch_err;
  hx_tls_launch_err = hipSuccess;
  return e;
}
