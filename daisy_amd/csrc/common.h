// Shared device/host helpers for the gfx950 attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/daisy_hip.h"

namespace daisy {

// ---- vector types ---------------------------------------------------------
typedef __bf16 bf16_t;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;

// ---- bf16 <-> fp32 ----------------------------------------------------------
// A bf16 is the high half of an fp32, so widening is a shift.
__device__ __forceinline__ float bf16lo_to_f32(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// Round-to-nearest-even pack of two fp32 into one dword of bf16 (lo = a, hi = b).
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  f32x2 x = {a, b};
  bf16x2 y = __builtin_convertvector(x, bf16x2);
  return __builtin_bit_cast(uint32_t, y);
}
__device__ __forceinline__ float round_bf16(float a) {
  return bf16lo_to_f32(pack_bf16x2(a, 0.f));
}

// Unpack 8 bf16 held in a 16-byte register quad into 8 floats.
__device__ __forceinline__ void unpack8(const u32x4& r, float* f) {
  f[0] = bf16lo_to_f32(r.x); f[1] = bf16hi_to_f32(r.x);
  f[2] = bf16lo_to_f32(r.y); f[3] = bf16hi_to_f32(r.y);
  f[4] = bf16lo_to_f32(r.z); f[5] = bf16hi_to_f32(r.z);
  f[6] = bf16lo_to_f32(r.w); f[7] = bf16hi_to_f32(r.w);
}
__device__ __forceinline__ u32x4 pack8(const float* f) {
  u32x4 r;
  r.x = pack_bf16x2(f[0], f[1]); r.y = pack_bf16x2(f[2], f[3]);
  r.z = pack_bf16x2(f[4], f[5]); r.w = pack_bf16x2(f[6], f[7]);
  return r;
}

// RoPE on one pair (x1 at channel i, x2 at channel i + D/2):
//   y1 = x1*cos + x2*sin,  y2 = -x1*sin + x2*cos.
// Products and sum are rounded separately (no fused multiply-add), the way an
// elementwise tensor library evaluates the expression, so that the bf16 result
// is bit-identical to it.
__device__ __forceinline__ float rope_lo(float x1, float x2, float c, float s) {
#pragma clang fp contract(off)
  const float a = x1 * c;
  const float b = x2 * s;
  return a + b;
}
__device__ __forceinline__ float rope_hi(float x1, float x2, float c, float s) {
#pragma clang fp contract(off)
  const float a = x1 * -s;
  const float b = x2 * c;
  return a + b;
}

// Element access for kernels templated on the tensor element: uint16_t = bf16 bits, float = fp32.
// round_elem rounds a computed value the way a tensor of that element type would hold it.
template <typename E> __device__ __forceinline__ float load_elem(const E* p, int64_t i);
template <> __device__ __forceinline__ float load_elem<uint16_t>(const uint16_t* p, int64_t i) { return bf16lo_to_f32(p[i]); }
template <> __device__ __forceinline__ float load_elem<float>(const float* p, int64_t i) { return p[i]; }
template <typename E> __device__ __forceinline__ void store_elem(E* p, int64_t i, float x);
template <> __device__ __forceinline__ void store_elem<uint16_t>(uint16_t* p, int64_t i, float x) {
  p[i] = (uint16_t)(pack_bf16x2(x, 0.f) & 0xffffu);
}
template <> __device__ __forceinline__ void store_elem<float>(float* p, int64_t i, float x) { p[i] = x; }
template <typename E> __device__ __forceinline__ float round_elem(float x);
template <> __device__ __forceinline__ float round_elem<uint16_t>(float x) { return round_bf16(x); }
template <> __device__ __forceinline__ float round_elem<float>(float x) { return x; }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- cross-lane sums with DPP (no LDS traffic) -------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  int y = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false);
  return x + __int_as_float(y);
}

// Sum over the LPR consecutive lanes that share a cache row; every lane of the
// group ends with the total.
template <int LPR>
__device__ __forceinline__ float group_sum(float x) {
  x = dpp_add<0xB1>(x);                     // quad_perm [1,0,3,2]   (xor 1)
  x = dpp_add<0x4E>(x);                     // quad_perm [2,3,0,1]   (xor 2)
  if (LPR >= 8) x = dpp_add<0x141>(x);      // row_half_mirror       (joins the two quads of 8 lanes)
  if (LPR >= 16) x = dpp_add<0x128>(x);     // row_ror 8             (joins the two halves of 16 lanes)
  if (LPR >= 32) x += __shfl_xor(x, 16);    // the neighbouring row of 16 lanes
  return x;
}

// ---- asynchronous global -> LDS copies ------------------------------------------
// Asynchronous 16-byte global -> LDS copy that bypasses the vector registers
// (global_load_lds_dwordx4): lane i of the wavefront deposits the 16 bytes at
// gbase + byte_off at LDS address lds_addr + 16*i.  gbase and lds_addr are wavefront-uniform.
// Issued as inline assembly so that the compiler does not serialise later LDS reads of the
// OTHER buffer behind it; the caller waits with s_waitcnt vmcnt(0) before publishing the tile.
__device__ __forceinline__ void copy16_to_lds_async(const uint16_t* gbase, int byte_off, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(byte_off), "s"(gbase), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(size_t)(__attribute__((address_space(3))) const void*)p;
}

// ---- host-side error plumbing --------------------------------------------
void set_error(const char* fmt, ...);

#define DAISY_CHECK_ARG(cond, ...)            \
  do {                                        \
    if (!(cond)) {                            \
      daisy::set_error(__VA_ARGS__);          \
      return DAISY_ERR_INVALID_ARGUMENT;      \
    }                                         \
  } while (0)

#define DAISY_CHECK_SUPPORTED(cond, ...)      \
  do {                                        \
    if (!(cond)) {                            \
      daisy::set_error(__VA_ARGS__);          \
      return DAISY_ERR_UNSUPPORTED;           \
    }                                         \
  } while (0)

// Checks the launch error state after a kernel launch.
#define DAISY_CHECK_LAUNCH(what)                                                   \
  do {                                                                             \
    hipError_t e_ = hipGetLastError();                                             \
    if (e_ != hipSuccess) {                                                        \
      daisy::set_error("%s: launch failed: %s", what, hipGetErrorString(e_));      \
      return DAISY_ERR_LAUNCH;                                                     \
    }                                                                              \
  } while (0)

}  // namespace daisy
