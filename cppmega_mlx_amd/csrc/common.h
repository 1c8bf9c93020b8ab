// Shared device/host helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cppmega_mi355.h"

namespace cm {

constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

// ---- thread-local error text (host) ---------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

#define CM_HIP_CHECK(expr)                                                          \
  do {                                                                              \
    hipError_t _e = (expr);                                                         \
    if (_e != hipSuccess)                                                           \
      return ::cm::fail(CPPMEGA_MI355_ERR_LAUNCH, "%s: %s", #expr, hipGetErrorString(_e)); \
  } while (0)

// ---- scalar conversions (device) ------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(unsigned short b) {
  return __uint_as_float(((unsigned)b) << 16);
}
// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ unsigned short f32_to_bf16_bits(float f) {
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float f16_bits_to_f32(unsigned short b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}
__device__ __forceinline__ unsigned short f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  unsigned short b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

// OCP e4m3fn byte -> float via the gfx950 converter (two bytes per instruction).
__device__ __forceinline__ f32x2 e4m3x2_lo(unsigned packed) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)packed, false);
}
__device__ __forceinline__ f32x2 e4m3x2_hi(unsigned packed) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)packed, true);
}
__device__ __forceinline__ float e4m3_to_f32(unsigned char b) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)(unsigned)b, false)[0];
}
// E8M0 scale byte: 0 and 255 decode to 0, otherwise 2^(b-127).
__device__ __forceinline__ float e8m0_to_f32(unsigned char b) {
  return (b == 0 || b == 255) ? 0.0f : __uint_as_float(((unsigned)b) << 23);
}

__device__ __forceinline__ void store_as(void* base, size_t i, int dtype, float v) {
  if (dtype == CPPMEGA_MI355_F32) {
    ((float*)base)[i] = v;
  } else if (dtype == CPPMEGA_MI355_BF16) {
    ((unsigned short*)base)[i] = f32_to_bf16_bits(v);
  } else {
    ((unsigned short*)base)[i] = f32_to_f16_bits(v);
  }
}

__device__ __forceinline__ float load_as(const void* base, size_t i, int dtype) {
  if (dtype == CPPMEGA_MI355_F32) return ((const float*)base)[i];
  if (dtype == CPPMEGA_MI355_BF16) return bf16_bits_to_f32(((const unsigned short*)base)[i]);
  if (dtype == CPPMEGA_MI355_F16) return f16_bits_to_f32(((const unsigned short*)base)[i]);
  return e4m3_to_f32(((const unsigned char*)base)[i]);
}

// ---- wavefront collectives -------------------------------------------------
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
// inclusive prefix sum across the 64 lanes
__device__ __forceinline__ unsigned wave_inclusive_sum(unsigned v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    unsigned t = __shfl_up(v, off, 64);
    if (lane >= off) v += t;
  }
  return v;
}
// inclusive prefix sum across the 64 lanes using DPP row shifts / broadcasts (VALU only)
__device__ __forceinline__ unsigned wave_inclusive_sum_dpp(unsigned v) {
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);   // row_shr:1
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);   // row_shr:2
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);   // row_shr:4
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);   // row_shr:8
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);   // row_bcast:15 -> rows 1,3
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);   // row_bcast:31 -> rows 2,3
  return v;
}
// number of set bits of `mask` below this lane
__device__ __forceinline__ unsigned mbcnt(unsigned long long mask) {
  return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
}

inline int dtype_size(int dtype) {
  switch (dtype) {
    case CPPMEGA_MI355_F32: return 4;
    case CPPMEGA_MI355_F16: return 2;
    case CPPMEGA_MI355_BF16: return 2;
    case CPPMEGA_MI355_E4M3: return 1;
    case CPPMEGA_MI355_I32: return 4;
    case CPPMEGA_MI355_I64: return 8;
    default: return 0;
  }
}

}  // namespace cm
