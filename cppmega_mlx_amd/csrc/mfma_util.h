// Device helpers shared by the matrix-core sparse-MLA kernels (gfx950).
#pragma once

#include "common.h"

namespace cm {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

// The two MFMA shapes as inline assembly with fixed register classes.  The
// 32 x 512 fp32 output accumulators fill all 256 accumulation registers (AGPRs);
// the small score accumulators therefore have to live in ordinary VGPRs, which
// the builtin form of the instruction cannot express once a kernel uses AGPRs.
// Dependent MFMAs on the same accumulator are interlocked by the hardware; a
// VALU read of a result is not, hence mfma_settle().  Nor is an A/B operand
// written by the VALU instruction directly in front of the MFMA (the compiler
// pads that hazard only for instructions it recognises): one wait state is
// required and sufficient (measured), hence the leading s_nop.
__device__ __forceinline__ void mfma_qk(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  asm("s_nop 0\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_pv(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm("s_nop 0\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// the same two shapes on float16 operands
__device__ __forceinline__ void mfma_qk_f16(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  asm("s_nop 0\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_pv_f16(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm("s_nop 0\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// wait states between the last MFMA writing these registers and the first non-MFMA use
__device__ __forceinline__ void mfma_settle(f32x4& s0, f32x4& s1) {
  asm volatile("s_nop 15\n\ts_nop 3" : "+v"(s0), "+v"(s1));
}
__device__ __forceinline__ void mfma_settle_acc(f32x16 (&o)[16]) {
  asm volatile("s_nop 15\n\ts_nop 7"
               : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(o[4]), "+a"(o[5]), "+a"(o[6]), "+a"(o[7]),
                 "+a"(o[8]), "+a"(o[9]), "+a"(o[10]), "+a"(o[11]), "+a"(o[12]), "+a"(o[13]), "+a"(o[14]), "+a"(o[15]));
}

__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
  // round-to-nearest-even; inputs are finite and non-negative probabilities or dequantised values
  typedef __attribute__((ext_vector_type(2))) __bf16 v2;
  v2 r;
  r[0] = (__bf16)a;
  r[1] = (__bf16)b;
  return __builtin_bit_cast(unsigned, r);
}

__device__ __forceinline__ unsigned pack_f16(float a, float b) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 r;
  r[0] = (_Float16)a;
  r[1] = (_Float16)b;
  return __builtin_bit_cast(unsigned, r);
}

__device__ __forceinline__ bool scale_is_pow2(float s) {
  const unsigned u = __float_as_uint(s);
  const unsigned e = u >> 23;                 // sign + exponent
  return (u & 0x007fffffu) == 0u && e >= 1u && e <= 254u;
}

// 16 e4m3 bytes * scale -> 16 bf16 (two 16-byte LDS chunks).  POW2: the scale is a
// normal power of two, which the converter applies exactly (it only looks at the
// exponent of its scale operand); otherwise convert unscaled and multiply in fp32.
template <bool POW2>
__device__ __forceinline__ void dequant16(const uint4 raw, float scale, uint4& lo, uint4& hi) {
  const unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
  unsigned o[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (POW2) {
      o[2 * i] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[i], scale, false));
      o[2 * i + 1] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[i], scale, true));
    } else {
      const f32x2 a = e4m3x2_lo(w[i]), b = e4m3x2_hi(w[i]);
      o[2 * i] = pack_bf16(a[0] * scale, a[1] * scale);
      o[2 * i + 1] = pack_bf16(b[0] * scale, b[1] * scale);
    }
  }
  lo = make_uint4(o[0], o[1], o[2], o[3]);
  hi = make_uint4(o[4], o[5], o[6], o[7]);
}

// value of lane (lane ^ 16) / (lane ^ 32), VALU only
__device__ __forceinline__ float xor16(float v) {
  const unsigned u = __float_as_uint(v);
  const u32x2 r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __uint_as_float((lane_id() & 16) ? r[0] : r[1]);
}
__device__ __forceinline__ float xor32(float v) {
  const unsigned u = __float_as_uint(v);
  const u32x2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float((lane_id() & 32) ? r[0] : r[1]);
}

}  // namespace cm
