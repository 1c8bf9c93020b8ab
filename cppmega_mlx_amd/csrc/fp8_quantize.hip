// FP8 (e4m3) producers for the sparse-attention path (gfx950): the quantisers that write the
// prepared buffers the attention kernels consume, and the matching dequantiser.
//
//   per token   scale[row] = max(amax(row) * (1/448), 1e-12); code = rne(clamp(x / scale, +-448))
//   per tensor  the same with one amax over the whole tensor, the scale replicated per row
//   mxfp8       per 32 channels: byte = clamp(127 + ceil(log2(amax / 448)), 1, 254) (127 for an
//               all-zero block); code = rne(clamp(x / 2^(byte-127), +-448))
//
// One wavefront per row.  Besides codes and scales a call can ask for the round trip
// dec(code) * scale in the input's dtype, which is what the float-carrier attention wrappers
// feed to the attention kernel.

#include "common.h"

namespace cm {
namespace {

struct QuantParams {
  const void* x;
  unsigned char* codes;
  void* scale;           // float32 [rows] (per token / per tensor) or uint8 [rows, k/32] (mxfp8)
  void* recovered;
  const unsigned char* in_codes;   // dequantise: source bytes
  long long rows;
  int k;
  int x_dtype;
  int mode;
};

// round-to-nearest-even onto the e4m3fn grid; |v| <= 448, v not NaN
__device__ __forceinline__ unsigned e4m3_encode(float v) {
  const unsigned u = __float_as_uint(v);
  const unsigned sign = (u >> 24) & 0x80u;
  const float a = fabsf(v);
  unsigned code;
  if (a < 0.015625f) {                          // below 2^-6: the subnormal grid m * 2^-9
    code = (unsigned)__builtin_rintf(a * 512.0f);          // 0..8 (8 is the first normal code)
  } else {
    unsigned m = __float_as_uint(a);
    m += 0x7ffffu + ((m >> 20) & 1u);           // keep three mantissa bits, ties to even
    code = (m >> 20) - (120u << 3);             // rebias 127 -> 7
    code = min(code, 0x7eu);
  }
  return sign | code;
}

__device__ __forceinline__ float wave_max_f(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// amax over the whole tensor -> amax_bits[0] (as uint; non-negative floats order like uints)
__global__ __launch_bounds__(256) void tensor_amax_kernel(const QuantParams p, unsigned* amax_bits) {
  const size_t n = (size_t)p.rows * p.k;
  float m = 0.0f;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    m = fmaxf(m, fabsf(load_as(p.x, i, p.x_dtype)));
  m = wave_max_f(m);
  if ((threadIdx.x & 63) == 0) atomicMax(amax_bits, __float_as_uint(m));
}
__global__ void zero_word_kernel(unsigned* w) { *w = 0u; }

// MODE 0: per token, 1: per tensor (amax at amax_bits[0]), 2: mxfp8
template <int MODE>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const QuantParams p, const unsigned* amax_bits) {
  const int lane = lane_id();
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.rows) return;
  const size_t base = (size_t)row * p.k;
  if (MODE == 2) {
    // a half-wavefront (32 lanes) owns one 32-channel block per step
    const int half = lane >> 5, l32 = lane & 31;
    const int blocks = p.k / 32;
    for (int b0 = 0; b0 < blocks; b0 += 2) {
      const int blk = b0 + half;
      const bool live = blk < blocks;
      const float v = live ? load_as(p.x, base + (size_t)blk * 32 + l32, p.x_dtype) : 0.0f;
      float am = fabsf(v);
#pragma unroll
      for (int off = 16; off >= 1; off >>= 1) am = fmaxf(am, __shfl_xor(am, off, 64));
      // smallest e with 448 * 2^e >= amax:  amax = m * 2^E, m in [1,2)  ->  e = E - 8 + (m > 1.75)
      int e = 0;
      if (am > 0.0f) {
        int ex;
        const float fr = frexpf(am, &ex);       // am = fr * 2^ex, fr in [0.5, 1)
        e = (ex - 1) - 8 + (fr > 0.875f ? 1 : 0);
      }
      const int byte = min(max(e + 127, 1), 254);
      const float inv = ldexpf(1.0f, 127 - byte), sc = ldexpf(1.0f, byte - 127);
      const float nv = fminf(fmaxf(v * inv, -448.0f), 448.0f);
      const unsigned code = e4m3_encode(nv);
      if (live) {
        if (p.codes) p.codes[base + (size_t)blk * 32 + l32] = (unsigned char)code;
        if (p.scale && l32 == 0) ((unsigned char*)p.scale)[(size_t)row * blocks + blk] = (unsigned char)byte;
        if (p.recovered) store_as(p.recovered, base + (size_t)blk * 32 + l32, p.x_dtype, e4m3_to_f32((unsigned char)code) * sc);
      }
    }
    return;
  }
  float am;
  if (MODE == 0) {
    am = 0.0f;
    for (int c = lane; c < p.k; c += 64) am = fmaxf(am, fabsf(load_as(p.x, base + c, p.x_dtype)));
    am = wave_max_f(am);
  } else {
    am = __uint_as_float(amax_bits[0]);
  }
  const float sc = fmaxf(am * (1.0f / 448.0f), 1.0e-12f);
  if (p.scale && lane == 0) ((float*)p.scale)[row] = sc;
  for (int c = lane; c < p.k; c += 64) {
    const float v = load_as(p.x, base + c, p.x_dtype);
    const float nv = fminf(fmaxf(__fdiv_rn(v, sc), -448.0f), 448.0f);
    const unsigned code = e4m3_encode(nv);
    if (p.codes) p.codes[base + c] = (unsigned char)code;
    if (p.recovered) store_as(p.recovered, base + c, p.x_dtype, e4m3_to_f32((unsigned char)code) * sc);
  }
}

// recovered[row, c] = dec(in_codes[row, c]) * scale  (MODE 2: E8M0 byte per 32 channels, else float32 per row)
template <int MODE>
__global__ __launch_bounds__(256) void dequantize_rows_kernel(const QuantParams p) {
  const size_t n = (size_t)p.rows * p.k;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    const size_t row = i / p.k;
    const int c = (int)(i - row * p.k);
    const float sc = MODE == 2 ? e8m0_to_f32(((const unsigned char*)p.scale)[row * (p.k / 32) + (c >> 5)])
                               : ((const float*)p.scale)[row];
    store_as(p.recovered, i, p.x_dtype, e4m3_to_f32(p.in_codes[i]) * sc);
  }
}

}  // namespace

int fp8_quantize_launch(const cppmega_mi355_quantize_args_t& a, hipStream_t stream) {
  if (a.rows < 0 || a.k < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "fp8_quantize: rows=%lld k=%d", (long long)a.rows, a.k);
  if (a.x_dtype != CPPMEGA_MI355_F32 && a.x_dtype != CPPMEGA_MI355_F16 && a.x_dtype != CPPMEGA_MI355_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "fp8_quantize: dtype %d is not float32/float16/bfloat16", a.x_dtype);
  if (a.mode < CPPMEGA_MI355_QUANT_PER_TOKEN || a.mode > CPPMEGA_MI355_DEQUANT_MXFP8)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "fp8_quantize: unknown mode %d", a.mode);
  const bool mx = a.mode == CPPMEGA_MI355_QUANT_MXFP8 || a.mode == CPPMEGA_MI355_DEQUANT_MXFP8;
  if (mx && a.k % 32 != 0) return fail(CPPMEGA_MI355_ERR_SHAPE, "fp8_quantize: MXFP8 last dim must be divisible by 32, got %d", a.k);
  if (a.rows == 0) return 0;
  QuantParams p;
  p.x = a.x; p.codes = a.codes; p.scale = a.scale; p.recovered = a.recovered; p.in_codes = a.codes;
  p.rows = a.rows; p.k = a.k; p.x_dtype = a.x_dtype; p.mode = a.mode;
  if (a.mode >= CPPMEGA_MI355_DEQUANT_PER_TOKEN) {
    if (!a.codes || !a.scale || !a.recovered) return fail(CPPMEGA_MI355_ERR_NULL, "fp8_dequantize: codes/scale/recovered is NULL");
    const size_t n = (size_t)a.rows * a.k;
    const unsigned blocks = (unsigned)min((n + 255) / 256, (size_t)65535 * 16);
    if (mx) hipLaunchKernelGGL(dequantize_rows_kernel<2>, dim3(blocks), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(dequantize_rows_kernel<0>, dim3(blocks), dim3(256), 0, stream, p);
    CM_HIP_CHECK(hipGetLastError());
    return 0;
  }
  if (!a.x) return fail(CPPMEGA_MI355_ERR_NULL, "fp8_quantize: x is NULL");
  if (!a.codes && !a.recovered && !a.scale) return fail(CPPMEGA_MI355_ERR_NULL, "fp8_quantize: no output requested");
  const dim3 grid((unsigned)((a.rows + 3) / 4)), block(256);
  if (a.mode == CPPMEGA_MI355_QUANT_PER_TOKEN) {
    hipLaunchKernelGGL(quantize_rows_kernel<0>, grid, block, 0, stream, p, (const unsigned*)nullptr);
  } else if (a.mode == CPPMEGA_MI355_QUANT_MXFP8) {
    hipLaunchKernelGGL(quantize_rows_kernel<2>, grid, block, 0, stream, p, (const unsigned*)nullptr);
  } else {
    // the whole-tensor amax is gathered in the first word of the caller's 4-byte scratch
    if (!a.scratch) return fail(CPPMEGA_MI355_ERR_WORKSPACE, "fp8_quantize: per-tensor mode needs a 4-byte scratch word");
    unsigned* word = (unsigned*)a.scratch;
    hipLaunchKernelGGL(zero_word_kernel, dim3(1), dim3(1), 0, stream, word);
    const size_t n = (size_t)a.rows * a.k;
    const unsigned blocks = (unsigned)min((n + 255) / 256, (size_t)2048);
    hipLaunchKernelGGL(tensor_amax_kernel, dim3(blocks), dim3(256), 0, stream, p, word);
    hipLaunchKernelGGL(quantize_rows_kernel<1>, grid, block, 0, stream, p, (const unsigned*)word);
  }
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
