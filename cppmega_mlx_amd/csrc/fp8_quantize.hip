// FP8 (e4m3) producers for the sparse-attention path (gfx950): the quantisers that write the
// prepared buffers the attention kernels consume, and the matching dequantiser.
//
//   per token   scale[row] = max(amax(row) * (1/448), 1e-12); code = rne(clamp(x / scale, +-448))
//   per tensor  the same with one amax over the whole tensor, the scale replicated per row
//   mxfp8       per 32 channels: byte = clamp(127 + rint(log2(amax / 448)), 1, 254) (127 for an
//               all-zero block; the exponent rounds to nearest, so values up to sqrt(2) above
//               the scaled range saturate); code = rne(clamp(x / 2^(byte-127), +-448))
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
      // e = rint(log2(amax / 448)):  amax = fr * 2^ex, fr in [0.5, 1), 448 = 0.875 * 2^9, so
      // log2(amax / 448) = (ex - 9) + log2(fr / 0.875) with the last term in [-0.81, 0.19): it
      // rounds to -1 iff fr / 0.875 < 2^-0.5, i.e. fr^2 < 0.875^2 / 2 (exact in double).
      int e = 0;
      if (am > 0.0f) {
        int ex;
        const float fr = frexpf(am, &ex);
        e = ex - 10 + ((double)fr * (double)fr > 0.3828125 ? 1 : 0);
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


// the bare conversions: codes = rne(clamp(x, +-448)) / recovered = dec(codes)
template <bool ENCODE>
__global__ __launch_bounds__(256) void unit_convert_kernel(const QuantParams p) {
  const size_t n = (size_t)p.rows * p.k;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    if (ENCODE) {
      const float v = load_as(p.x, i, p.x_dtype);
      const unsigned code = v != v ? (((__float_as_uint(v) >> 24) & 0x80u) | 0x7fu) : e4m3_encode(fminf(fmaxf(v, -448.0f), 448.0f));
      p.codes[i] = (unsigned char)code;
    } else {
      store_as(p.recovered, i, p.x_dtype, e4m3_to_f32(p.in_codes[i]));
    }
  }
}

// ---- cache append -------------------------------------------------------------------------
struct AppendParams {
  const void* src;
  const float* src_scale;
  const void* rope;
  unsigned char* kv_cache;
  float* scale_cache;
  unsigned short* rope_cache;
  const int* positions;
  int position;
  int B, S, G, D, R, cap;
  int src_dtype, rope_dtype, scale_block, pow2;
};

// One wavefront per new (batch, token, group) row.  A lane owns 8 consecutive channels of every
// 512-channel piece, so a 128-channel block is 16 lanes and its amax four butterfly steps.
template <bool PREPARED>
__global__ __launch_bounds__(256) void cache_append_kernel(const AppendParams p) {
  const int lane = lane_id();
  // (32-bit arithmetic, the launcher checks that the row count fits: 64-bit divisions per
  // wavefront were most of this kernel's instructions)
  const unsigned row = blockIdx.x * 4u + (threadIdx.x >> 6);                  // (b * S + s) * G + g
  const unsigned rows = (unsigned)p.B * (unsigned)p.S * (unsigned)p.G;
  if (row >= rows) return;
  const unsigned bs = row / (unsigned)p.G;
  const int g = (int)(row - bs * (unsigned)p.G);
  const int b = (int)(bs / (unsigned)p.S), s = (int)(bs - (unsigned)b * (unsigned)p.S);
  const int pos = (p.positions ? p.positions[b] : p.position) + s;
  if (pos < 0 || pos >= p.cap) return;                                         // (checked on the host when positions is NULL)
  const size_t crow = ((size_t)b * p.cap + pos) * p.G + g;                     // cache row
  const int nsc = p.scale_block ? p.D / p.scale_block : 1;
  const size_t sbase = (size_t)row * p.D;
  if (PREPARED) {
    for (int c = lane * 16; c < p.D; c += 64 * 16)
      *reinterpret_cast<uint4*>(p.kv_cache + crow * p.D + c) = *reinterpret_cast<const uint4*>((const unsigned char*)p.src + sbase + c);
    if (lane < nsc) p.scale_cache[crow * nsc + lane] = p.src_scale[(size_t)row * nsc + lane];
  } else {
    constexpr int kMaxPieces = 4;                                              // D <= 2048
    float v[kMaxPieces][8];
    float am[kMaxPieces];
    const int pieces = (p.D + 511) / 512;
#pragma unroll
    for (int pc = 0; pc < kMaxPieces; ++pc) {
      am[pc] = 0.0f;
      const int c0 = pc * 512 + lane * 8;
      const bool live = pc < pieces && c0 < p.D;           // (D % 128 == 0: a lane's 8 channels are all in or all out)
      if (live && p.src_dtype != CPPMEGA_MI355_F32) {      // 16-bit sources: one 16-byte load
        const uint4 t = *reinterpret_cast<const uint4*>((const unsigned short*)p.src + sbase + c0);
        const unsigned w[4] = {t.x, t.y, t.z, t.w};
        const bool bf = p.src_dtype == CPPMEGA_MI355_BF16;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const unsigned short lo = (unsigned short)(w[i] & 0xffffu), hi = (unsigned short)(w[i] >> 16);
          v[pc][2 * i] = bf ? bf16_bits_to_f32(lo) : f16_bits_to_f32(lo);
          v[pc][2 * i + 1] = bf ? bf16_bits_to_f32(hi) : f16_bits_to_f32(hi);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[pc][i] = live ? load_as(p.src, sbase + c0 + i, p.src_dtype) : 0.0f;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) am[pc] = fmaxf(am[pc], fabsf(v[pc][i]));
#pragma unroll
      for (int off = 1; off <= 8; off <<= 1) am[pc] = fmaxf(am[pc], __shfl_xor(am[pc], off, 64));   // the lane's 128-channel block
    }
    float row_am = 0.0f;
    if (!p.scale_block) {
#pragma unroll
      for (int pc = 0; pc < kMaxPieces; ++pc) row_am = fmaxf(row_am, am[pc]);
      row_am = wave_max_f(row_am);
    }
#pragma unroll
    for (int pc = 0; pc < kMaxPieces; ++pc) {
      if (pc >= pieces) break;
      const int c0 = pc * 512 + lane * 8;
      if (c0 >= p.D) continue;
      const float a = p.scale_block ? am[pc] : row_am;
      float sc;
      if (p.pow2) {
        // smallest power of two s with 448 * s >= amax:  amax = fr * 2^ex, fr in [0.5, 1)
        sc = 1.0f;
        if (a > 0.0f) {
          int ex;
          const float fr = frexpf(a, &ex);
          sc = ldexpf(1.0f, (ex - 1) - 8 + (fr > 0.875f ? 1 : 0));
        }
      } else {
        sc = fmaxf(a * (1.0f / 448.0f), 1.0e-12f);
      }
      unsigned w0 = 0, w1 = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float nv = fminf(fmaxf(__fdiv_rn(v[pc][i], sc), -448.0f), 448.0f);
        const unsigned code = e4m3_encode(nv);
        if (i < 4) w0 |= code << (8 * i); else w1 |= code << (8 * (i - 4));
      }
      *reinterpret_cast<uint2*>(p.kv_cache + crow * p.D + c0) = make_uint2(w0, w1);
      if (p.scale_block) {
        if ((lane & 15) == 0) p.scale_cache[crow * nsc + (c0 >> 7)] = sc;
      } else if (lane == 0 && pc == 0) {
        p.scale_cache[crow] = sc;
      }
    }
  }
  if (p.rope_cache) {
    for (int c = lane; c < p.R; c += 64)
      store_as(p.rope_cache, crow * p.R + c, CPPMEGA_MI355_BF16, load_as(p.rope, (size_t)row * p.R + c, p.rope_dtype));
  }
}

}  // namespace

int fp8_quantize_launch(const cppmega_mi355_quantize_args_t& a, hipStream_t stream) {
  if (a.rows < 0 || a.k < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "fp8_quantize: rows=%lld k=%d", (long long)a.rows, a.k);
  if (a.x_dtype != CPPMEGA_MI355_F32 && a.x_dtype != CPPMEGA_MI355_F16 && a.x_dtype != CPPMEGA_MI355_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "fp8_quantize: dtype %d is not float32/float16/bfloat16", a.x_dtype);
  if (a.mode < CPPMEGA_MI355_QUANT_PER_TOKEN || a.mode > CPPMEGA_MI355_DEQUANT_UNIT)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "fp8_quantize: unknown mode %d", a.mode);
  const bool mx = a.mode == CPPMEGA_MI355_QUANT_MXFP8 || a.mode == CPPMEGA_MI355_DEQUANT_MXFP8;
  if (mx && a.k % 32 != 0) return fail(CPPMEGA_MI355_ERR_SHAPE, "fp8_quantize: MXFP8 last dim must be divisible by 32, got %d", a.k);
  if (a.rows == 0) return 0;
  QuantParams p;
  p.x = a.x; p.codes = a.codes; p.scale = a.scale; p.recovered = a.recovered; p.in_codes = a.codes;
  p.rows = a.rows; p.k = a.k; p.x_dtype = a.x_dtype; p.mode = a.mode;
  if (a.mode == CPPMEGA_MI355_QUANT_UNIT || a.mode == CPPMEGA_MI355_DEQUANT_UNIT) {
    const bool enc = a.mode == CPPMEGA_MI355_QUANT_UNIT;
    if (!a.codes || (enc ? !a.x : !a.recovered)) return fail(CPPMEGA_MI355_ERR_NULL, "fp8_quantize: the bare conversions need codes and %s", enc ? "x" : "recovered");
    const size_t n = (size_t)a.rows * a.k;
    const unsigned blocks = (unsigned)min((n + 255) / 256, (size_t)65535 * 16);
    if (enc) hipLaunchKernelGGL(unit_convert_kernel<true>, dim3(blocks), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(unit_convert_kernel<false>, dim3(blocks), dim3(256), 0, stream, p);
    CM_HIP_CHECK(hipGetLastError());
    return 0;
  }
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

int kv_cache_append_launch(const cppmega_mi355_cache_append_args_t& a, hipStream_t stream) {
  if (a.batch < 1 || a.new_tokens < 0 || a.groups < 1 || a.dim < 1 || a.capacity < 1 || a.rope_dim < 0)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "kv_cache_append: B=%d S_new=%d G=%d D=%d R=%d capacity=%d", a.batch, a.new_tokens, a.groups, a.dim, a.rope_dim, a.capacity);
  if (a.dim % 128 != 0 || a.dim > 2048 || a.rope_dim > 256)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "kv_cache_append: D must be a multiple of 128 up to 2048 and R <= 256, got D=%d R=%d", a.dim, a.rope_dim);
  if (a.scale_block != 0 && a.scale_block != 128)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "kv_cache_append: scale_block must be 0 (per row) or 128, got %d", a.scale_block);
  const bool prepared = a.src_dtype == CPPMEGA_MI355_E4M3;
  if (!prepared && a.src_dtype != CPPMEGA_MI355_F32 && a.src_dtype != CPPMEGA_MI355_F16 && a.src_dtype != CPPMEGA_MI355_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "kv_cache_append: source dtype %d", a.src_dtype);
  if (a.new_tokens == 0) return 0;
  if (!a.src || !a.kv_cache || !a.scale_cache || (prepared && !a.src_scale))
    return fail(CPPMEGA_MI355_ERR_NULL, "kv_cache_append: src / src_scale / kv_cache / scale_cache is NULL");
  const bool with_rope = a.rope_dim > 0 && a.rope_cache != nullptr;
  if (with_rope) {
    if (!a.rope) return fail(CPPMEGA_MI355_ERR_NULL, "kv_cache_append: rope cache given but no rope rows");
    if (a.rope_dtype != CPPMEGA_MI355_F32 && a.rope_dtype != CPPMEGA_MI355_F16 && a.rope_dtype != CPPMEGA_MI355_BF16)
      return fail(CPPMEGA_MI355_ERR_DTYPE, "kv_cache_append: rope dtype %d", a.rope_dtype);
  }
  if (!a.positions && (a.position < 0 || (long long)a.position + a.new_tokens > a.capacity))
    return fail(CPPMEGA_MI355_ERR_SHAPE, "kv_cache_append: positions %d..%lld exceed the capacity %d", a.position, (long long)a.position + a.new_tokens, a.capacity);
  if (((size_t)a.src | (size_t)a.kv_cache) & 15)
    return fail(CPPMEGA_MI355_ERR_ALIGNMENT, "kv_cache_append: src and kv_cache must be 16-byte aligned");
  AppendParams p;
  p.src = a.src; p.src_scale = a.src_scale; p.rope = a.rope; p.kv_cache = a.kv_cache; p.scale_cache = a.scale_cache;
  p.rope_cache = with_rope ? (unsigned short*)a.rope_cache : nullptr;
  p.positions = a.positions; p.position = a.position;
  p.B = a.batch; p.S = a.new_tokens; p.G = a.groups; p.D = a.dim; p.R = a.rope_dim; p.cap = a.capacity;
  p.src_dtype = a.src_dtype; p.rope_dtype = a.rope_dtype; p.scale_block = a.scale_block; p.pow2 = a.pow2_scales;
  const long long rows = (long long)a.batch * a.new_tokens * a.groups;
  if (rows > 0x7fffffffll) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "kv_cache_append: %lld rows in one call", rows);
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  if (prepared) hipLaunchKernelGGL(cache_append_kernel<true>, grid, block, 0, stream, p);
  else hipLaunchKernelGGL(cache_append_kernel<false>, grid, block, 0, stream, p);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
