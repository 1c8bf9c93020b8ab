// Per-head projections around the latent attention call, and the block-128 FP8 weight dequantiser.
//
// The reference's absorbed MLA decode (cppmega_v4/nn/mla_absorb.py:39-138) folds the key
// up-projection into the query and the value up-projection into the output:
//
//   q_abs[b,t,h,:] = q[b,t,h,:] . W_UK^T[h]            "bthk,hkv->bthv"   (:118)
//   out[b,t,:]     = sum_h v_abs[b,t,h,:] . (W_UV W_O)[h]   "bthv,hvm->btm"   (:133)
//
// Both are one shape of work: Y[m, g, n] = sum_k X[m, g, k] * W[g, n, k], a skinny matrix
// product per group g (a head; or one group whose contraction runs over all heads), with few
// rows m at decode time, so the weights stream from memory once and that stream is the cost.
// head_gemm_kernel keeps the weights in the layout where the contraction index is contiguous
// (W[g][n][k], what absorb_weights prepares once at load time):
//
//   * a workgroup (4 wavefronts) owns 64 output channels n of one group and up to 64 rows m;
//   * the rows' X values for a chunk of 512 k go to LDS as bf16 (fp32 inputs as bf16 hi + lo,
//     16 significand bits);
//   * W rows are the MFMA's A operand, loaded straight from memory 16 bytes per lane
//     (fp32 weights split into hi + lo on the way), the X rows its B operand from LDS:
//     v_mfma_f32_16x16x32_bf16, fp32 accumulation over the whole contraction;
//   * a lane ends with four consecutive n of one row m and writes them in one store; the output
//     has its own row and group pitch, so q_abs can land inside the [.., 576]-wide query rows the
//     attention kernel takes.
//
// dequant_grid128_kernel restates dequant_block_fp8
// (cppmega_v4/nn/_external/_mlx_lm_fp8_dequant_vendored.py:24-46): e4m3 byte -> bf16 (exact),
// times the float32 scale of its 128 x 128 block in fp32, rounded to the output type.

#include "common.h"

namespace cm {
namespace {

constexpr int kThreads = 256;
constexpr int kNPerWg = 64;       // output channels per workgroup: 4 wavefronts x 16
constexpr int kKChunk = 512;      // contraction elements staged in LDS at a time
constexpr int kPitch = kKChunk + 8;

struct HeadGemmParams {
  const void* x;
  const void* w;
  void* y;
  int x_dtype, w_dtype, y_dtype;
  int M, G, N, K;
  long long xs_m, xs_g, ys_m, ys_g;   // pitches in elements
  int x_vec, w_vec;                   // 16-byte loads allowed
};

__device__ __forceinline__ void split_bf16(float v, unsigned short& hi, unsigned short& lo) {
  hi = f32_to_bf16_bits(v);
  lo = f32_to_bf16_bits(v - bf16_bits_to_f32(hi));
}

__device__ __forceinline__ bf16x8 pack8(const unsigned short (&e)[8]) {
  return __builtin_bit_cast(bf16x8, make_uint4(e[0] | ((unsigned)e[1] << 16), e[2] | ((unsigned)e[3] << 16),
                                               e[4] | ((unsigned)e[5] << 16), e[6] | ((unsigned)e[7] << 16)));
}

template <bool X_F32, bool W_F32, int MT>
__global__ __launch_bounds__(kThreads) void head_gemm_kernel(const HeadGemmParams p) {
  extern __shared__ __align__(16) unsigned short x_lds[];       // [X_F32 ? 2 : 1][16 MT][kPitch]
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = (int)blockIdx.y;
  const int m0 = 16 * MT * (int)blockIdx.z;
  const int rows_here = min(16 * MT, p.M - m0);
  const int n = lane & 15, kg = lane >> 4;
  const int n_row = (int)blockIdx.x * kNPerWg + 16 * wave + n;   // the W row this lane feeds to the A operand
  const int n_clamped = min(n_row, p.N - 1);
  unsigned short* x_hi = x_lds;
  unsigned short* x_lo = x_lds + 16 * MT * kPitch;
  const size_t w_row = ((size_t)g * p.N + (size_t)n_clamped) * (size_t)p.K;

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  for (int kc = 0; kc < p.K; kc += kKChunk) {
    const int klen = min(kKChunk, p.K - kc);
    const int kpad = (klen + 31) & ~31;
    __syncthreads();                                            // the previous chunk has been consumed
    for (int e = tid; e < 16 * MT * (kpad / 8); e += kThreads) {
      const int r = e / (kpad / 8), c = e % (kpad / 8);
      unsigned short hi[8] = {0, 0, 0, 0, 0, 0, 0, 0}, lo[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (r < rows_here) {
        const size_t at = (size_t)(m0 + r) * p.xs_m + (size_t)g * p.xs_g + (size_t)(kc + 8 * c);
        if (!X_F32 && p.x_vec && 8 * c + 8 <= klen) {
          const uint4 t = *reinterpret_cast<const uint4*>((const unsigned short*)p.x + at);
          const unsigned u[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) { hi[2 * i] = (unsigned short)(u[i] & 0xffffu); hi[2 * i + 1] = (unsigned short)(u[i] >> 16); }
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            if (8 * c + i < klen) {
              if (X_F32) split_bf16(((const float*)p.x)[at + i], hi[i], lo[i]);
              else hi[i] = ((const unsigned short*)p.x)[at + i];
            }
          }
        }
      }
      *reinterpret_cast<bf16x8*>(&x_hi[r * kPitch + 8 * c]) = pack8(hi);
      if (X_F32) *reinterpret_cast<bf16x8*>(&x_lo[r * kPitch + 8 * c]) = pack8(lo);
    }
    __syncthreads();
#pragma unroll 4
    for (int ks = 0; ks < kpad / 32; ++ks) {
      const int d0 = 32 * ks + 8 * kg;
      unsigned short wh[8] = {0, 0, 0, 0, 0, 0, 0, 0}, wl[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      const size_t at = w_row + (size_t)(kc + d0);
      if (!W_F32) {
        if (p.w_vec && d0 + 8 <= klen) {
          const uint4 t = *reinterpret_cast<const uint4*>((const unsigned short*)p.w + at);
          const unsigned u[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) { wh[2 * i] = (unsigned short)(u[i] & 0xffffu); wh[2 * i + 1] = (unsigned short)(u[i] >> 16); }
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (d0 + i < klen) wh[i] = ((const unsigned short*)p.w)[at + i];
        }
      } else {
        float v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (p.w_vec && d0 + 8 <= klen) {
          const float4 t0 = *reinterpret_cast<const float4*>((const float*)p.w + at);
          const float4 t1 = *reinterpret_cast<const float4*>((const float*)p.w + at + 4);
          v[0] = t0.x; v[1] = t0.y; v[2] = t0.z; v[3] = t0.w; v[4] = t1.x; v[5] = t1.y; v[6] = t1.z; v[7] = t1.w;
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (d0 + i < klen) v[i] = ((const float*)p.w)[at + i];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) split_bf16(v[i], wh[i], wl[i]);
      }
      const bf16x8 a_hi = pack8(wh), a_lo = pack8(wl);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 b_hi = *reinterpret_cast<const bf16x8*>(&x_hi[(16 * mt + n) * kPitch + d0]);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b_hi, acc[mt], 0, 0, 0);
        if (W_F32) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b_hi, acc[mt], 0, 0, 0);
        if (X_F32) {
          const bf16x8 b_lo = *reinterpret_cast<const bf16x8*>(&x_lo[(16 * mt + n) * kPitch + d0]);
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b_lo, acc[mt], 0, 0, 0);
        }
      }
    }
  }
  // lane (n, kg): row m0 + 16 mt + n of X, output channels n_out .. n_out + 3
  const int n_out = (int)blockIdx.x * kNPerWg + 16 * wave + 4 * kg;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = 16 * mt + n;
    if (r >= rows_here) continue;
    const size_t at = (size_t)(m0 + r) * p.ys_m + (size_t)g * p.ys_g + (size_t)n_out;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n_out + i < p.N) store_as(p.y, at + i, p.y_dtype, acc[mt][i]);
  }
}

template <bool X_F32, bool W_F32>
void launch_head_gemm(const HeadGemmParams& p, hipStream_t stream) {
  const int mt = p.M <= 16 ? 1 : (p.M <= 32 ? 2 : 4);
  const dim3 grid((unsigned)((p.N + kNPerWg - 1) / kNPerWg), (unsigned)p.G, (unsigned)((p.M + 16 * mt - 1) / (16 * mt)));
  const size_t lds = (size_t)(X_F32 ? 2 : 1) * 16 * mt * kPitch * sizeof(unsigned short);   // <= 133 KB
  auto go = [&](auto kernel) {
    if (lds > 64 * 1024) (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds, stream, p);
  };
  if (mt == 1) go(head_gemm_kernel<X_F32, W_F32, 1>);
  else if (mt == 2) go(head_gemm_kernel<X_F32, W_F32, 2>);
  else go(head_gemm_kernel<X_F32, W_F32, 4>);
}

struct DequantParams {
  const unsigned char* w;
  const float* scale;
  void* out;
  int rows, cols, scale_cols, out_dtype;
};

// one thread per 8 consecutive columns of a row
__global__ __launch_bounds__(kThreads) void dequant_grid128_kernel(const DequantParams p) {
  const int groups = (p.cols + 7) / 8;
  const size_t slot = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (slot >= (size_t)p.rows * groups) return;
  const int r = (int)(slot / groups), c0 = 8 * (int)(slot % groups);
  const size_t at = (size_t)r * p.cols + c0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (c0 + i >= p.cols) break;
    const unsigned char byte = p.w[at + i];
    const float s = p.scale[(size_t)(r / 128) * p.scale_cols + (c0 + i) / 128];
    const float v = ((byte & 0x7f) == 0x7f) ? __uint_as_float(0x7fc00000u) : e4m3_to_f32(byte) * s;
    store_as(p.out, at + i, p.out_dtype, v);
  }
}

}  // namespace

int head_gemm_launch(const cppmega_mi355_head_gemm_args_t& a, hipStream_t stream) {
  if (!a.x || !a.w || !a.y) return fail(CPPMEGA_MI355_ERR_NULL, "head_gemm: x/w/y is NULL");
  if (a.m < 0 || a.groups < 1 || a.n < 1 || a.k < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "head_gemm: m=%d groups=%d n=%d k=%d", a.m, a.groups, a.n, a.k);
  if (a.groups > 65535) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "head_gemm: at most 65535 groups");
  const int fl[2] = {a.x_dtype, a.w_dtype};
  for (int i = 0; i < 2; ++i)
    if (fl[i] != CPPMEGA_MI355_F32 && fl[i] != CPPMEGA_MI355_BF16)
      return fail(CPPMEGA_MI355_ERR_DTYPE, "head_gemm: x and w must be float32 or bfloat16");
  if (a.y_dtype != CPPMEGA_MI355_F32 && a.y_dtype != CPPMEGA_MI355_BF16 && a.y_dtype != CPPMEGA_MI355_F16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "head_gemm: y must be float32, float16 or bfloat16");
  if (a.x_row_pitch < 0 || a.x_group_pitch < 0 || a.y_row_pitch < 0 || a.y_group_pitch < 0)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "head_gemm: negative pitch");
  if (a.m == 0) return 0;
  if ((a.m + 63) / 64 > 65535) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "head_gemm: m %d too large for one launch", a.m);
  HeadGemmParams p;
  p.x = a.x; p.w = a.w; p.y = a.y;
  p.x_dtype = a.x_dtype; p.w_dtype = a.w_dtype; p.y_dtype = a.y_dtype;
  p.M = a.m; p.G = a.groups; p.N = a.n; p.K = a.k;
  p.xs_m = a.x_row_pitch; p.xs_g = a.x_group_pitch; p.ys_m = a.y_row_pitch; p.ys_g = a.y_group_pitch;
  p.x_vec = a.x_dtype == CPPMEGA_MI355_BF16 && ((uintptr_t)a.x & 15) == 0 && a.x_row_pitch % 8 == 0 && a.x_group_pitch % 8 == 0;
  p.w_vec = ((uintptr_t)a.w & 15) == 0 && a.k % 8 == 0;
  const bool xf = a.x_dtype == CPPMEGA_MI355_F32, wf = a.w_dtype == CPPMEGA_MI355_F32;
  if (xf && wf) launch_head_gemm<true, true>(p, stream);
  else if (xf) launch_head_gemm<true, false>(p, stream);
  else if (wf) launch_head_gemm<false, true>(p, stream);
  else launch_head_gemm<false, false>(p, stream);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

int dequant_block_fp8_launch(const cppmega_mi355_dequant_block_args_t& a, hipStream_t stream) {
  if (!a.weight || !a.scale_inv || !a.out) return fail(CPPMEGA_MI355_ERR_NULL, "dequant_block_fp8: weight/scale_inv/out is NULL");
  if (a.rows < 0 || a.cols < 0) return fail(CPPMEGA_MI355_ERR_SHAPE, "dequant_block_fp8: rows=%d cols=%d", a.rows, a.cols);
  if (a.out_dtype != CPPMEGA_MI355_F32 && a.out_dtype != CPPMEGA_MI355_BF16 && a.out_dtype != CPPMEGA_MI355_F16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "dequant_block_fp8: out must be float32, float16 or bfloat16");
  if ((size_t)a.rows * a.cols == 0) return 0;
  DequantParams p;
  p.w = (const unsigned char*)a.weight; p.scale = a.scale_inv; p.out = a.out;
  p.rows = a.rows; p.cols = a.cols; p.scale_cols = (a.cols + 127) / 128; p.out_dtype = a.out_dtype;
  const size_t slots = (size_t)a.rows * ((a.cols + 7) / 8);
  hipLaunchKernelGGL(dequant_grid128_kernel, dim3((unsigned)((slots + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, p);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
