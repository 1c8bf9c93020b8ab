// FP8 (e4m3) block-scaled vecmat / skinny GEMM for decode projections (gfx950).
//
//   out[m, n] = sum_k dec(w[n, k]) * w_scale(n, k / 128) * x[m, k]
//
// The weight is read from HBM exactly once; everything else is sized so that
// the weight stream is the only traffic that matters.
//
//  * M <= 4 (M == 1 for e4m3 / fp32 activations), K a multiple of 16 up to 32768
//    (gemv_stream_kernel): no matrix cores.  W wavefronts share a weight row and read it in
//    contiguous 1 KiB pieces; the activation rows stay in registers; weights are converted two
//    bytes per instruction and accumulated with v_dot2 (bf16 / fp16) or v_fma (fp32) in fp32 per
//    128-wide scale block; a row pair's sums are reduced together across the wavefront.
//  * M == 1, other K or misaligned rows (gemv_kernel): the same shape with bounds tests, fp32 math.
//  * 5 <= M <= 16 bf16 activations (any M >= 5 for fp16, in passes of 16), K a multiple of 128
//    (skinny_rows_kernel): a workgroup owns up to
//    32 weight rows for the whole K; weights converted to bf16 in registers, v_mfma_f32_16x16x32_bf16 on
//    the activations as they are; one kernel, no workspace.
//  * 17 <= M <= 32, bf16 activations (skinny_mfma_kernel): split-K over 8 workgroup columns with
//    v_mfma_scale_f32_16x16x128_f8f6f4.  The weights feed the matrix cores as the e4m3 bytes
//    they are; the activations are split once per workgroup into two e4m3 planes in LDS.  The
//    per-split partial sums go to a workspace and a second kernel adds them in split order.
//  * anything else (odd K, misaligned rows): rowwise_kernel, one wavefront per
//    output row, scalar byte loads.

#include <type_traits>

#include "common.h"

namespace cm {
namespace {

struct VecmatParams {
  const void* x;
  const float* scale_x;
  const unsigned char* w;
  const float* scale_w;
  void* out;
  float* partial;          // [splits][M][N] fp32 (skinny kernel)
  int m, n, k;
  int x_dtype, out_dtype;
  int srow_shift;          // scale row index = n >> srow_shift
  int srow_stride;         // floats between scale rows
  int scol_stride;         // floats between 128-wide K blocks (0 or 1)
  int rows_per_wg;
  int k_splits;
};

__device__ __forceinline__ float wscale(const VecmatParams& p, int n, int kb) {
  return p.scale_w[(size_t)(n >> p.srow_shift) * p.srow_stride + (size_t)kb * p.scol_stride];
}

// 16 consecutive activation values starting at element k -> fp32
__device__ __forceinline__ void load_x16(const VecmatParams& p, size_t off, float (&o)[16]) {
  if (p.x_dtype == CPPMEGA_MI355_F32) {
    const float4* s = reinterpret_cast<const float4*>((const float*)p.x + off);
#pragma unroll
    for (int i = 0; i < 4; ++i) { const float4 t = s[i]; o[4*i] = t.x; o[4*i+1] = t.y; o[4*i+2] = t.z; o[4*i+3] = t.w; }
  } else if (p.x_dtype == CPPMEGA_MI355_E4M3) {
    const uint4 t = *reinterpret_cast<const uint4*>((const unsigned char*)p.x + off);
    const unsigned wds[4] = {t.x, t.y, t.z, t.w};
    const float sx = p.scale_x ? p.scale_x[0] : 1.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f32x2 lo = e4m3x2_lo(wds[i]), hi = e4m3x2_hi(wds[i]);
      o[4*i] = lo[0] * sx; o[4*i+1] = lo[1] * sx; o[4*i+2] = hi[0] * sx; o[4*i+3] = hi[1] * sx;
    }
  } else {
    const uint4* s = reinterpret_cast<const uint4*>((const unsigned short*)p.x + off);
    const bool bf = p.x_dtype == CPPMEGA_MI355_BF16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint4 t = s[h];
      const unsigned wds[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const unsigned short a = (unsigned short)(wds[i] & 0xffffu), b = (unsigned short)(wds[i] >> 16);
        o[8*h + 2*i] = bf ? bf16_bits_to_f32(a) : f16_bits_to_f32(a);
        o[8*h + 2*i + 1] = bf ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
      }
    }
  }
}

// 16 weight bytes that are read exactly once: loaded with the non-temporal hint, so they do not
// displace the activations and scales (which every workgroup re-reads) from the caches
__device__ __forceinline__ uint4 load_w16(const unsigned char* src) {
  typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src));
  return make_uint4(t[0], t[1], t[2], t[3]);
}

__device__ __forceinline__ float dot16(const uint4 wv, const float (&x)[16]) {
  const unsigned wds[4] = {wv.x, wv.y, wv.z, wv.w};
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f32x2 lo = e4m3x2_lo(wds[i]), hi = e4m3x2_hi(wds[i]);
    s = fmaf(lo[0], x[4*i], s);
    s = fmaf(lo[1], x[4*i+1], s);
    s = fmaf(hi[0], x[4*i+2], s);
    s = fmaf(hi[1], x[4*i+3], s);
  }
  return s;
}

constexpr int kGemvWaves = 4;
constexpr int kChunk = 1024;        // bytes of one row a wavefront reads per load instruction
constexpr int kRowUnroll = 4;
constexpr int kMaxRowsPerWg = 32;

// M == 1.  CH = 1 KiB chunks per wavefront per pass over K.
template <int CH>
__global__ __launch_bounds__(kGemvWaves * 64) void gemv_kernel(const VecmatParams p) {
  __shared__ float red[kGemvWaves][kMaxRowsPerWg];
  const int lane = lane_id();
  const int wave = (int)(threadIdx.x >> 6);
  const int K = p.k;
  const int row0 = (int)blockIdx.x * p.rows_per_wg;
  const int nrows = min(p.rows_per_wg, p.n - row0);

  float acc[kMaxRowsPerWg / kRowUnroll][kRowUnroll];
#pragma unroll
  for (int i = 0; i < kMaxRowsPerWg / kRowUnroll; ++i)
#pragma unroll
    for (int u = 0; u < kRowUnroll; ++u) acc[i][u] = 0.0f;

  for (int kpass = 0; kpass < K; kpass += kGemvWaves * CH * kChunk) {
    float xr[CH][16];
    int koff[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      koff[c] = kpass + (c * kGemvWaves + wave) * kChunk + lane * 16;
      if (koff[c] < K) {
        load_x16(p, (size_t)koff[c], xr[c]);
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) xr[c][i] = 0.0f;
      }
    }
#pragma unroll
    for (int rg = 0; rg < kMaxRowsPerWg / kRowUnroll; ++rg) {
      if (rg * kRowUnroll < nrows) {
        uint4 wv[kRowUnroll][CH];
        float sc[kRowUnroll][CH];
#pragma unroll
        for (int u = 0; u < kRowUnroll; ++u) {
          const int n = row0 + min(rg * kRowUnroll + u, nrows - 1);
          const unsigned char* wrow = p.w + (size_t)n * K;
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (koff[c] < K) {
              wv[u][c] = load_w16(wrow + koff[c]);
              sc[u][c] = wscale(p, n, koff[c] >> 7);
            } else {
              wv[u][c] = make_uint4(0, 0, 0, 0);
              sc[u][c] = 0.0f;
            }
          }
        }
#pragma unroll
        for (int u = 0; u < kRowUnroll; ++u)
#pragma unroll
          for (int c = 0; c < CH; ++c) acc[rg][u] = fmaf(sc[u][c], dot16(wv[u][c], xr[c]), acc[rg][u]);
      }
    }
  }

#pragma unroll
  for (int rg = 0; rg < kMaxRowsPerWg / kRowUnroll; ++rg)
#pragma unroll
    for (int u = 0; u < kRowUnroll; ++u) {
      const float s = wave_sum(acc[rg][u]);
      if (lane == 0) red[wave][rg * kRowUnroll + u] = s;
    }
  __syncthreads();
  if ((int)threadIdx.x < nrows) {
    const int r = (int)threadIdx.x;
    const float s = ((red[0][r] + red[1][r]) + red[2][r]) + red[3][r];
    store_as(p.out, (size_t)(row0 + r), p.out_dtype, s);
  }
}

// M <= 4 bf16 activations, K a multiple of 16 up to 32768: the streaming kernel.
//   * W wavefronts share a row; a wavefront covers CH chunks of 1 KiB of it (16 bytes per lane).
//     Lanes whose chunk lies past K take zero activations and re-read the row's first bytes, so
//     the row loop itself carries no bounds test;
//   * activations stay in registers as packed bf16 pairs;
//   * weights go e4m3 -> bf16 pairs two bytes per instruction (exact) and meet
//     the activations in v_dot2_f32_bf16, fp32 accumulation;
//   * rows are processed in groups of U with the loads of the next group issued
//     before the arithmetic of the current one (two register buffers);
//   * per row group: one joint DPP reduction of its U x M sums, then a fixed-order LDS combine.

constexpr int kStreamU = 2;              // rows per group (measured: 2 streams at least as fast as 4, in fewer registers)
constexpr int kStreamMaxRows = 32;       // rows per workgroup, a multiple of kStreamU chosen by the host
constexpr int kStreamMaxK = 8 * 4 * kChunk;

template <int CH>
struct StreamBuf {
  uint4 w[kStreamU][CH];
  float sc[kStreamU][CH];
};

// XT, the activation type: bf16; e4m3 bytes with one fp32 scale (exactly representable as bf16
// pairs; the scale multiplies the finished sums); fp16 (weights become fp16 pairs, exact, and meet
// them in v_dot2_f32_f16); fp32 (weights become fp32, v_fma_f32).
constexpr int kXBf16 = 0, kXF8 = 1, kXF16 = 2, kXF32 = 3;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <int M, int CH, int W, int XT = kXBf16>
__global__ __launch_bounds__(W * 64) void gemv_stream_kernel(const VecmatParams p) {
  constexpr int U = kStreamU;
  __shared__ float red[W][4][kStreamMaxRows][M];
  const int lane = lane_id();
  const int wave = (int)(threadIdx.x >> 6);
  const int K = p.k;
  const int R = p.rows_per_wg;
  const int G = R / U;
  const int row0 = (int)blockIdx.x * R;
  const int last_row = p.n - 1;

  int koff[CH];
  constexpr bool XF8 = XT == kXF8;
  constexpr int XW = XT == kXF32 ? 16 : 8;             // registers per activation row and chunk
  unsigned xp[M][CH][XW];
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int k = (c * W + wave) * kChunk + lane * 16;
    const bool live = k < K;                       // (K is a multiple of 16: a lane's 16 channels are all in or all out)
    koff[c] = live ? k : 0;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      uint4 a = make_uint4(0, 0, 0, 0), b = a;
      if constexpr (XF8) {
        if (live) a = *reinterpret_cast<const uint4*>((const unsigned char*)p.x + (size_t)m * K + k);
        const unsigned wds[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          xp[m][c][2 * i] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wds[i], 1.0f, false));
          xp[m][c][2 * i + 1] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wds[i], 1.0f, true));
        }
      } else if constexpr (XT == kXF32) {
        uint4 q[4] = {a, a, a, a};
        if (live) {
          const uint4* src = reinterpret_cast<const uint4*>((const float*)p.x + (size_t)m * K + k);
#pragma unroll
          for (int i = 0; i < 4; ++i) q[i] = src[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) { xp[m][c][4 * i] = q[i].x; xp[m][c][4 * i + 1] = q[i].y; xp[m][c][4 * i + 2] = q[i].z; xp[m][c][4 * i + 3] = q[i].w; }
      } else {
        if (live) {
          const uint4* src = reinterpret_cast<const uint4*>((const unsigned short*)p.x + (size_t)m * K + k);
          a = src[0]; b = src[1];
        }
        const unsigned wds[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) xp[m][c][i] = wds[i];
      }
    }
  }

  auto load = [&](StreamBuf<CH>& buf, int g) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = min(row0 + g * U + u, last_row);
      const unsigned char* wrow = p.w + (size_t)n * K;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        buf.w[u][c] = load_w16(wrow + koff[c]);
        buf.sc[u][c] = wscale(p, n, koff[c] >> 7);
      }
    }
  };
  // Per row group: U x M per-lane sums.  They are reduced together: select steps at lane distances
  // 1 and 2 halve the number of live values (a lane keeps the value its low lane bits name and adds
  // its partner's copy of it), then row shifts by (2,) 4 and 8 finish the 16-lane rows.  The last
  // MP lanes of each 16-lane row then hold that row's sums; the four rows are added in the final
  // combine.
  constexpr int MP = M == 3 ? 4 : M;               // values per weight row in the reduction (a power of two)
  const bool bit0 = (lane & 1) != 0, bit1 = (lane & 2) != 0;
  const bool writer = (lane & 15) >= 16 - MP && (lane & (MP - 1)) < M;
  const int lrow = lane >> 4, wm = lane & (MP - 1);
  auto dpp_add = [](float v, float moved_src, auto ctrl) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, moved_src), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  auto compute = [&](const StreamBuf<CH>& buf, int g) {
    float acc[U][MP];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int m = 0; m < MP; ++m) acc[u][m] = 0.0f;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const unsigned wds[4] = {buf.w[u][c].x, buf.w[u][c].y, buf.w[u][c].z, buf.w[u][c].w};
        if constexpr (XT == kXF32) {
          f32x2 wf[8];
#pragma unroll
          for (int i = 0; i < 4; ++i) { wf[2 * i] = e4m3x2_lo(wds[i]); wf[2 * i + 1] = e4m3x2_hi(wds[i]); }
#pragma unroll
          for (int m = 0; m < M; ++m) {
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              part = fmaf(wf[i][0], __uint_as_float(xp[m][c][2 * i]), part);
              part = fmaf(wf[i][1], __uint_as_float(xp[m][c][2 * i + 1]), part);
            }
            acc[u][m] = fmaf(buf.sc[u][c], part, acc[u][m]);
          }
        } else if constexpr (XT == kXF16) {
          f16x2 wp[8];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            wp[2 * i] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wds[i], 1.0f, false);
            wp[2 * i + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wds[i], 1.0f, true);
          }
#pragma unroll
          for (int m = 0; m < M; ++m) {
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) part = __builtin_amdgcn_fdot2(wp[i], __builtin_bit_cast(f16x2, xp[m][c][i]), part, false);
            acc[u][m] = fmaf(buf.sc[u][c], part, acc[u][m]);
          }
        } else {
          bf16x2 wp[8];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            wp[2 * i] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wds[i], 1.0f, false);
            wp[2 * i + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wds[i], 1.0f, true);
          }
#pragma unroll
          for (int m = 0; m < M; ++m) {
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) part = __builtin_amdgcn_fdot2_f32_bf16(wp[i], __builtin_bit_cast(bf16x2, xp[m][c][i]), part, false);
            acc[u][m] = fmaf(buf.sc[u][c], part, acc[u][m]);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float v;
      if constexpr (MP == 4) {
        const float k0 = bit0 ? acc[u][1] : acc[u][0], s0 = bit0 ? acc[u][0] : acc[u][1];
        const float k1 = bit0 ? acc[u][3] : acc[u][2], s1 = bit0 ? acc[u][2] : acc[u][3];
        const float b0 = dpp_add(k0, s0, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
        const float b1 = dpp_add(k1, s1, std::integral_constant<int, 0xB1>{});
        const float k = bit1 ? b1 : b0, sd = bit1 ? b0 : b1;
        v = dpp_add(k, sd, std::integral_constant<int, 0x4E>{});                 // quad_perm [2,3,0,1]
      } else if constexpr (MP == 2) {
        const float k = bit0 ? acc[u][1] : acc[u][0], sd = bit0 ? acc[u][0] : acc[u][1];
        v = dpp_add(k, sd, std::integral_constant<int, 0xB1>{});
        v = dpp_add(v, v, std::integral_constant<int, 0x112>{});                 // row_shr:2
      } else {
        v = dpp_add(acc[u][0], acc[u][0], std::integral_constant<int, 0x111>{}); // row_shr:1
        v = dpp_add(v, v, std::integral_constant<int, 0x112>{});
      }
      v = dpp_add(v, v, std::integral_constant<int, 0x114>{});                   // row_shr:4
      v = dpp_add(v, v, std::integral_constant<int, 0x118>{});                   // row_shr:8
      if (writer) red[wave][lrow][g * U + u][wm] = v;
    }
  };

  StreamBuf<CH> a, b;
  load(a, 0);
  // (the loads inside the loop are unconditional, so every wait in it counts loads exactly: a load
  // under a branch would make the compiler wait for everything in flight after the join)
  int g = 0;
  for (; g + 2 < G; g += 2) {                      // (uniform trip count)
    load(b, g + 1);
    compute(a, g);
    load(a, g + 2);
    compute(b, g + 1);
  }
  if (g + 1 < G) {
    load(b, g + 1);
    compute(a, g);
    compute(b, g + 1);
  } else {
    compute(a, g);
  }
  __syncthreads();
  for (int t = (int)threadIdx.x; t < R * M; t += W * 64) {
    const int r = t / M, m = t % M;
    if (row0 + r <= last_row) {
      float s = 0.0f;
#pragma unroll
      for (int w = 0; w < W; ++w) s += (red[w][0][r][m] + red[w][1][r][m]) + (red[w][2][r][m] + red[w][3][r][m]);
      if constexpr (XF8) s *= p.scale_x[0];
      store_as(p.out, (size_t)m * p.n + row0 + r, p.out_dtype, s);
    }
  }
}

// 5 <= M <= 32 with bf16 activations, K a multiple of 1024: the split-K matrix-core kernel.
//
// The weights never leave e4m3: they are the B operand of v_mfma_scale_f32_16x16x128_f8f6f4
// as they come from memory (32 contiguous bytes per lane, a whole 128-byte line per weight row
// and 128-channel block).  The activations are the A operand.  A workgroup first writes its K
// slice of them to LDS as two e4m3 planes hi + lo with x = hi 2^(e-127) + lo 2^(e-131), e one
// exponent per activation row and 128-channel block, which the instruction applies as the
// operand scales: hi carries the upper four significant bits of a bf16 value and lo the lower
// four, so the pair is exact for every element within 2^-14 of the largest of its 128 and off
// by less than 2^-22 of that largest one otherwise.  One block is two MFMAs (hi, lo) into a
// zeroed tile whose lanes all belong to one weight row, so the block's fp32 weight scale (any
// value, not only powers of two) is applied exactly as acc += scale * tile.
constexpr int kSkinnySplits = 8;         // K is cut into eighths, one per workgroup column
constexpr int kSkinnyWaves = 14;         // 448 row tiles x 8 splits = 256 workgroups x 14 wavefronts at N = 7168
constexpr int kSkinnyDepth = 4;          // 128-channel weight blocks in flight per wavefront
constexpr int kSkinnyMaxKw = 2048;       // channels per split the LDS activation slice can hold
constexpr int kXPitch = kSkinnyMaxKw + 16;            // bytes per row of an e4m3 plane: 16 rows fall on distinct banks
constexpr int kXBlocks = kSkinnyMaxKw / 128;

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef short i16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr int skinny_lds_bytes(int mt) { return 2 * 16 * mt * kXPitch + 16 * mt * kXBlocks * 4; }

// 32 bf16 channels of one lane (four 16-byte pieces) -> 32 e4m3 hi + 32 e4m3 lo bytes in channel
// order.  The exponent is shared by the four lanes of a quad (one activation row's 128 channels).
__device__ __forceinline__ int split_bf16_quad(const uint4 (&x)[4], i32x8& hi, i32x8& lo) {
  u16x2 top = {0, 0};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const unsigned w[4] = {x[j].x, x[j].y, x[j].z, x[j].w};
#pragma unroll
    for (int d = 0; d < 4; ++d) top = __builtin_elementwise_max(top, __builtin_bit_cast(u16x2, w[d] & 0x7fff7fffu));
  }
  int amax_bits = max((int)top[0], (int)top[1]);             // bf16 bits of the largest magnitude
  amax_bits = max(amax_bits, __builtin_amdgcn_update_dpp(0, amax_bits, 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
  amax_bits = max(amax_bits, __builtin_amdgcn_update_dpp(0, amax_bits, 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
  const int e = max((amax_bits >> 7) - 7, 5);                 // |x| / 2^(e-127) < 256
  const float unit = __uint_as_float((unsigned)e << 23);
  const float unit_lo = __uint_as_float((unsigned)(e - 4) << 23);   // the remainder is below 2^-4 of the element
  const i16x2 zero = {0, 0};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const unsigned w[4] = {x[j].x, x[j].y, x[j].z, x[j].w};
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      const unsigned w0 = w[2 * d], w1 = w[2 * d + 1];
      i16x2 h = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(zero, __builtin_bit_cast(bf16x2, w0), unit, false);
      h = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(h, __builtin_bit_cast(bf16x2, w1), unit, true);
      const unsigned hw = __builtin_bit_cast(unsigned, h);
      const f32x2 d0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(hw, unit, false);
      const f32x2 d1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(hw, unit, true);
      i16x2 l = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(zero, __uint_as_float(w0 << 16) - d0[0],
                                                         __uint_as_float(w0 & 0xffff0000u) - d0[1], unit_lo, false);
      l = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(l, __uint_as_float(w1 << 16) - d1[0],
                                                   __uint_as_float(w1 & 0xffff0000u) - d1[1], unit_lo, true);
      hi[2 * j + d] = (int)hw;
      lo[2 * j + d] = __builtin_bit_cast(int, l);
    }
  }
  return e;
}

// MT: groups of 16 activation rows
template <int MT>
__global__ __launch_bounds__(kSkinnyWaves * 64) void skinny_mfma_kernel(const VecmatParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* xh = smem;                                            // [16 MT][kXPitch] e4m3 hi
  unsigned char* xl = smem + 16 * MT * kXPitch;                        // [16 MT][kXPitch] e4m3 lo
  int* xe = reinterpret_cast<int*>(smem + 2 * 16 * MT * kXPitch);      // [16 MT][kXBlocks] exponents of the two planes
  const int lane = lane_id();
  const int wave = (int)(threadIdx.x >> 6);
  const int K = p.k;
  const int kw = K / kSkinnySplits;                      // channels of this split (multiple of 128)
  const int split = (int)blockIdx.y;
  const int k0 = split * kw;
  const int blocks = kw / 128;
  // lane (r16, g): B operand = weight row r16 of the tile, channels 32 g .. 32 g + 31 of a block;
  // A operand = activation row r16 (+ 16 mt), the same channels.  The result tile has weight row
  // r16 in every register of the lane: register i is activation row 4 g + i.
  const int r16 = lane & 15, g = lane >> 4;
  const int perm_addr = 4 * (8 * (r16 & 7) + g + (r16 >= 8 ? 4 : 0));   // source lane of this lane's weight bytes
  const unsigned char* ah = xh + r16 * kXPitch + 16 * g;
  const unsigned char* al = xl + r16 * kXPitch + 16 * g;
  const int* ae = xe + r16 * kXBlocks;
  const int tiles = (p.n + 15) / 16;
  // this wavefront's tiles: first, first + kSkinnyWaves, ...; their blocks form one continuous
  // stream so the weight prefetch never drains between tiles
  const int first = (int)blockIdx.x * p.rows_per_wg + wave;
  const int tile_end = min(tiles, ((int)blockIdx.x + 1) * p.rows_per_wg);
  const int my_tiles = first < tile_end ? (tile_end - first + kSkinnyWaves - 1) / kSkinnyWaves : 0;
  const int total = my_tiles * blocks;
  // prefetch cursor: next weight bytes / scale of this lane, advanced block by block
  int pf_tile = first, pf_b = 0;
  const unsigned char* pf_w = nullptr;
  const unsigned char* pf_w2 = nullptr;
  const float* pf_s = nullptr;
  auto pf_seek = [&]() {                                 // (per tile) row of this lane in tile pf_tile
    const int n = min(pf_tile * 16 + r16, p.n - 1);
    // (weights are fetched by lane 8 r + q = bytes 16 q of the block's 128-byte line of row r
    // (first load) and row 8 + r (second load): eight neighbouring lanes read a whole line, which
    // the memory pipeline requests in one piece; two DPP moves and a lane permutation per
    // register then hand the bytes to the matrix core's row-major lanes)
    const int nl = min(pf_tile * 16 + (lane >> 3), p.n - 1);
    const int nl2 = min(pf_tile * 16 + 8 + (lane >> 3), p.n - 1);
    pf_w = p.w + (size_t)nl * K + k0 + 16 * (lane & 7);
    pf_w2 = p.w + (size_t)nl2 * K + k0 + 16 * (lane & 7);
    pf_s = p.scale_w + (size_t)(n >> p.srow_shift) * p.srow_stride + (size_t)(k0 >> 7) * p.scol_stride;
  };
  auto pf_next = [&](uint4& w0, uint4& w1, float& sc) {
    w0 = load_w16(pf_w + 128 * pf_b);
    w1 = load_w16(pf_w2 + 128 * pf_b);
    sc = pf_s[(size_t)pf_b * p.scol_stride];
    if (++pf_b == blocks) {                              // (uniform)
      pf_b = 0;
      pf_tile += kSkinnyWaves;
      if (pf_tile < tile_end) pf_seek();
    }
  };
  uint4 wq0[kSkinnyDepth], wq1[kSkinnyDepth];
  float sq[kSkinnyDepth];
  if (total > 0) {
    pf_seek();
#pragma unroll
    for (int d = 0; d < kSkinnyDepth; ++d) {
      if (d < total) pf_next(wq0[d], wq1[d], sq[d]);
      else { wq0[d] = make_uint4(0, 0, 0, 0); wq1[d] = wq0[d]; sq[d] = 0.0f; }
    }
  }
  // (the first weight blocks are already on their way: the conversion below runs in their shadow)
  // activation slice -> LDS: a quad of lanes per (row, block), 32 channels per lane (rows >= M are zero)
  for (int t = (int)threadIdx.x; t < 16 * MT * blocks * 4; t += kSkinnyWaves * 64) {
    const int q = t & 3, item = t >> 2;
    const int m = item / blocks, b = item % blocks;
    uint4 x[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) x[j] = make_uint4(0, 0, 0, 0);
    if (m < p.m) {
      const uint4* src = reinterpret_cast<const uint4*>((const unsigned short*)p.x + (size_t)m * K + k0 + 128 * b + 32 * q);
#pragma unroll
      for (int j = 0; j < 4; ++j) x[j] = src[j];
    }
    i32x8 hi, lo;
    const int e = split_bf16_quad(x, hi, lo);
    uint4* dh = reinterpret_cast<uint4*>(xh + m * kXPitch + 128 * b + 32 * q);
    uint4* dl = reinterpret_cast<uint4*>(xl + m * kXPitch + 128 * b + 32 * q);
    dh[0] = make_uint4((unsigned)hi[0], (unsigned)hi[1], (unsigned)hi[2], (unsigned)hi[3]);
    dh[1] = make_uint4((unsigned)hi[4], (unsigned)hi[5], (unsigned)hi[6], (unsigned)hi[7]);
    dl[0] = make_uint4((unsigned)lo[0], (unsigned)lo[1], (unsigned)lo[2], (unsigned)lo[3]);
    dl[1] = make_uint4((unsigned)lo[4], (unsigned)lo[5], (unsigned)lo[6], (unsigned)lo[7]);
    if (q == 0) xe[m * kXBlocks + b] = e | ((e - 4) << 8);          // byte 0: hi plane, byte 1: lo plane
  }
  __syncthreads();

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  int b = 0, tile = first;                               // position of flat block f0 + d, tracked incrementally
  for (int f0 = 0; f0 < total; f0 += kSkinnyDepth) {
#pragma unroll
    for (int d = 0; d < kSkinnyDepth; ++d) {
      const int f = f0 + d;
      const uint4 w0 = wq0[d], w1 = wq1[d];
      const float sc = sq[d];
      if (f + kSkinnyDepth < total) pf_next(wq0[d], wq1[d], sq[d]);
      if (f < total) {                                   // (uniform)
        // x0: pieces 0..3 of all 16 rows (the second load's, moved up four lanes, fill lanes 4..7 of
        // every eight); x1: pieces 4..7 (the first load's, moved down four lanes, fill lanes 0..3)
        const int a_[4] = {(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w}, b_[4] = {(int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
        i32x8 bw;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int x0 = __builtin_amdgcn_update_dpp(a_[d], b_[d], 0x114, 0xf, 0xa, false);   // row_shr:4 into banks 1, 3
          const int x1 = __builtin_amdgcn_update_dpp(b_[d], a_[d], 0x104, 0xf, 0x5, false);   // row_shl:4 into banks 0, 2
          bw[d] = __builtin_amdgcn_ds_bpermute(perm_addr, x0);
          bw[4 + d] = __builtin_amdgcn_ds_bpermute(perm_addr, x1);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const uint4 h0 = *reinterpret_cast<const uint4*>(ah + mt * 16 * kXPitch + 128 * b);
          const uint4 h1 = *reinterpret_cast<const uint4*>(ah + mt * 16 * kXPitch + 128 * b + 64);
          const uint4 l0 = *reinterpret_cast<const uint4*>(al + mt * 16 * kXPitch + 128 * b);
          const uint4 l1 = *reinterpret_cast<const uint4*>(al + mt * 16 * kXPitch + 128 * b + 64);
          const int e = ae[mt * 16 * kXBlocks + b];
          const i32x8 ahi = {(int)h0.x, (int)h0.y, (int)h0.z, (int)h0.w, (int)h1.x, (int)h1.y, (int)h1.z, (int)h1.w};
          const i32x8 alo = {(int)l0.x, (int)l0.y, (int)l0.z, (int)l0.w, (int)l1.x, (int)l1.y, (int)l1.z, (int)l1.w};
          f32x4 t = {0.f, 0.f, 0.f, 0.f};
          t = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ahi, bw, t, 0, 0, 0, e, 0, 0x7f7f7f7f);
          t = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(alo, bw, t, 0, 0, 1, e, 0, 0x7f7f7f7f);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[mt][i] = fmaf(sc, t[i], acc[mt][i]);
        }
        if (++b == blocks) {                             // (uniform) tile finished: partial[split][m][row]
          const int row = tile * 16 + r16;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int m = 16 * mt + 4 * g + i;
              if (m < p.m && row < p.n) p.partial[((size_t)split * p.m + m) * p.n + row] = acc[mt][i];
            }
            acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
          b = 0;
          tile += kSkinnyWaves;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// 5 <= M <= 32 without a K split: a workgroup owns up to 32 weight rows for the whole K.
//
// Each of its 8 wavefronts takes a contiguous eighth of the 128-channel blocks, so a weight row
// is streamed as 8 sequential runs.  Per block a wavefront fetches the 32 x 128 weight bytes and
// the 16 MT x 128 bfloat16 activations with loads in which neighbouring lanes ask for
// neighbouring 16-byte pieces (8 lanes = one 128-byte weight line, 16 lanes = 256 bytes of an
// activation row: loads whose lanes all point into different lines move a quarter of the bytes
// per clock), a few blocks ahead, in registers; the block then passes through a private LDS
// tile, written in load order and read in matrix-operand order (16-byte slots XOR-swizzled by
// the row so both directions are free of bank conflicts).  The weight bytes become bfloat16 in
// registers (v_cvt_scalef32_pk_bf16_fp8, exact) and four v_mfma_f32_16x16x32_bf16 per (row tile,
// activation tile) multiply them with the activations as they are: no activation planes, no
// operand exponents, products exact.  A block's tile starts from zero and is added as
// acc += scale * tile, so any fp32 block scale is applied exactly; the scales of the workgroup's
// rows are staged in LDS once.  The activations (M x K bf16, 512 KB at M = 16) are re-read by
// every workgroup out of the L2.  The 8 partial tiles meet in LDS in wavefront order
// (deterministic); there is no workspace and no second kernel.
// ---------------------------------------------------------------------------
constexpr int kRowsMax = 32;              // weight rows per workgroup (two MFMA row tiles)
__host__ __device__ constexpr int rows_waves(int) { return 8; }

typedef _Float16 f16x8v __attribute__((ext_vector_type(8)));

// F16: float16 activations (weights become float16 pairs, exact; v_mfma_f32_16x16x32_f16)
template <int MT, bool F16 = false>
__global__ __launch_bounds__(rows_waves(MT) * 64) void skinny_rows_kernel(const VecmatParams p) {
  constexpr int kRowsWaves = rows_waves(MT);
  constexpr int DEPTH = MT == 1 ? 3 : 2;               // blocks in flight per wavefront (registers)
  constexpr int kWTile = 32 * 128;                     // bytes: 32 rows x 8 slots of 16
  constexpr int kXTile = 16 * 256;                     // bytes: 16 rows x 16 slots of 16
  constexpr int kWaveBytes = kWTile + MT * kXTile;            // tiles of one wavefront
  extern __shared__ __align__(16) unsigned char lds_b[];
  const int KB = p.k / 128;
  unsigned char* stage = lds_b + (size_t)(threadIdx.x >> 6) * kWaveBytes;            // this wavefront's tiles
  float* sc = reinterpret_cast<float*>(lds_b + (size_t)kRowsWaves * kWaveBytes);      // [KB][32] block scales of the rows
  float* red = reinterpret_cast<float*>(lds_b);                                       // [waves][32][16 MT], reuses the tiles
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kg = lane >> 4;
  const int n0 = (int)blockIdx.x * p.rows_per_wg;
  const int rows_here = min(p.rows_per_wg, p.n - n0);

  const int per_wave = (KB + kRowsWaves - 1) / kRowsWaves;
  const int kb_begin = wave * per_wave, kb_end = min(KB, kb_begin + per_wave);
  // Workgroups start at different places of their runs, so that at any time they ask for different
  // activation lines and different memory channels (every workgroup's rows begin at the same
  // channel alignment).  The order in which a row's blocks are added depends on the workgroup only.
  const int nblk = max(kb_end - kb_begin, 0);
  const int rot = nblk > 0 ? (int)((blockIdx.x * 5u) % (unsigned)nblk) : 0;
  auto block_at = [&](int i) { const int j = i + rot; return kb_begin + (j >= nblk ? j - nblk : j); };
  // the block scales of this wavefront's run (32 rows x nblk): written and read by this wavefront only
  for (int e = lane; e < 32 * nblk; e += 64) {
    const int r = e & 31, kb = kb_begin + (e >> 5);
    sc[kb * 32 + r] = r < rows_here ? wscale(p, n0 + r, kb) : 0.0f;
  }

  // load order: position = lane + 64 j holds (row, slot); the piece fetched into a slot is slot ^ swizzle(row)
  // (32-bit lane offsets from a uniform base: the address of a load is scalar base + lane offset, no vector arithmetic)
  const unsigned char* wbase = p.w + (size_t)n0 * p.k;
  unsigned woff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int pos = lane + 64 * j, row = pos >> 3, slot = pos & 7;
    woff[j] = (unsigned)min(row, rows_here - 1) * (unsigned)p.k + 16u * (unsigned)(slot ^ ((row >> 1) & 7));
  }
  const unsigned char* xbase = (const unsigned char*)p.x;
  unsigned xoff[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int pos = lane + 64 * j, row = pos >> 4, slot = pos & 15;
      xoff[mt][j] = (unsigned)min(16 * mt + row, p.m - 1) * (unsigned)p.k * 2u + 16u * (unsigned)(slot ^ row);
    }
  // operand order: lane (r16, kg)
  int a_off[2][2], b_off[MT][4];                       // byte offsets inside a tile set
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = 16 * rt + r16;
      a_off[rt][h] = row * 128 + 16 * ((2 * kg + h) ^ ((row >> 1) & 7));
    }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) b_off[mt][s4] = kWTile + mt * kXTile + r16 * 256 + 16 * ((4 * kg + s4) ^ r16);

  typedef __attribute__((ext_vector_type(4))) unsigned u4;
  u4 wq[DEPTH][4];
  u4 xq[DEPTH][MT][4];
  auto fetch = [&](int slot, int kb) {
    const unsigned char* wb = wbase + (size_t)kb * 128;
    const unsigned char* xb_ = xbase + (size_t)kb * 256;
#pragma unroll
    for (int j = 0; j < 4; ++j) wq[slot][j] = __builtin_nontemporal_load(reinterpret_cast<const u4*>(wb + woff[j]));
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) xq[slot][mt][j] = *reinterpret_cast<const u4*>(xb_ + xoff[mt][j]);
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (d < nblk) fetch(d, block_at(d));

  f32x4 acc[2][MT];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // registers -> the wavefront's LDS tiles, in load order
  auto to_lds = [&](int slot) {
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<u4*>(stage + (lane + 64 * j) * 16) = wq[slot][j];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) *reinterpret_cast<u4*>(stage + kWTile + mt * kXTile + (lane + 64 * j) * 16) = xq[slot][mt][j];
  };
  for (int i0 = 0; i0 < nblk; i0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int i = i0 + d;
      if (i < nblk) {                                  // (uniform)
        const int kb = block_at(i);
        to_lds(d);
        if (i + DEPTH < nblk) fetch(d, block_at(i + DEPTH));            // refill the slot just emptied
        const unsigned char* src = stage;
        uint4 xb[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int s4 = 0; s4 < 4; ++s4) xb[mt][s4] = *reinterpret_cast<const uint4*>(src + b_off[mt][s4]);
        f32x4 tile[2][MT];
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
          const uint4 w0 = *reinterpret_cast<const uint4*>(src + a_off[rt][0]);
          const uint4 w1 = *reinterpret_cast<const uint4*>(src + a_off[rt][1]);
          const unsigned wd[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) tile[rt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s4 = 0; s4 < 4; ++s4) {             // MFMA step s4: channels 32 kg + 8 s4 .. + 7 of the block
            uint4 a;
            if (F16) {
              a.x = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wd[2 * s4], 1.0f, false));
              a.y = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wd[2 * s4], 1.0f, true));
              a.z = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wd[2 * s4 + 1], 1.0f, false));
              a.w = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wd[2 * s4 + 1], 1.0f, true));
            } else {
              a.x = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wd[2 * s4], 1.0f, false));
              a.y = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wd[2 * s4], 1.0f, true));
              a.z = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wd[2 * s4 + 1], 1.0f, false));
              a.w = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wd[2 * s4 + 1], 1.0f, true));
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              if (F16)
                tile[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8v, a), __builtin_bit_cast(f16x8v, xb[mt][s4]),
                                                                      tile[rt][mt], 0, 0, 0);
              else
                tile[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, xb[mt][s4]),
                                                                       tile[rt][mt], 0, 0, 0);
            }
          }
        }
        // tile element i: weight row 16 rt + 4 kg + i, activation row 16 mt + r16
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
          const f32x4 s4v = *reinterpret_cast<const f32x4*>(sc + kb * 32 + 16 * rt + 4 * kg);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[rt][mt][e] = fmaf(s4v[e], tile[rt][mt][e], acc[rt][mt][e]);
        }
      }
    }
  }

  // partial tiles of the 8 wavefronts -> LDS (over the staging tiles) -> sums in wavefront order
  __syncthreads();
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(wave * 32 + 16 * rt + 4 * kg + i) * (16 * MT) + 16 * mt + r16] = acc[rt][mt][i];
  __syncthreads();
  for (int e = tid; e < 16 * MT * 32; e += kRowsWaves * 64) {
    const int m = e >> 5, r = e & 31;                  // consecutive threads: consecutive output columns
    if (m < p.m && r < rows_here) {
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < kRowsWaves; ++w) sum += red[(w * 32 + r) * (16 * MT) + m];
      store_as(p.out, (size_t)m * p.n + n0 + r, p.out_dtype, sum);
    }
  }
}

// out[m][n] = sum over the K splits of partial[split][m][n], in split order
__global__ __launch_bounds__(256) void skinny_reduce_kernel(const VecmatParams p) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t total = (size_t)p.m * p.n;
  if (i >= total) return;
  float s = 0.0f;
#pragma unroll
  for (int z = 0; z < kSkinnySplits; ++z) s += p.partial[(size_t)z * total + i];
  store_as(p.out, i, p.out_dtype, s);
}

// Any shape: one wavefront per output row, all M activations in turn.
__global__ __launch_bounds__(256) void rowwise_kernel(const VecmatParams p) {
  const int lane = lane_id();
  const int n = (int)(blockIdx.x * 4 + (threadIdx.x >> 6));
  if (n >= p.n) return;
  const unsigned char* wrow = p.w + (size_t)n * p.k;
  const float sx = (p.x_dtype == CPPMEGA_MI355_E4M3 && p.scale_x) ? p.scale_x[0] : 1.0f;
  for (int m = 0; m < p.m; ++m) {
    float acc = 0.0f;
    for (int k = lane; k < p.k; k += 64) {
      const float wv = e4m3_to_f32(wrow[k]) * wscale(p, n, k >> 7);
      acc = fmaf(wv, load_as(p.x, (size_t)m * p.k + k, p.x_dtype) * sx, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) store_as(p.out, (size_t)m * p.n + n, p.out_dtype, acc);
  }
}

}  // namespace

static int fill_scale_layout(const cppmega_mi355_vecmat_args_t& a, VecmatParams& p) {
  const int kb = (a.k + 127) / 128;
  switch (a.scale_w_kind) {
    case CPPMEGA_MI355_WSCALE_SCALAR: p.srow_shift = 0; p.srow_stride = 0; p.scol_stride = 0; return 0;
    case CPPMEGA_MI355_WSCALE_PER_ROW: p.srow_shift = 0; p.srow_stride = 1; p.scol_stride = 0; return 0;
    case CPPMEGA_MI355_WSCALE_ROW_BLOCK: p.srow_shift = 0; p.srow_stride = kb; p.scol_stride = 1; return 0;
    case CPPMEGA_MI355_WSCALE_GRID_128: p.srow_shift = 7; p.srow_stride = kb; p.scol_stride = 1; return 0;
    default: return fail(CPPMEGA_MI355_ERR_SHAPE, "vecmat: unknown scale_w_kind %d", a.scale_w_kind);
  }
}

static int validate(const cppmega_mi355_vecmat_args_t& a) {
  if (!a.x || !a.w || !a.scale_w || !a.out) return fail(CPPMEGA_MI355_ERR_NULL, "vecmat: x/w/scale_w/out is NULL");
  if (a.m < 1 || a.n < 1 || a.k < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "vecmat: M=%d N=%d K=%d", a.m, a.n, a.k);
  if (a.x_dtype != CPPMEGA_MI355_F32 && a.x_dtype != CPPMEGA_MI355_F16 && a.x_dtype != CPPMEGA_MI355_BF16 &&
      a.x_dtype != CPPMEGA_MI355_E4M3)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "vecmat: x dtype %d", a.x_dtype);
  if (a.x_dtype == CPPMEGA_MI355_E4M3 && !a.scale_x)
    return fail(CPPMEGA_MI355_ERR_NULL, "vecmat: e4m3 activation needs scale_x");
  if (a.out_dtype != CPPMEGA_MI355_F32 && a.out_dtype != CPPMEGA_MI355_F16 && a.out_dtype != CPPMEGA_MI355_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "vecmat: out dtype %d", a.out_dtype);
  return 0;
}

static bool vecmat_aligned(const cppmega_mi355_vecmat_args_t& a) {
  const size_t xelt = (size_t)dtype_size(a.x_dtype);
  return (a.k % 16 == 0) && ((uintptr_t)a.w % 16 == 0) && ((uintptr_t)a.x % 16 == 0) && (((size_t)a.k * xelt) % 16 == 0);
}
// activation rows one launch of the streaming kernel takes (0: not a type it reads)
static int stream_row_cap(int x_dtype) {
  if (x_dtype == CPPMEGA_MI355_BF16 || x_dtype == CPPMEGA_MI355_F16) return 4;
  if (x_dtype == CPPMEGA_MI355_E4M3 || x_dtype == CPPMEGA_MI355_F32) return 1;
  return 0;
}
static bool stream_k(const cppmega_mi355_vecmat_args_t& a) {
  return stream_row_cap(a.x_dtype) > 0 && (a.k % 16 == 0) && a.k <= kStreamMaxK;
}
static bool stream_shape(const cppmega_mi355_vecmat_args_t& a) { return stream_k(a) && a.m <= stream_row_cap(a.x_dtype); }
// the split-K MFMA kernel: bf16 activations, M >= 5 (in passes of 32 rows), K in eighths of whole scale blocks that fit the LDS slice
constexpr int kSkinnyMaxRows = 32;
constexpr int kRowsMaxM = 16;             // activation rows the kernel without a K split takes (17..32 measured no faster than the split-K kernel)
static bool skinny_shape(const cppmega_mi355_vecmat_args_t& a) {
  return a.x_dtype == CPPMEGA_MI355_BF16 && a.m >= 5 &&
         (a.k % (kSkinnySplits * 128) == 0) && a.k / kSkinnySplits <= kSkinnyMaxKw;
}
static bool skinny_ok(const cppmega_mi355_vecmat_args_t& a) { return vecmat_aligned(a) && skinny_shape(a); }
// the kernel without a K split: bf16 activations, M >= 5 (in passes of 32 rows), whole 128-channel blocks,
// scales of 32 rows and partial tiles within the LDS
static size_t rows_lds_bytes(int k, int mt) { return (size_t)rows_waves(mt) * (32 * 128 + mt * 16 * 256) + (size_t)(k / 128) * 32 * sizeof(float); }
static bool rows_shape(const cppmega_mi355_vecmat_args_t& a) {
  const bool bf16 = a.x_dtype == CPPMEGA_MI355_BF16;
  // float16 rows have no split-K kernel behind them (they would run in passes of 4 on the streaming kernel): any M >= 5
  if (a.x_dtype == CPPMEGA_MI355_F16) return a.m >= 5 && a.k % 128 == 0 && rows_lds_bytes(a.k, 1) <= 160 * 1024;
  return bf16 && a.m >= 5 && a.m <= kRowsMaxM && a.k % 128 == 0 && rows_lds_bytes(a.k, a.m <= 16 ? 1 : 2) <= 160 * 1024;
}

int fp8_vecmat_workspace_bytes(const cppmega_mi355_vecmat_args_t& a, size_t* bytes) {
  if (!bytes) return fail(CPPMEGA_MI355_ERR_NULL, "vecmat: bytes is NULL");
  // pointers may be absent in a sizing call: decided from the shape alone (a misaligned call then
  // simply does not use the workspace)
  *bytes = (skinny_shape(a) && !rows_shape(a)) ? (size_t)kSkinnySplits * (a.m < kSkinnyMaxRows ? a.m : kSkinnyMaxRows) * a.n * sizeof(float) : 0;
  return 0;
}

static int device_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    else cus = 256;
  }
  return cus;
}

// Rows per workgroup of the streaming kernel.  Few rows: about one workgroup per compute unit.
// Many rows: of 16, 28 and 14 the one whose grid leaves the smallest idle share in its last
// round over the compute units (ties: the earlier candidate).
static int stream_rows(int n, int m) {
  const int cus = device_cus();
  if (n < 16 * cus) {
    const int r = (n / cus) & ~(kStreamU - 1);
    return r < kStreamU ? kStreamU : r;
  }
  if (m == 1) return 16;
  const int cand[3] = {16, 28, 14};
  int best = 16;
  double best_eff = -1.0;
  for (int r : cand) {
    const long long wgs = (n + r - 1) / r;
    const long long rounds = (wgs + cus - 1) / cus;
    const double eff = (double)wgs / (double)(rounds * cus);
    if (eff > best_eff + 1e-9) { best_eff = eff; best = r; }
  }
  return best;
}

// Wavefronts per row (W) and 1 KiB chunks per wavefront (CH) of the streaming kernel: the pair
// with the fewest idle chunk slots, W * CH >= ceil(K / 1024); among equals the one named first
// in the preference order below.
static void stream_split(int k, int* w_out, int* ch_out) {
  const int chunks = (k + kChunk - 1) / kChunk;
  if (chunks < 4) { *w_out = chunks; *ch_out = 1; return; }
  const int pref[5] = {4, 8, 7, 6, 5};
  int best_w = 8, best_ch = 4, best_waste = 1 << 30;
  for (int w : pref) {
    const int ch = (chunks + w - 1) / w;
    if (ch > 4) continue;
    const int waste = w * ch - chunks;
    if (waste < best_waste) { best_waste = waste; best_w = w; best_ch = ch; }
  }
  *w_out = best_w; *ch_out = best_ch;
}

template <int M, int W, int XF8>
static void stream_launch_ch(int ch, dim3 grid, hipStream_t stream, const VecmatParams& p) {
  const dim3 block(W * 64);
  if (ch == 1) hipLaunchKernelGGL((gemv_stream_kernel<M, 1, W, XF8>), grid, block, 0, stream, p);
  else if (ch == 2) hipLaunchKernelGGL((gemv_stream_kernel<M, 2, W, XF8>), grid, block, 0, stream, p);
  else if (ch == 3) hipLaunchKernelGGL((gemv_stream_kernel<M, 3, W, XF8>), grid, block, 0, stream, p);
  else hipLaunchKernelGGL((gemv_stream_kernel<M, 4, W, XF8>), grid, block, 0, stream, p);
}
template <int M, int XF8 = kXBf16>
static void stream_launch(int w, int ch, dim3 grid, hipStream_t stream, const VecmatParams& p) {
  switch (w) {
    case 1: hipLaunchKernelGGL((gemv_stream_kernel<M, 1, 1, XF8>), grid, dim3(64), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((gemv_stream_kernel<M, 1, 2, XF8>), grid, dim3(128), 0, stream, p); break;
    case 3: hipLaunchKernelGGL((gemv_stream_kernel<M, 1, 3, XF8>), grid, dim3(192), 0, stream, p); break;
    case 4: stream_launch_ch<M, 4, XF8>(ch, grid, stream, p); break;
    case 5: stream_launch_ch<M, 5, XF8>(ch, grid, stream, p); break;
    case 6: stream_launch_ch<M, 6, XF8>(ch, grid, stream, p); break;
    case 7: stream_launch_ch<M, 7, XF8>(ch, grid, stream, p); break;
    default: stream_launch_ch<M, 8, XF8>(ch, grid, stream, p); break;
  }
}

int fp8_vecmat_launch(const cppmega_mi355_vecmat_args_t& a, hipStream_t stream) {
  int rc = validate(a);
  if (rc) return rc;
  VecmatParams p;
  p.x = a.x; p.scale_x = a.scale_x; p.w = a.w; p.scale_w = a.scale_w; p.out = a.out;
  p.partial = nullptr;
  p.m = a.m; p.n = a.n; p.k = a.k; p.x_dtype = a.x_dtype; p.out_dtype = a.out_dtype;
  p.rows_per_wg = 0; p.k_splits = 1;
  rc = fill_scale_layout(a, p);
  if (rc) return rc;

  const bool aligned = vecmat_aligned(a);
  // one launch of the streaming kernel over `rows` activation rows starting at row m0
  auto stream_pass = [&](VecmatParams q, int m0, int rows) -> int {
    q.x = (const char*)a.x + (size_t)m0 * a.k * dtype_size(a.x_dtype);
    q.out = (char*)a.out + (size_t)m0 * a.n * dtype_size(a.out_dtype);
    q.m = rows;
    int w = 4, ch = 4;
    stream_split(a.k, &w, &ch);
    if (w < 4 && ch != 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "vecmat: no streaming split for k=%d", a.k);
    q.rows_per_wg = stream_rows(a.n, rows);
    const dim3 grid((unsigned)((a.n + q.rows_per_wg - 1) / q.rows_per_wg));
    if (a.x_dtype == CPPMEGA_MI355_E4M3) stream_launch<1, kXF8>(w, ch, grid, stream, q);
    else if (a.x_dtype == CPPMEGA_MI355_F32) stream_launch<1, kXF32>(w, ch, grid, stream, q);
    else if (a.x_dtype == CPPMEGA_MI355_F16) {
      if (rows == 1) stream_launch<1, kXF16>(w, ch, grid, stream, q);
      else if (rows == 2) stream_launch<2, kXF16>(w, ch, grid, stream, q);
      else if (rows == 3) stream_launch<3, kXF16>(w, ch, grid, stream, q);
      else stream_launch<4, kXF16>(w, ch, grid, stream, q);
    }
    else if (rows == 1) stream_launch<1>(w, ch, grid, stream, q);
    else if (rows == 2) stream_launch<2>(w, ch, grid, stream, q);
    else if (rows == 3) stream_launch<3>(w, ch, grid, stream, q);
    else stream_launch<4>(w, ch, grid, stream, q);
    CM_HIP_CHECK(hipGetLastError());
    return 0;
  };
  if (aligned && stream_shape(a)) {
    rc = stream_pass(p, 0, a.m);
    if (rc) return rc;
  } else if (aligned && rows_shape(a)) {
    // about one workgroup per CU, whole MFMA row tiles where that is possible
    int rows = (a.n + device_cus() - 1) / device_cus();
    rows = rows < 16 ? 16 : (rows > kRowsMax ? kRowsMax : rows);
    p.rows_per_wg = rows;
    const dim3 grid((unsigned)((a.n + rows - 1) / rows));
    const size_t smem = rows_lds_bytes(a.k, 1);
    const bool f16 = a.x_dtype == CPPMEGA_MI355_F16;
    const void* fn = f16 ? (const void*)skinny_rows_kernel<1, true> : (const void*)skinny_rows_kernel<1, false>;
    if (smem > 64 * 1024) CM_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    for (int m0 = 0; m0 < a.m; m0 += 16) {             // (more than 16 rows: float16 only, in passes)
      VecmatParams q = p;
      q.m = a.m - m0 < 16 ? a.m - m0 : 16;
      q.x = (const char*)a.x + (size_t)m0 * a.k * dtype_size(a.x_dtype);
      q.out = (char*)a.out + (size_t)m0 * a.n * dtype_size(a.out_dtype);
      void* kargs[] = {(void*)&q};
      CM_HIP_CHECK(hipLaunchKernel(fn, grid, dim3(rows_waves(1) * 64), kargs, smem, stream));
    }
  } else if (skinny_ok(a)) {
    // more than 32 activation rows: passes of 32 over the same workspace (stream order keeps them apart)
    const int cap = a.m < kSkinnyMaxRows ? a.m : kSkinnyMaxRows;
    const size_t need = (size_t)kSkinnySplits * cap * a.n * sizeof(float);
    if (!a.workspace || a.workspace_bytes < need)
      return fail(CPPMEGA_MI355_ERR_WORKSPACE, "vecmat: workspace of %zu bytes needed, %zu given", need, (size_t)a.workspace_bytes);
    p.partial = (float*)a.workspace;
    // row tiles per workgroup: about one workgroup per CU and split, a multiple of the wavefront count
    const int tiles = (a.n + 15) / 16;
    int per_wave = (tiles * kSkinnySplits + 256 * kSkinnyWaves - 1) / (256 * kSkinnyWaves);
    if (per_wave < 1) per_wave = 1;
    p.rows_per_wg = per_wave * kSkinnyWaves;
    const dim3 grid((unsigned)((tiles + p.rows_per_wg - 1) / p.rows_per_wg), kSkinnySplits), block(kSkinnyWaves * 64);
    for (int m0 = 0; m0 < a.m; m0 += kSkinnyMaxRows) {
      VecmatParams q = p;
      q.m = a.m - m0 < kSkinnyMaxRows ? a.m - m0 : kSkinnyMaxRows;
      q.x = (const char*)a.x + (size_t)m0 * a.k * dtype_size(a.x_dtype);
      q.out = (char*)a.out + (size_t)m0 * a.n * dtype_size(a.out_dtype);
      if (q.m <= 16) {
        const int smem = skinny_lds_bytes(1);
        CM_HIP_CHECK(hipFuncSetAttribute((const void*)skinny_mfma_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
        hipLaunchKernelGGL(skinny_mfma_kernel<1>, grid, block, smem, stream, q);
      } else {
        const int smem = skinny_lds_bytes(2);
        CM_HIP_CHECK(hipFuncSetAttribute((const void*)skinny_mfma_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
        hipLaunchKernelGGL(skinny_mfma_kernel<2>, grid, block, smem, stream, q);
      }
      CM_HIP_CHECK(hipGetLastError());
      hipLaunchKernelGGL(skinny_reduce_kernel, dim3((unsigned)(((size_t)q.m * a.n + 255) / 256)), dim3(256), 0, stream, q);
    }
  } else if (aligned && stream_k(a)) {
    // more rows than one launch takes: passes over the weights (which the last-level cache may keep)
    const int cap = stream_row_cap(a.x_dtype);
    for (int m0 = 0; m0 < a.m; m0 += cap) {
      rc = stream_pass(p, m0, a.m - m0 < cap ? a.m - m0 : cap);
      if (rc) return rc;
    }
  } else if (a.m == 1 && aligned) {
    // rows per workgroup: keep at least ~3 workgroups per CU in the grid
    int rows = 16;
    while (rows > 4 && (a.n + rows - 1) / rows < 768) rows >>= 1;
    p.rows_per_wg = rows;
    const dim3 grid((unsigned)((a.n + rows - 1) / rows)), block(kGemvWaves * 64);
    const int chunks = (a.k + kChunk - 1) / kChunk;
    if (chunks <= kGemvWaves) hipLaunchKernelGGL(gemv_kernel<1>, grid, block, 0, stream, p);
    else if (chunks <= 2 * kGemvWaves) hipLaunchKernelGGL(gemv_kernel<2>, grid, block, 0, stream, p);
    else hipLaunchKernelGGL(gemv_kernel<4>, grid, block, 0, stream, p);
  } else {
    const dim3 grid((unsigned)((a.n + 3) / 4)), block(256);
    hipLaunchKernelGGL(rowwise_kernel, grid, block, 0, stream, p);
  }
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
