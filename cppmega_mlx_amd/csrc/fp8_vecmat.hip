// FP8 (e4m3) block-scaled vecmat / skinny GEMM for decode projections (gfx950).
//
//   out[m, n] = sum_k dec(w[n, k]) * w_scale(n, k / 128) * x[m, k]
//
// The weight is read from HBM exactly once; everything else is sized so that
// the weight stream is the only traffic that matters.
//
//  * M == 1  (gemv_kernel): no matrix cores.  A workgroup of 4 wavefronts owns
//    a few output rows; wavefront w owns the 1 KiB K-chunks c with c % 4 == w,
//    so the four wavefronts read 4 KiB of one row contiguously.  The activation
//    slice a wavefront needs is converted to fp32 once and stays in registers
//    for all rows.  Per row a lane issues 16-byte weight loads, converts two
//    bytes per instruction, accumulates in fp32 per 128-wide scale block, and
//    the row sum is a wavefront reduction followed by a 4-way LDS combine.
//  * 2 <= M <= 4, bf16 activations (gemv_stream_kernel): the same streaming shape with the
//    M activation rows held in registers and v_dot2_f32_bf16 accumulation.
//  * 5 <= M <= 32, bf16 activations (skinny_mfma_kernel): v_mfma_f32_16x16x32_bf16 with 16
//    weight rows as the M side and the (padded) activation rows, in one or two groups of 16,
//    as the N side.  A
//    workgroup owns 16 weight rows; its 8 wavefronts own one eighth of K each and add
//    their 16x16 partial tiles through LDS at the end, so nothing but the result is
//    written to memory.  Weight fragments go from HBM straight into registers
//    (16 bytes per lane and load: two MFMA k-steps, with the contraction order inside
//    the 64-channel step permuted the same way for both operands) and are converted
//    e4m3 -> bf16 with the 128-channel block scale applied in the conversion; the
//    activations (L2-resident) are loaded per step.
//  * anything else (odd K, misaligned rows): rowwise_kernel, one wavefront per
//    output row, scalar byte loads.

#include <type_traits>
#include <cstdlib>

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
  unsigned* counters;      // [row tiles]       (skinny kernel)
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

__device__ __forceinline__ float wave_total_dpp(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

constexpr int kStreamU = 2;              // rows per group (measured: 2 streams at least as fast as 4, in fewer registers)
constexpr int kStreamMaxRows = 32;       // rows per workgroup, a multiple of kStreamU chosen by the host
constexpr int kStreamMaxK = 8 * 4 * kChunk;

template <int CH>
struct StreamBuf {
  uint4 w[kStreamU][CH];
  float sc[kStreamU][CH];
};

template <int M, int CH, int W>
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
  bf16x2 xp[M][CH][8];
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int k = (c * W + wave) * kChunk + lane * 16;
    const bool live = k < K;                       // (K is a multiple of 16: a lane's 16 channels are all in or all out)
    koff[c] = live ? k : 0;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      uint4 a = make_uint4(0, 0, 0, 0), b = a;
      if (live) {
        const uint4* src = reinterpret_cast<const uint4*>((const unsigned short*)p.x + (size_t)m * K + k);
        a = src[0]; b = src[1];
      }
      const unsigned wds[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) xp[m][c][i] = __builtin_bit_cast(bf16x2, wds[i]);
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
          for (int i = 0; i < 8; ++i) part = __builtin_amdgcn_fdot2_f32_bf16(wp[i], xp[m][c][i], part, false);
          acc[u][m] = fmaf(buf.sc[u][c], part, acc[u][m]);
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
      store_as(p.out, (size_t)m * p.n + row0 + r, p.out_dtype, s);
    }
  }
}

// 5 <= M <= 32 with bf16 activations, K a multiple of 1024: see the file header.  MT: groups of 16 activation rows.
constexpr int kSkinnySplits = 8;         // K is cut into eighths, one per workgroup column
constexpr int kSkinnyWaves = 7;          // 448 row tiles x 8 splits = 256 workgroups x 7 wavefronts x 2 tiles at N = 7168
constexpr int kSkinnyDepth = 8;          // 64-channel weight steps in flight per wavefront
constexpr int kSkinnyMaxKw = 2048;       // channels per split the LDS activation slice can hold
constexpr int kXPitchBytes = kSkinnyMaxKw * 2 + 16;   // row pitch of the slice: 16 rows fall on distinct banks

template <int MT>
__global__ __launch_bounds__(kSkinnyWaves * 64) void skinny_mfma_kernel(const VecmatParams p) {
  extern __shared__ __align__(16) unsigned char xs[];    // [16 MT][kXPitchBytes]: bf16 activations of this split
  const int lane = lane_id();
  const int wave = (int)(threadIdx.x >> 6);
  const int K = p.k;
  const int kw = K / kSkinnySplits;                      // channels of this split (multiple of 128)
  const int split = (int)blockIdx.y;
  const int k0 = split * kw;
  const int steps = kw / 64;
  // activation slice -> LDS (rows >= M are zero)
  for (int i = (int)threadIdx.x; i < 16 * MT * (kw / 8); i += kSkinnyWaves * 64) {
    const int m = i / (kw / 8), c = i % (kw / 8);
    uint4 v = make_uint4(0, 0, 0, 0);
    if (m < p.m) v = *reinterpret_cast<const uint4*>((const unsigned short*)p.x + (size_t)m * K + k0 + 8 * c);
    *reinterpret_cast<uint4*>(xs + m * kXPitchBytes + 16 * c) = v;
  }
  __syncthreads();

  const int r16 = lane & 15, kq = lane >> 4;
  const unsigned char* xrow = xs + r16 * kXPitchBytes + 32 * kq;        // B fragments: activation r16, channels 16kq.. of a step
  const int tiles = (p.n + 15) / 16;
  // this wavefront's tiles: first, first + 7, ...; their steps form one continuous stream so the
  // weight prefetch never drains between tiles
  const int first = (int)blockIdx.x * p.rows_per_wg + wave;
  const int tile_end = min(tiles, ((int)blockIdx.x + 1) * p.rows_per_wg);
  const int my_tiles = first < tile_end ? (tile_end - first + kSkinnyWaves - 1) / kSkinnyWaves : 0;
  const int total = my_tiles * steps;
  // prefetch cursor: next weight bytes / scale of this lane, advanced step by step
  int pf_tile = first, pf_st = 0;
  const unsigned char* pf_w = nullptr;
  const float* pf_s = nullptr;
  auto pf_seek = [&]() {                                 // (per tile) row of this lane in tile pf_tile
    const int n = min(pf_tile * 16 + r16, p.n - 1);
    pf_w = p.w + (size_t)n * K + k0 + 16 * kq;
    pf_s = p.scale_w + (size_t)(n >> p.srow_shift) * p.srow_stride + (size_t)(k0 >> 7) * p.scol_stride;
  };
  auto pf_next = [&](uint4& wdst, float& sdst, bool with_scale) {
    wdst = *reinterpret_cast<const uint4*>(pf_w + 64 * pf_st);   // (plain load: the other half of the cache line follows next step)
    if (with_scale) sdst = pf_s[(size_t)(pf_st >> 1) * p.scol_stride];
    if (++pf_st == steps) {                              // (uniform)
      pf_st = 0;
      pf_tile += kSkinnyWaves;
      if (pf_tile < tile_end) pf_seek();
    }
  };
  uint4 wq[kSkinnyDepth];
  float sq[kSkinnyDepth / 2];                            // one scale per 128 channels = two steps
  if (total > 0) {
    pf_seek();
#pragma unroll
    for (int d = 0; d < kSkinnyDepth; ++d) {
      if (d < total) pf_next(wq[d], sq[d >> 1], (d & 1) == 0);
      else { wq[d] = make_uint4(0, 0, 0, 0); if ((d & 1) == 0) sq[d >> 1] = 1.0f; }
    }
  }
  float sq_next[kSkinnyDepth / 2];
#pragma unroll
  for (int i = 0; i < kSkinnyDepth / 2; ++i) sq_next[i] = 1.0f;
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  int st = 0, tile = first;                              // position of flat step f0 + d, tracked incrementally
  for (int f0 = 0; f0 < total; f0 += kSkinnyDepth) {     // steps is a multiple of the depth? not required: see the guards
#pragma unroll
    for (int d = 0; d < kSkinnyDepth; ++d) {
      const int f = f0 + d;
      const uint4 wv = wq[d];
      const float sc = sq[d >> 1];
      float sc_next = sc;
      if (f + kSkinnyDepth < total) pf_next(wq[d], sc_next, (d & 1) == 0);
      if ((d & 1) == 0) sq_next[d >> 1] = sc_next;       // takes effect once the odd step of the pair is done
      else sq[d >> 1] = sq_next[d >> 1];
      if (f < total) {                                   // (uniform)
        uint4 x0[MT], x1[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          x0[mt] = *reinterpret_cast<const uint4*>(xrow + mt * 16 * kXPitchBytes + 128 * st);
          x1[mt] = *reinterpret_cast<const uint4*>(xrow + mt * 16 * kXPitchBytes + 128 * st + 16);
        }
        bf16x8 a0, a1;
        const bool pow2 = (__float_as_uint(sc) & 0x007fffffu) == 0u && sc > 0.0f && sc < INFINITY;
        if (__ballot(!pow2) == 0ull) {                   // the conversion applies a power-of-two scale exactly
          const unsigned o0 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.x, sc, false));
          const unsigned o1 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.x, sc, true));
          const unsigned o2 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.y, sc, false));
          const unsigned o3 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.y, sc, true));
          const unsigned o4 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.z, sc, false));
          const unsigned o5 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.z, sc, true));
          const unsigned o6 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.w, sc, false));
          const unsigned o7 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wv.w, sc, true));
          a0 = __builtin_bit_cast(bf16x8, make_uint4(o0, o1, o2, o3));
          a1 = __builtin_bit_cast(bf16x8, make_uint4(o4, o5, o6, o7));
        } else {                                         // general scale: fp32 multiply, round to bf16
          const unsigned wd[4] = {wv.x, wv.y, wv.z, wv.w};
          unsigned o[8];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const f32x2 lo = e4m3x2_lo(wd[i]), hi = e4m3x2_hi(wd[i]);
            typedef __attribute__((ext_vector_type(2))) __bf16 v2;
            v2 r0, r1;
            r0[0] = (__bf16)(lo[0] * sc); r0[1] = (__bf16)(lo[1] * sc);
            r1[0] = (__bf16)(hi[0] * sc); r1[1] = (__bf16)(hi[1] * sc);
            o[2 * i] = __builtin_bit_cast(unsigned, r0);
            o[2 * i + 1] = __builtin_bit_cast(unsigned, r1);
          }
          a0 = __builtin_bit_cast(bf16x8, make_uint4(o[0], o[1], o[2], o[3]));
          a1 = __builtin_bit_cast(bf16x8, make_uint4(o[4], o[5], o[6], o[7]));
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, __builtin_bit_cast(bf16x8, x0[mt]), acc[mt], 0, 0, 0);
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, __builtin_bit_cast(bf16x8, x1[mt]), acc[mt], 0, 0, 0);
        }
        if (++st == steps) {                             // (uniform) tile finished: partial[split][m][row]
          // lane (m = lane%16, g = lane/16) holds weight rows 4g + i of activation 16 mt + m
          const int row0 = tile * 16;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const int m = 16 * mt + r16;
            if (m < p.m) {
              float* dst = p.partial + ((size_t)split * p.m + m) * p.n + row0 + 4 * kq;
              if (row0 + 4 * kq + 3 < p.n && (p.n & 3) == 0) {
                *reinterpret_cast<float4*>(dst) = make_float4(acc[mt][0], acc[mt][1], acc[mt][2], acc[mt][3]);
              } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  if (row0 + 4 * kq + i < p.n) dst[i] = acc[mt][i];
              }
            }
            acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
          st = 0;
          tile += kSkinnyWaves;
        }
      }
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
static bool stream_shape(const cppmega_mi355_vecmat_args_t& a) {
  return a.x_dtype == CPPMEGA_MI355_BF16 && a.m <= 4 && (a.k % 16 == 0) && a.k <= kStreamMaxK;
}
// the split-K MFMA kernel: bf16 activations, 2 <= M <= 32, K in eighths of whole scale blocks that fit the LDS slice
static bool skinny_shape(const cppmega_mi355_vecmat_args_t& a) {
  return a.x_dtype == CPPMEGA_MI355_BF16 && a.m >= 2 && a.m <= 32 && !stream_shape(a) &&
         (a.k % (kSkinnySplits * 128) == 0) && a.k / kSkinnySplits <= kSkinnyMaxKw;
}
static bool skinny_ok(const cppmega_mi355_vecmat_args_t& a) { return vecmat_aligned(a) && skinny_shape(a); }

int fp8_vecmat_workspace_bytes(const cppmega_mi355_vecmat_args_t& a, size_t* bytes) {
  if (!bytes) return fail(CPPMEGA_MI355_ERR_NULL, "vecmat: bytes is NULL");
  // pointers may be absent in a sizing call: decided from the shape alone (a misaligned call then
  // simply does not use the workspace)
  *bytes = skinny_shape(a) ? (size_t)kSkinnySplits * a.m * a.n * sizeof(float) : 0;
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
  if (const char* e = getenv("CPPMEGA_MI355_VECMAT_ROWS")) {
    const int v = atoi(e);
    if (v >= kStreamU && v <= kStreamMaxRows && v % kStreamU == 0) return v;
  }
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
  if (const char* e = getenv("CPPMEGA_MI355_VECMAT_WAVES")) {
    const int w = atoi(e);
    if (w >= 1 && w <= 8 && (chunks + w - 1) / w <= 4) { *w_out = w; *ch_out = (chunks + w - 1) / w; return; }
  }
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

template <int M, int W>
static void stream_launch_ch(int ch, dim3 grid, hipStream_t stream, const VecmatParams& p) {
  const dim3 block(W * 64);
  if (ch == 1) hipLaunchKernelGGL((gemv_stream_kernel<M, 1, W>), grid, block, 0, stream, p);
  else if (ch == 2) hipLaunchKernelGGL((gemv_stream_kernel<M, 2, W>), grid, block, 0, stream, p);
  else if (ch == 3) hipLaunchKernelGGL((gemv_stream_kernel<M, 3, W>), grid, block, 0, stream, p);
  else hipLaunchKernelGGL((gemv_stream_kernel<M, 4, W>), grid, block, 0, stream, p);
}
template <int M>
static void stream_launch(int w, int ch, dim3 grid, hipStream_t stream, const VecmatParams& p) {
  switch (w) {
    case 1: hipLaunchKernelGGL((gemv_stream_kernel<M, 1, 1>), grid, dim3(64), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((gemv_stream_kernel<M, 1, 2>), grid, dim3(128), 0, stream, p); break;
    case 3: hipLaunchKernelGGL((gemv_stream_kernel<M, 1, 3>), grid, dim3(192), 0, stream, p); break;
    case 4: stream_launch_ch<M, 4>(ch, grid, stream, p); break;
    case 5: stream_launch_ch<M, 5>(ch, grid, stream, p); break;
    case 6: stream_launch_ch<M, 6>(ch, grid, stream, p); break;
    case 7: stream_launch_ch<M, 7>(ch, grid, stream, p); break;
    default: stream_launch_ch<M, 8>(ch, grid, stream, p); break;
  }
}

int fp8_vecmat_launch(const cppmega_mi355_vecmat_args_t& a, hipStream_t stream) {
  int rc = validate(a);
  if (rc) return rc;
  VecmatParams p;
  p.x = a.x; p.scale_x = a.scale_x; p.w = a.w; p.scale_w = a.scale_w; p.out = a.out;
  p.partial = nullptr; p.counters = nullptr;
  p.m = a.m; p.n = a.n; p.k = a.k; p.x_dtype = a.x_dtype; p.out_dtype = a.out_dtype;
  p.rows_per_wg = 0; p.k_splits = 1;
  rc = fill_scale_layout(a, p);
  if (rc) return rc;

  const bool aligned = vecmat_aligned(a);
  const bool stream_ok = aligned && stream_shape(a);
  if (stream_ok) {
    int w = 4, ch = 4;
    stream_split(a.k, &w, &ch);
    if (w < 4 && ch != 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "vecmat: no streaming split for k=%d", a.k);
    p.rows_per_wg = stream_rows(a.n, a.m);
    const dim3 grid((unsigned)((a.n + p.rows_per_wg - 1) / p.rows_per_wg));
    if (a.m == 1) stream_launch<1>(w, ch, grid, stream, p);
    else if (a.m == 2) stream_launch<2>(w, ch, grid, stream, p);
    else if (a.m == 3) stream_launch<3>(w, ch, grid, stream, p);
    else stream_launch<4>(w, ch, grid, stream, p);
  } else if (skinny_ok(a)) {
    const size_t need = (size_t)kSkinnySplits * a.m * a.n * sizeof(float);
    if (!a.workspace || a.workspace_bytes < need)
      return fail(CPPMEGA_MI355_ERR_WORKSPACE, "vecmat: workspace of %zu bytes needed, %zu given", need, (size_t)a.workspace_bytes);
    p.partial = (float*)a.workspace;
    // row tiles per workgroup: about one workgroup per CU and split, a multiple of the wavefront count
    const int tiles = (a.n + 15) / 16;
    int per_wave = (tiles * kSkinnySplits + 256 * kSkinnyWaves - 1) / (256 * kSkinnyWaves);
    if (per_wave < 1) per_wave = 1;
    p.rows_per_wg = per_wave * kSkinnyWaves;
    const dim3 grid((unsigned)((tiles + p.rows_per_wg - 1) / p.rows_per_wg), kSkinnySplits), block(kSkinnyWaves * 64);
    if (a.m <= 16) {
      const int smem = 16 * kXPitchBytes;
      CM_HIP_CHECK(hipFuncSetAttribute((const void*)skinny_mfma_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
      hipLaunchKernelGGL(skinny_mfma_kernel<1>, grid, block, smem, stream, p);
    } else {
      const int smem = 32 * kXPitchBytes;
      CM_HIP_CHECK(hipFuncSetAttribute((const void*)skinny_mfma_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
      hipLaunchKernelGGL(skinny_mfma_kernel<2>, grid, block, smem, stream, p);
    }
    CM_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(skinny_reduce_kernel, dim3((unsigned)(((size_t)a.m * a.n + 255) / 256)), dim3(256), 0, stream, p);
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
