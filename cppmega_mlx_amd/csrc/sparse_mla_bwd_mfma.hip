// Sparse MLA backward on the matrix cores: bfloat16 or float16 operands, or e4m3 q / kv with
// per-token scales (gfx950).
//
// Same gradients as sparse_mla_bwd.hip (the reference's sparse_mla_bwd_direct,
// cppmega_mlx/nn/_tilelang/sparse_mla_path_c.py:2644-2816), organised so that the heads of a KV
// group share every gathered row and every atomic add:
//
//   workgroup = (batch, query, KV group, chunk of 16 or 32 heads), 4 wavefronts;
//   q and d_out of the chunk stay in LDS for the whole kernel; the selected rows pass through
//   LDS in tiles of 64 (16-head chunks) or 32 (32-head chunks) keys, fetched one tile ahead
//   into registers.
//
//   pass 1  S^T = K . Q^T and dP^T = K[:, :d_v] . dO^T per (16 keys, 16 heads) on
//           v_mfma_f32_16x16x32_bf16 (both products read the same K fragments); running
//           maximum, sum and sum of p * dP per head: the softmax statistics and
//           delta = sum_k p_k dP_k without storing a score;
//   pass 2  the same two products again, then P = exp2(s - m) / l and
//           dS = sm_scale * P * (dP - delta) as bfloat16 [head][key] tiles in LDS, and per
//           wavefront (which owns every fourth block of 16 channels):
//             dQ^T[ch, head] += K^T[ch, key] . dS^T[key, head]          (accumulated in registers)
//             dKV[key, ch]    = dS^T[key, head] . Q[head, ch] + P^T[key, head] . dO[head, ch]
//           and one float32 atomic add per (key, channel) of the tile into dkv.  Operands that
//           are needed transposed (K^T, dS^T, Q and dO by head) come from the row-major LDS
//           tiles through the transposing read ds_read_b64_tr_b16.
//
// P and dS enter the second pair of products as two bfloat16 planes each, hi = bf16(x) and
// lo = bf16(x - hi), so a term carries a relative error of about 2^-17 instead of 2^-9 and the
// gradients agree with fp32 arithmetic on the same bfloat16 inputs to ~1e-5 of their scale; the
// extra matrix instructions are hidden behind the atomic adds.  The atomic adds per selected row
// drop from one per head to one per chunk of heads.
//
// Per-token FP8 operands (the reference's fp8_sparse_mla_bwd_kernel,
// cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:1966-2214): the e4m3 bytes of q and of the
// gathered rows become bfloat16 (exactly) on their way into LDS, so the products run on the raw
// code values; the scales q_scale[b,s,h] and kv_scale[b,t,g] multiply the scores and dP afterwards,
// and are folded into dS before the second pair of products (dS * kv_scale for dQ, dS * q_scale
// for dKV), so the gradients are with respect to the dequantised values, as in the reference.

#include "common.h"
#include "mfma_util.h"

namespace cm {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxBlk = 9;            // 16-channel blocks per wavefront: d_qk <= 4 * 9 * 16 = 576
constexpr int kPad = 8;               // bfloat16 elements of padding per LDS row

struct BwdMfmaParams {
  const void* q;                // [B, S, H, D] bf16, or e4m3 bytes
  const void* kv;               // [B, Skv, G, D] bf16, or e4m3 bytes
  const float* q_scale;         // [B, S, H] (e4m3 only)
  const float* kv_scale;        // [B, Skv, G] (e4m3 only)
  const unsigned short* d_out;  // [B, S, H, d_v] bf16
  const void* indices;          // [B, S, G, topk]
  const float* sm_scale_dev;
  void* dq;                     // [B, S, H, D]
  float* dkv;                   // [B, Skv, G, D]
  int dq_dtype, index_dtype;
  int B, S, H, G, Skv, topk, D, d_v;
  int chunks;                   // head chunks per KV group
  int ntiles;
  float sm_scale;
};

__device__ __forceinline__ bf16x8 lds_b128(const unsigned short* p) { return *reinterpret_cast<const bf16x8*>(p); }

// Transposing read: within a group of 16 lanes, lane i points at 4 consecutive elements
// (row i / 4, columns 4 * (i % 4) ..) of a 4 x 16 block and receives column i of rows 0..3.
__device__ __forceinline__ bf16x4 lds_tr16(const unsigned short* p) {
  typedef __attribute__((ext_vector_type(4))) short s16x4;
  const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
  return __builtin_bit_cast(bf16x4, v);
}
__device__ __forceinline__ bf16x8 join(const bf16x4 a, const bf16x4 b) {
  bf16x8 r;
  r[0] = a[0]; r[1] = a[1]; r[2] = a[2]; r[3] = a[3];
  r[4] = b[0]; r[5] = b[1]; r[6] = b[2]; r[7] = b[3];
  return r;
}
// 8 e4m3 bytes -> 8 float16 / 8 bfloat16, exact
__device__ __forceinline__ uint4 e4m3x8_to_f16(const uint2 v) {
  uint4 r;
  r.x = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v.x, 1.0f, false));
  r.y = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v.x, 1.0f, true));
  r.z = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v.y, 1.0f, false));
  r.w = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v.y, 1.0f, true));
  return r;
}
__device__ __forceinline__ uint4 e4m3x8_to_bf16(const uint2 v) {
  uint4 r;
  r.x = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.x, 1.0f, false));
  r.y = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.x, 1.0f, true));
  r.z = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.y, 1.0f, false));
  r.w = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.y, 1.0f, true));
  return r;
}
typedef _Float16 f16x8b __attribute__((ext_vector_type(8)));
// one matrix instruction on operands held as 8 x 16 bits: bfloat16, or float16 when F16
template <bool F16>
__device__ __forceinline__ f32x4 mm(const bf16x8 a, const bf16x8 b, const f32x4 c) {
  if (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8b, a), __builtin_bit_cast(f16x8b, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ bf16x8 zero8() {
  return __builtin_bit_cast(bf16x8, make_uint4(0u, 0u, 0u, 0u));
}

// EL: 0 bfloat16 operands, 1 per-token e4m3 operands with a bfloat16 cotangent, 2 float16 operands,
//     3 per-token e4m3 operands with a float16 cotangent
template <int HB, int EL>
__global__ __launch_bounds__(kThreads, 1) void sparse_mla_bwd_mfma_kernel(const BwdMfmaParams p) {
  constexpr bool FP8 = EL == 1 || EL == 3, F16 = EL == 2 || EL == 3;
  // float16 planes of P and dS are kept at 16 times their value: a float16 is flushed below 6e-8 and overflows above
  // 65504, so entries down to 4e-9 survive and |dS| may reach 4000
  constexpr float kPlaneScale = F16 ? 16.0f : 1.0f, kPlaneUnscale = F16 ? 1.0f / 16.0f : 1.0f;
  constexpr int HC = 16 * HB;            // heads per workgroup
  constexpr int KT = 64 / HB;            // keys per tile
  constexpr int KSUB = KT / 16;          // 16-key blocks per tile
  constexpr int Kp = KT + kPad;
  constexpr int NP = KT * 72 / kThreads; // 16-byte pieces of a tile per thread at d_qk = 576

  extern __shared__ __align__(16) unsigned char smem[];
  const int D = p.D, dv = p.d_v;
  const int Dp = D + kPad, Dvp = dv + kPad;
  unsigned short* Qs = reinterpret_cast<unsigned short*>(smem);     // [HC][Dp]
  unsigned short* dOs = Qs + HC * Dp;                               // [HC][Dvp]
  unsigned short* Ks = dOs + HC * Dvp;                              // [KT][Dp]
  constexpr int kPlane = HC * Kp;
  unsigned short* Ps = Ks + KT * Dp;                                // [hi, lo][HC][Kp]
  unsigned short* dSs = Ps + 2 * kPlane;                            // [hi, lo][HC][Kp]: dS (* kv_scale of the key)
  unsigned short* dSq = FP8 ? dSs + 2 * kPlane : dSs;               // [hi, lo][HC][Kp]: dS * q_scale of the head
  float* wstat = reinterpret_cast<float*>(dSq + 2 * kPlane);        // [4 waves][16 heads][3]
  float* stat = wstat + 4 * 16 * 3;                                 // [HC][3]: max, 1 / sum, delta
  float* qsc = stat + HC * 3;                                       // [HC] q scales (e4m3 only)
  float* ksc = qsc + HC;                                            // [KT] kv scales of the tile (e4m3 only)
  int* rows = reinterpret_cast<int*>(ksc + KT);                     // [ntiles * KT]

  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kg = lane >> 4;
  const int chunk = (int)(blockIdx.x % p.chunks);
  const int g = (int)((blockIdx.x / p.chunks) % p.G);
  const size_t bs = blockIdx.x / ((size_t)p.chunks * p.G);
  const int b = (int)(bs / p.S);
  const int Hg = p.H / p.G;
  const int h0 = g * Hg + chunk * HC;                 // first head of the chunk
  const int nh = min(HC, Hg - chunk * HC);            // heads of the chunk that exist
  const float sm_scale = p.sm_scale_dev ? *p.sm_scale_dev : p.sm_scale;
  const float scale2 = sm_scale * kLog2e;
  const int dpr = D / 8;                              // 16-byte pieces per key row
  const int dv32 = dv / 32, d32 = D / 32;
  const int nblk = D / 16;                            // 16-channel blocks

  // ---- prologue: the index list, q and d_out of the chunk --------------------------------
  {
    const size_t idx_base = (bs * p.G + g) * (size_t)p.topk;
    for (int k = tid; k < p.ntiles * KT; k += kThreads) {
      long long i = -1;
      if (k < p.topk)
        i = p.index_dtype == CPPMEGA_MI355_I64 ? static_cast<const long long*>(p.indices)[idx_base + k]
                                               : (long long)static_cast<const int*>(p.indices)[idx_base + k];
      rows[k] = (i >= 0 && i < p.Skv) ? (int)i : -1;
    }
    const float inv_dpr = 1.0f / (float)dpr, inv_vpr = 1.0f / (float)(dv / 8);
    for (int piece = tid; piece < HC * dpr; piece += kThreads) {
      const int h = (int)(((float)piece + 0.5f) * inv_dpr), c8 = piece - h * dpr;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (h < nh) {
        const size_t at = (bs * p.H + h0 + h) * (size_t)D + c8 * 8;
        if (FP8) {
          const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const unsigned char*>(p.q) + at);
          v = F16 ? e4m3x8_to_f16(raw) : e4m3x8_to_bf16(raw);
        }
        else v = *reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(p.q) + at);
      }
      *reinterpret_cast<uint4*>(Qs + h * Dp + c8 * 8) = v;
    }
    if (FP8 && tid < HC) qsc[tid] = tid < nh ? p.q_scale[bs * p.H + h0 + tid] : 0.0f;
    for (int piece = tid; piece < HC * (dv / 8); piece += kThreads) {
      const int h = (int)(((float)piece + 0.5f) * inv_vpr), c8 = piece - h * (dv / 8);
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (h < nh) v = *reinterpret_cast<const uint4*>(p.d_out + (bs * p.H + h0 + h) * (size_t)dv + c8 * 8);
      *reinterpret_cast<uint4*>(dOs + h * Dvp + c8 * 8) = v;
    }
  }
  __syncthreads();

  // ---- tile staging: global -> registers one tile ahead -> LDS ----------------------------
  uint4 pre[NP];                                      // (e4m3: the 8 bytes of a piece in .x, .y and the row's scale in .z)
  int pre_off[NP];                                    // LDS element offset of each piece, -1 = none
  {
    const float inv_dpr = 1.0f / (float)dpr;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int piece = tid + i * kThreads;
      const int r = (int)(((float)piece + 0.5f) * inv_dpr), c8 = piece - r * dpr;
      pre_off[i] = piece < KT * dpr ? ((r << 16) | c8) : -1;
    }
  }
  auto issue = [&](int t) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      pre[i] = make_uint4(0u, 0u, 0u, 0u);
      if (pre_off[i] >= 0) {
        const int r = pre_off[i] >> 16, c8 = pre_off[i] & 0xffff;
        const int row = rows[t * KT + r];
        if (row >= 0) {
          const size_t krow = ((size_t)b * p.Skv + (size_t)row) * p.G + g;
          if (FP8) {
            const uint2 v = *reinterpret_cast<const uint2*>(static_cast<const unsigned char*>(p.kv) + krow * (size_t)D + c8 * 8);
            pre[i].x = v.x;
            pre[i].y = v.y;
            if (c8 == 0) pre[i].z = __float_as_uint(p.kv_scale[krow]);
          } else {
            pre[i] = *reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(p.kv) + krow * (size_t)D + c8 * 8);
          }
        }
      }
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < NP; ++i)
      if (pre_off[i] >= 0) {
        const int r = pre_off[i] >> 16, c8 = pre_off[i] & 0xffff;
        if (FP8) {
          *reinterpret_cast<uint4*>(Ks + r * Dp + c8 * 8) = F16 ? e4m3x8_to_f16(make_uint2(pre[i].x, pre[i].y)) : e4m3x8_to_bf16(make_uint2(pre[i].x, pre[i].y));
          if (c8 == 0) ksc[r] = __uint_as_float(pre[i].z);
        } else {
          *reinterpret_cast<uint4*>(Ks + r * Dp + c8 * 8) = pre[i];
        }
      }
  };

  // ---- the two products of a wavefront's (16 keys, 16 heads) block ------------------------
  const int ks = wave % KSUB, hb = wave / KSUB;
  const unsigned short* a_base = Ks + (16 * ks + l16) * Dp + 8 * kg;
  const unsigned short* q_base = Qs + (16 * hb + l16) * Dp + 8 * kg;
  const unsigned short* o_base = dOs + (16 * hb + l16) * Dvp + 8 * kg;
  auto products = [&](f32x4& s, f32x4& dp) {
    s = f32x4{0.f, 0.f, 0.f, 0.f};
    dp = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int kk = 0; kk < dv32; ++kk) {
      const bf16x8 a = lds_b128(a_base + kk * 32);
      s = mm<F16>(a, lds_b128(q_base + kk * 32), s);
      dp = mm<F16>(a, lds_b128(o_base + kk * 32), dp);
    }
    for (int kk = dv32; kk < d32; ++kk)
      s = mm<F16>(lds_b128(a_base + kk * 32), lds_b128(q_base + kk * 32), s);
    if (FP8) {                                        // code-value products -> products of the dequantised values
      const f32x4 kscale = *reinterpret_cast<const f32x4*>(ksc + 16 * ks + 4 * kg);
      const float qscale = qsc[16 * hb + l16];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        s[i] *= qscale * kscale[i];
        dp[i] *= kscale[i];
      }
    }
  };
  // this lane's accumulator element i is (key 16 * ks + 4 * kg + i of the tile, head 16 * hb + l16)

  // ---- pass 1: softmax statistics and delta ------------------------------------------------
  float m_run = -INFINITY, l_run = 0.0f, d_run = 0.0f;
  issue(0);
  for (int t = 0; t < p.ntiles; ++t) {
    commit();
    __syncthreads();
    if (t + 1 < p.ntiles) issue(t + 1);
    f32x4 s, dp;
    products(s, dp);
    float s2[4], tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s2[i] = rows[t * KT + 16 * ks + 4 * kg + i] >= 0 ? s[i] * scale2 : -INFINITY;
      tmax = fmaxf(tmax, s2[i]);
    }
    tmax = fmaxf(tmax, xor16(tmax));
    tmax = fmaxf(tmax, xor32(tmax));
    const float m_new = fmaxf(m_run, tmax);
    if (m_new > -INFINITY) {
      const float f = exp2f(m_run - m_new);           // 0 when nothing was valid before
      l_run *= f;
      d_run *= f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e = exp2f(s2[i] - m_new);
        l_run += e;
        d_run = fmaf(e, dp[i], d_run);
      }
      m_run = m_new;
    }
    __syncthreads();                                  // Ks is free again
  }
  l_run += xor16(l_run); l_run += xor32(l_run);
  d_run += xor16(d_run); d_run += xor32(d_run);
  if (kg == 0) {
    wstat[(wave * 16 + l16) * 3 + 0] = m_run;
    wstat[(wave * 16 + l16) * 3 + 1] = l_run;
    wstat[(wave * 16 + l16) * 3 + 2] = d_run;
  }
  __syncthreads();
  if (tid < HC) {
    const int hb2 = tid >> 4, hl = tid & 15;
    float M = -INFINITY;
    for (int w = hb2 * KSUB; w < (hb2 + 1) * KSUB; ++w) M = fmaxf(M, wstat[(w * 16 + hl) * 3]);
    float L = 0.0f, Dl = 0.0f;
    if (M > -INFINITY)
      for (int w = hb2 * KSUB; w < (hb2 + 1) * KSUB; ++w) {
        const float f = exp2f(wstat[(w * 16 + hl) * 3] - M);
        L = fmaf(wstat[(w * 16 + hl) * 3 + 1], f, L);
        Dl = fmaf(wstat[(w * 16 + hl) * 3 + 2], f, Dl);
      }
    const float linv = L > 0.0f ? 1.0f / L : 0.0f;
    stat[tid * 3 + 0] = M > -INFINITY ? M : 0.0f;
    stat[tid * 3 + 1] = linv;
    stat[tid * 3 + 2] = Dl * linv;
  }
  __syncthreads();
  const float st_m = stat[(16 * hb + l16) * 3], st_linv = stat[(16 * hb + l16) * 3 + 1], st_delta = stat[(16 * hb + l16) * 3 + 2];

  // ---- pass 2 ---------------------------------------------------------------------------------
  f32x4 accq[kMaxBlk][HB];
#pragma unroll
  for (int j = 0; j < kMaxBlk; ++j)
#pragma unroll
    for (int h2 = 0; h2 < HB; ++h2) accq[j][h2] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int tr_row = l16 >> 2, tr_col = (l16 & 3) * 4;   // this lane's place in a transposing read

  issue(0);
  for (int t = 0; t < p.ntiles; ++t) {
    commit();
    __syncthreads();
    if (t + 1 < p.ntiles) issue(t + 1);
    {
      f32x4 s, dp;
      products(s, dp);
      float pv[4], ds[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool ok = rows[t * KT + 16 * ks + 4 * kg + i] >= 0;
        pv[i] = ok ? exp2f(s[i] * scale2 - st_m) * st_linv : 0.0f;
        ds[i] = pv[i] * (dp[i] - st_delta) * sm_scale;
      }
      const int off = (16 * hb + l16) * Kp + 16 * ks + 4 * kg;
      auto planes = [&](unsigned short* base, const float (&v)[4]) {      // hi and lo bfloat16 planes of 4 values
        float hi[4], lo[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          hi[i] = v[i] * kPlaneScale;
          lo[i] = hi[i] - (F16 ? (float)(_Float16)hi[i] : (float)(__bf16)hi[i]);
        }
        if (F16) {
          *reinterpret_cast<uint2*>(base + off) = make_uint2(pack_f16(hi[0], hi[1]), pack_f16(hi[2], hi[3]));
          *reinterpret_cast<uint2*>(base + kPlane + off) = make_uint2(pack_f16(lo[0], lo[1]), pack_f16(lo[2], lo[3]));
        } else {
          *reinterpret_cast<uint2*>(base + off) = make_uint2(pack_bf16(hi[0], hi[1]), pack_bf16(hi[2], hi[3]));
          *reinterpret_cast<uint2*>(base + kPlane + off) = make_uint2(pack_bf16(lo[0], lo[1]), pack_bf16(lo[2], lo[3]));
        }
      };
      planes(Ps, pv);
      if (FP8) {
        const f32x4 kscale = *reinterpret_cast<const f32x4*>(ksc + 16 * ks + 4 * kg);
        const float qscale = qsc[16 * hb + l16];
        float dk[4], dq_[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          dk[i] = ds[i] * kscale[i];
          dq_[i] = ds[i] * qscale;
        }
        planes(dSs, dk);
        planes(dSq, dq_);
      } else {
        planes(dSs, ds);
      }
    }
    __syncthreads();

    // dQ^T += K^T . dS^T
#pragma unroll
    for (int kk = 0; kk < KT / 32; ++kk) {
      bf16x8 bds[HB][2];
#pragma unroll
      for (int h2 = 0; h2 < HB; ++h2)
#pragma unroll
        for (int pl = 0; pl < 2; ++pl) bds[h2][pl] = lds_b128(dSs + pl * kPlane + (16 * h2 + l16) * Kp + 32 * kk + 8 * kg);
#pragma unroll
      for (int j = 0; j < kMaxBlk; ++j) {
        const int cb = wave + 4 * j;
        if (cb < nblk) {
          const unsigned short* src = Ks + (32 * kk + 8 * kg + tr_row) * Dp + cb * 16 + tr_col;
          const bf16x8 a = join(lds_tr16(src), lds_tr16(src + 4 * Dp));
#pragma unroll
          for (int h2 = 0; h2 < HB; ++h2) {
            accq[j][h2] = mm<F16>(a, bds[h2][0], accq[j][h2]);
            accq[j][h2] = mm<F16>(a, bds[h2][1], accq[j][h2]);
          }
        }
      }
    }

    // dKV = dS^T . Q + P^T . dO, added to the selected rows
#pragma unroll
    for (int kb = 0; kb < KSUB; ++kb) {
      bf16x8 a_ds[2], a_p[2];                          // hi and lo planes
#pragma unroll
      for (int pl = 0; pl < 2; ++pl) {
        if (HB == 2) {
          const int o = pl * kPlane + (8 * kg + tr_row) * Kp + kb * 16 + tr_col;
          a_ds[pl] = join(lds_tr16(dSq + o), lds_tr16(dSq + o + 4 * Kp));
          a_p[pl] = join(lds_tr16(Ps + o), lds_tr16(Ps + o + 4 * Kp));
        } else {                                      // contraction slots 0..15: dS of the 16 heads, 16..31: P
          const unsigned short* src = (kg < 2 ? dSq : Ps) + pl * kPlane + (8 * (kg & 1) + tr_row) * Kp + kb * 16 + tr_col;
          a_ds[pl] = join(lds_tr16(src), lds_tr16(src + 4 * Kp));
          a_p[pl] = a_ds[pl];
        }
      }
      int row_i[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) row_i[i] = rows[t * KT + kb * 16 + 4 * kg + i];
#pragma unroll
      for (int j = 0; j < kMaxBlk; ++j) {
        const int cb = wave + 4 * j;
        if (cb < nblk) {
          f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
          const bool has_v = cb * 16 < dv;
          if (HB == 2) {
            const unsigned short* qsrc = Qs + (8 * kg + tr_row) * Dp + cb * 16 + tr_col;
            const bf16x8 bq = join(lds_tr16(qsrc), lds_tr16(qsrc + 4 * Dp));
            acc = mm<F16>(a_ds[0], bq, acc);
            acc = mm<F16>(a_ds[1], bq, acc);
            if (has_v) {
              const unsigned short* osrc = dOs + (8 * kg + tr_row) * Dvp + cb * 16 + tr_col;
              const bf16x8 bo = join(lds_tr16(osrc), lds_tr16(osrc + 4 * Dvp));
              acc = mm<F16>(a_p[0], bo, acc);
              acc = mm<F16>(a_p[1], bo, acc);
            }
          } else {
            // every lane issues the transposing read (it moves data between the lanes of a group of
            // 16, so it must not sit under a divergent branch); lanes without a d_out part zero theirs
            const bool from_q = kg < 2 || !has_v;
            const unsigned short* src = from_q ? Qs + (8 * (kg & 1) + tr_row) * Dp + cb * 16 + tr_col
                                               : dOs + (8 * (kg - 2) + tr_row) * Dvp + cb * 16 + tr_col;
            const int pitch4 = 4 * (from_q ? Dp : Dvp);
            bf16x8 bq = join(lds_tr16(src), lds_tr16(src + pitch4));
            if (kg >= 2 && !has_v) bq = zero8();
            acc = mm<F16>(a_ds[0], bq, acc);
            acc = mm<F16>(a_ds[1], bq, acc);
          }
          // element i: key kb * 16 + 4 * kg + i of the tile, channel cb * 16 + l16
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (row_i[i] >= 0)
              atomicAdd(p.dkv + (((size_t)b * p.Skv + (size_t)row_i[i]) * p.G + g) * (size_t)D + cb * 16 + l16, acc[i] * kPlaneUnscale);
        }
      }
    }
    __syncthreads();                                  // Ks, Ps and dSs are free again
  }

  // ---- dq: element i of accq[j][h2] is (channel cb * 16 + 4 * kg + i, head 16 * h2 + l16) ----
#pragma unroll
  for (int j = 0; j < kMaxBlk; ++j) {
    const int cb = wave + 4 * j;
    if (cb < nblk) {
#pragma unroll
      for (int h2 = 0; h2 < HB; ++h2) {
        const int h = 16 * h2 + l16;
        if (h < nh) {
          const size_t base = (bs * p.H + h0 + h) * (size_t)D + cb * 16 + 4 * kg;
#pragma unroll
          for (int i = 0; i < 4; ++i) store_as(p.dq, base + i, p.dq_dtype, accq[j][h2][i] * kPlaneUnscale);
        }
      }
    }
  }
}

template <int HB>
size_t lds_bytes(int D, int dv, int ntiles, bool fp8) {
  constexpr int HC = 16 * HB, KT = 64 / HB;
  return (size_t)2 * (HC * (D + kPad) + HC * (dv + kPad) + KT * (D + kPad) + (fp8 ? 6 : 4) * HC * (KT + kPad)) +
         (4 * 16 * 3 + HC * 3 + HC + KT) * 4 + (size_t)ntiles * KT * 4;
}

bool fp8_operands(const cppmega_mi355_sparse_mla_bwd_args_t& a) {
  return a.q_dtype == CPPMEGA_MI355_E4M3 && a.kv_dtype == CPPMEGA_MI355_E4M3 && a.q_scale && a.kv_scale;
}

}  // namespace

// Whether the matrix-core kernel takes this problem (else the fp32 kernel runs).
bool sparse_mla_bwd_mfma_supports(const cppmega_mi355_sparse_mla_bwd_args_t& a) {
  const bool bf16 = a.q_dtype == CPPMEGA_MI355_BF16 && a.kv_dtype == CPPMEGA_MI355_BF16;
  const bool f16 = a.q_dtype == CPPMEGA_MI355_F16 && a.kv_dtype == CPPMEGA_MI355_F16;
  if (fp8_operands(a)) {
    if (a.d_out_dtype != CPPMEGA_MI355_BF16 && a.d_out_dtype != CPPMEGA_MI355_F16) return false;
  } else if (f16 ? a.d_out_dtype != CPPMEGA_MI355_F16 : (!bf16 || a.d_out_dtype != CPPMEGA_MI355_BF16)) {
    return false;
  }
  if (a.d_qk % 32 != 0 || a.d_v % 32 != 0 || a.d_qk > kMaxBlk * 64 || a.topk < 1) return false;
  const int hg = a.heads / a.kv_groups;
  const int kt = hg > 16 ? 32 : 64;
  const int ntiles = (a.topk + kt - 1) / kt;
  const size_t lds = hg > 16 ? lds_bytes<2>(a.d_qk, a.d_v, ntiles, fp8_operands(a)) : lds_bytes<1>(a.d_qk, a.d_v, ntiles, fp8_operands(a));
  return lds <= 160 * 1024;
}

int sparse_mla_bwd_mfma_launch(const cppmega_mi355_sparse_mla_bwd_args_t& a, hipStream_t stream) {
  const int hg = a.heads / a.kv_groups;
  const bool wide = hg > 16, fp8 = fp8_operands(a);
  const int hc = wide ? 32 : 16, kt = wide ? 32 : 64;
  BwdMfmaParams p;
  p.q = a.q; p.kv = a.kv; p.q_scale = a.q_scale; p.kv_scale = a.kv_scale;
  p.d_out = static_cast<const unsigned short*>(a.d_out);
  p.indices = a.indices; p.sm_scale_dev = a.sm_scale_dev; p.dq = a.dq; p.dkv = a.dkv;
  p.dq_dtype = a.dq_dtype; p.index_dtype = a.index_dtype;
  p.B = a.batch; p.S = a.seq_q; p.H = a.heads; p.G = a.kv_groups; p.Skv = a.seq_kv; p.topk = a.topk; p.D = a.d_qk; p.d_v = a.d_v;
  p.chunks = (hg + hc - 1) / hc;
  p.ntiles = (a.topk + kt - 1) / kt;
  p.sm_scale = a.sm_scale;
  const size_t grid = (size_t)a.batch * a.seq_q * a.kv_groups * p.chunks;
  if (grid == 0) return 0;
  if (grid > 0x7fffffffull) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla_bwd: too many (batch, query, head chunk) workgroups for one launch");
  const size_t lds = wide ? lds_bytes<2>(a.d_qk, a.d_v, p.ntiles, fp8) : lds_bytes<1>(a.d_qk, a.d_v, p.ntiles, fp8);
  const bool f16 = a.d_out_dtype == CPPMEGA_MI355_F16;     // the cotangent's carrier decides the arithmetic type
  const int el = fp8 ? (f16 ? 3 : 1) : (f16 ? 2 : 0);
  const void* fns[2][4] = {
      {(const void*)sparse_mla_bwd_mfma_kernel<1, 0>, (const void*)sparse_mla_bwd_mfma_kernel<1, 1>, (const void*)sparse_mla_bwd_mfma_kernel<1, 2>,
       (const void*)sparse_mla_bwd_mfma_kernel<1, 3>},
      {(const void*)sparse_mla_bwd_mfma_kernel<2, 0>, (const void*)sparse_mla_bwd_mfma_kernel<2, 1>, (const void*)sparse_mla_bwd_mfma_kernel<2, 2>,
       (const void*)sparse_mla_bwd_mfma_kernel<2, 3>}};
  const void* fn = fns[wide ? 1 : 0][el];
  if (lds > 64 * 1024) CM_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  void* kargs[] = {(void*)&p};
  CM_HIP_CHECK(hipLaunchKernel(fn, dim3((unsigned)grid), dim3(kThreads), kargs, lds, stream));
  return 0;
}

}  // namespace cm
