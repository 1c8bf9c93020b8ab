// Sparse MLA forward, shape-agnostic kernel: one wavefront per (batch, query, head).
//
// This is the straight fp32 restatement of the reference kernels' arithmetic
// for every storage variant (float carriers, e4m3 with per-token / E8M0 /
// fp32-block scales, optional rope tail, attention sinks).  It takes any
// head count, width and top-k, and is what runs when the head-batched MFMA
// kernel does not cover a shape.
//
//   * the dequantised query row lives in LDS as fp32;
//   * keys are processed 64 at a time: lane j owns key j of the tile and
//     accumulates its dot product per scale block, so the block scale is
//     applied once per block in fp32;
//   * softmax is online across tiles (running max / denominator);
//   * for P.V the lanes switch to owning output channels, so the value reads
//     of one key are coalesced across the wavefront.

#include "sparse_mla_common.h"

namespace cm {
namespace {

template <int DT>
__device__ __forceinline__ float elem(const void* base, size_t i);
template <> __device__ __forceinline__ float elem<CPPMEGA_MI355_F32>(const void* b, size_t i) { return ((const float*)b)[i]; }
template <> __device__ __forceinline__ float elem<CPPMEGA_MI355_F16>(const void* b, size_t i) { return f16_bits_to_f32(((const unsigned short*)b)[i]); }
template <> __device__ __forceinline__ float elem<CPPMEGA_MI355_BF16>(const void* b, size_t i) { return bf16_bits_to_f32(((const unsigned short*)b)[i]); }
template <> __device__ __forceinline__ float elem<CPPMEGA_MI355_E4M3>(const void* b, size_t i) { return e4m3_to_f32(((const unsigned char*)b)[i]); }

// sum_{d in [d0,d1)} qf[d] * kvrow[d]
template <int DT>
__device__ __forceinline__ float dot_span(const void* kv, size_t row_off, const float* qf, int d0, int d1) {
  float s = 0.0f;
  if (DT == CPPMEGA_MI355_E4M3 && ((row_off | (size_t)d0 | (size_t)d1) & 3) == 0) {
    const unsigned* w = reinterpret_cast<const unsigned*>((const unsigned char*)kv + row_off);
    for (int d = d0; d < d1; d += 4) {
      const unsigned pk = w[d >> 2];
      const f32x2 lo = e4m3x2_lo(pk), hi = e4m3x2_hi(pk);
      s = fmaf(qf[d], lo[0], s);
      s = fmaf(qf[d + 1], lo[1], s);
      s = fmaf(qf[d + 2], hi[0], s);
      s = fmaf(qf[d + 3], hi[1], s);
    }
  } else {
    for (int d = d0; d < d1; ++d) s = fmaf(qf[d], elem<DT>(kv, row_off + d), s);
  }
  return s;
}

template <int KVDT, int DVI>
__global__ __launch_bounds__(64) void sparse_mla_scalar_kernel(const MlaParams p) {
  extern __shared__ __align__(16) float smem[];
  float* qf = smem;                       // [d_qk]
  float* pt = smem + p.d_qk;              // [64] tile probabilities
  int* it = reinterpret_cast<int*>(pt + 64);  // [64] tile key rows (-1 = skip)

  const int lane = lane_id();
  const size_t bsh = blockIdx.x;          // ((b*S + s)*H + h)
  const int h = (int)(bsh % p.H);
  const size_t bs = bsh / p.H;
  const int b = (int)(bs / p.S);
  const int g = h / p.heads_per_group;
  const size_t idx_base = (bs * p.G + g) * (size_t)p.topk;

  // ---- dequantised query row -> LDS ---------------------------------------
  {
    const int qblk = p.q_scale_kind == CPPMEGA_MI355_SCALE_NONE || p.q_scale_kind == CPPMEGA_MI355_SCALE_PER_TOKEN
                         ? p.d_qk : p.q_scale_block;
    const int nblk = (p.d_qk + qblk - 1) / qblk;
    for (int d = lane; d < p.d_qk; d += 64) {
      const float sc = row_scale(p.q_scale, p.q_scale_kind, bsh, nblk, d / qblk);
      qf[d] = load_as(p.q, bsh * p.d_qk + d, p.q_dtype) * sc;
    }
  }
  __syncthreads();

  const int kblk = (p.kv_scale_kind == CPPMEGA_MI355_SCALE_NONE || p.kv_scale_kind == CPPMEGA_MI355_SCALE_PER_TOKEN)
                       ? p.d_kv : p.kv_scale_block;
  const int nkblk = (p.d_kv + kblk - 1) / kblk;

  const bool has_sink = mla_has_sinks(p);
  const float sm_scale = mla_sm_scale(p);
  float m = has_sink ? p.sinks[h] : -INFINITY;
  float l = has_sink ? 1.0f : 0.0f;
  float acc[DVI];
#pragma unroll
  for (int i = 0; i < DVI; ++i) acc[i] = 0.0f;

  for (int t0 = 0; t0 < p.topk; t0 += 64) {
    const int jj = t0 + lane;
    long long key = (jj < p.topk) ? load_index(p, idx_base + jj) : -1;
    const bool valid = key >= 0 && key < p.Skv;
    float score = -INFINITY;
    if (valid) {
      const size_t krow = ((size_t)b * p.Skv_pitch + (size_t)key) * p.G + g;
      float dot = 0.0f;
      for (int kb = 0; kb < nkblk; ++kb) {
        const int d0 = kb * kblk, d1 = min(d0 + kblk, p.d_kv);
        const float sc = row_scale(p.kv_scale, p.kv_scale_kind, krow, nkblk, kb);
        dot = fmaf(sc, dot_span<KVDT>(p.kv, krow * p.d_kv, qf, d0, d1), dot);
      }
      if (p.rope_dim > 0) {
        const size_t roff = krow * p.rope_dim;
        for (int d = 0; d < p.rope_dim; ++d)
          dot = fmaf(qf[p.d_kv + d], load_as(p.rope, roff + d, p.rope_dtype), dot);
      }
      score = dot * sm_scale;
    }
    const float tmax = wave_max(score);
    const float m_new = fmaxf(m, tmax);
    if (m_new == -INFINITY) continue;      // uniform: nothing attendable yet
    const float corr = (m == -INFINITY) ? 0.0f : expf(m - m_new);
    const float pj = valid ? expf(score - m_new) : 0.0f;
    l = l * corr + wave_sum(pj);
#pragma unroll
    for (int i = 0; i < DVI; ++i) acc[i] *= corr;
    m = m_new;
    __syncthreads();
    pt[lane] = pj;
    it[lane] = valid ? (int)key : -1;
    __syncthreads();
    for (int jx = 0; jx < 64; ++jx) {
      const int key_j = it[jx];
      if (key_j < 0) continue;             // uniform
      const float pw = pt[jx];
      const size_t krow = ((size_t)b * p.Skv_pitch + (size_t)key_j) * p.G + g;
#pragma unroll
      for (int i = 0; i < DVI; ++i) {
        const int dv = lane + 64 * i;
        if (dv < p.d_v) {
          const float sc = row_scale(p.kv_scale, p.kv_scale_kind, krow, nkblk, dv / kblk);
          acc[i] = fmaf(pw * sc, elem<KVDT>(p.kv, krow * p.d_kv + dv), acc[i]);
        }
      }
    }
  }

  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
  for (int i = 0; i < DVI; ++i) {
    const int dv = lane + 64 * i;
    if (dv < p.d_v) store_as(p.out, bsh * p.d_v + dv, p.out_dtype, acc[i] * inv);
  }
  if (p.lse && lane == 0) p.lse[bsh] = l > 0.0f ? m + logf(l) : 0.0f;
}

// Scores only: scores[b, s, h, j] = sm_scale * q . key(indices[b, s, g, j]) in fp32; a skipped slot
// (index < 0 or >= Skv) holds the most negative finite fp32 value.  One wavefront per (b, s, h).
template <int KVDT>
__global__ __launch_bounds__(64) void sparse_mla_scores_kernel(const MlaParams p) {
  extern __shared__ __align__(16) float smem[];
  float* qf = smem;                       // [d_qk]
  const int lane = lane_id();
  const size_t bsh = blockIdx.x;
  const int h = (int)(bsh % p.H);
  const size_t bs = bsh / p.H;
  const int b = (int)(bs / p.S);
  const int g = h / p.heads_per_group;
  const size_t idx_base = (bs * p.G + g) * (size_t)p.topk;
  {
    const int qblk = p.q_scale_kind == CPPMEGA_MI355_SCALE_NONE || p.q_scale_kind == CPPMEGA_MI355_SCALE_PER_TOKEN
                         ? p.d_qk : p.q_scale_block;
    const int nblk = (p.d_qk + qblk - 1) / qblk;
    for (int d = lane; d < p.d_qk; d += 64) {
      const float sc = row_scale(p.q_scale, p.q_scale_kind, bsh, nblk, d / qblk);
      qf[d] = load_as(p.q, bsh * p.d_qk + d, p.q_dtype) * sc;
    }
  }
  __syncthreads();
  const int kblk = (p.kv_scale_kind == CPPMEGA_MI355_SCALE_NONE || p.kv_scale_kind == CPPMEGA_MI355_SCALE_PER_TOKEN)
                       ? p.d_kv : p.kv_scale_block;
  const int nkblk = (p.d_kv + kblk - 1) / kblk;
  const float sm_scale = mla_sm_scale(p);
  for (int jj = lane; jj < p.topk; jj += 64) {
    const long long key = load_index(p, idx_base + jj);
    float score = -3.4028234663852886e38f;
    if (key >= 0 && key < p.Skv) {
      const size_t krow = ((size_t)b * p.Skv_pitch + (size_t)key) * p.G + g;
      float dot = 0.0f;
      for (int kb = 0; kb < nkblk; ++kb) {
        const int d0 = kb * kblk, d1 = min(d0 + kblk, p.d_kv);
        const float sc = row_scale(p.kv_scale, p.kv_scale_kind, krow, nkblk, kb);
        dot = fmaf(sc, dot_span<KVDT>(p.kv, krow * p.d_kv, qf, d0, d1), dot);
      }
      if (p.rope_dim > 0) {
        const size_t roff = krow * p.rope_dim;
        for (int d = 0; d < p.rope_dim; ++d)
          dot = fmaf(qf[p.d_kv + d], load_as(p.rope, roff + d, p.rope_dtype), dot);
      }
      score = dot * sm_scale;
    }
    p.scores[bsh * p.topk + jj] = score;
  }
}

template <int KVDT>
int launch_dv(const MlaParams& p, hipStream_t stream) {
  const dim3 grid((unsigned)((size_t)p.B * p.S * p.H)), block(64);
  const size_t smem = ((size_t)p.d_qk + 128) * 4;
  const int dvi = (p.d_v + 63) / 64;
#define CM_MLA_SCALAR(DVI)                                                                       \
  do {                                                                                           \
    hipLaunchKernelGGL((sparse_mla_scalar_kernel<KVDT, DVI>), grid, block, smem, stream, p);     \
    return 0;                                                                                    \
  } while (0)
  if (dvi <= 1) CM_MLA_SCALAR(1);
  if (dvi <= 2) CM_MLA_SCALAR(2);
  if (dvi <= 4) CM_MLA_SCALAR(4);
  if (dvi <= 8) CM_MLA_SCALAR(8);
  if (dvi <= 16) CM_MLA_SCALAR(16);
#undef CM_MLA_SCALAR
  return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla: d_v %d exceeds 1024", p.d_v);
}

}  // namespace

int sparse_mla_scalar_launch(const MlaParams& p, hipStream_t stream) {
  if ((size_t)p.B * p.S * p.H == 0) return 0;
  if (p.d_qk > 8192) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla: d_qk %d exceeds 8192", p.d_qk);
  int rc;
  switch (p.kv_dtype) {
    case CPPMEGA_MI355_F32: rc = launch_dv<CPPMEGA_MI355_F32>(p, stream); break;
    case CPPMEGA_MI355_F16: rc = launch_dv<CPPMEGA_MI355_F16>(p, stream); break;
    case CPPMEGA_MI355_BF16: rc = launch_dv<CPPMEGA_MI355_BF16>(p, stream); break;
    case CPPMEGA_MI355_E4M3: rc = launch_dv<CPPMEGA_MI355_E4M3>(p, stream); break;
    default: return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla: kv dtype %d", p.kv_dtype);
  }
  if (rc) return rc;
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

int sparse_mla_scores_launch(const MlaParams& p, hipStream_t stream) {
  if ((size_t)p.B * p.S * p.H == 0 || p.topk == 0) return 0;
  if (p.d_qk > 8192) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla: d_qk %d exceeds 8192", p.d_qk);
  const dim3 grid((unsigned)((size_t)p.B * p.S * p.H)), block(64);
  const size_t smem = (size_t)p.d_qk * 4;
  switch (p.kv_dtype) {
    case CPPMEGA_MI355_F32: hipLaunchKernelGGL(sparse_mla_scores_kernel<CPPMEGA_MI355_F32>, grid, block, smem, stream, p); break;
    case CPPMEGA_MI355_F16: hipLaunchKernelGGL(sparse_mla_scores_kernel<CPPMEGA_MI355_F16>, grid, block, smem, stream, p); break;
    case CPPMEGA_MI355_BF16: hipLaunchKernelGGL(sparse_mla_scores_kernel<CPPMEGA_MI355_BF16>, grid, block, smem, stream, p); break;
    case CPPMEGA_MI355_E4M3: hipLaunchKernelGGL(sparse_mla_scores_kernel<CPPMEGA_MI355_E4M3>, grid, block, smem, stream, p); break;
    default: return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla: kv dtype %d", p.kv_dtype);
  }
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
