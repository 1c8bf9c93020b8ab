// DSA indexer KL loss, per position (gfx950).
//
// The two fused stages of the reference (cppmega_mlx/nn/_tilelang/dsa_splitk_indexer_loss.py:
// stage 1 :327-656 collects softmax statistics, stage 2 :781-1165 reduces the divergence) as one
// pass per (batch, query position), which needs no statistics buffers in memory:
//
//   s_h[j] = scale * q[sq,b,h,:] . k[j,b,h,:] (+ mask[b,sq,j])   for j <= sq (causal), per head h
//   p[j]   = (1 / AH) * sum_h exp(s_h[j] - m_h) / d_h            m_h, d_h: max and sum of exp over j <= sq
//   v[j]   = index_scores[b,sq,j] (+ mask[b,sq,j])               for every j < Sk (no causal cut: :585-601)
//   q_[j]  = exp(v[j] - m1) / d1
//   loss[b,sq] = sum_{j <= sq} p[j] * (log(p[j] + 1e-10) - log(q_[j] + 1e-10))
//
// with the reference's guards: a maximum that is still the "nothing valid" sentinel becomes 0 and
// a denominator <= 0 becomes 1 (:556-561, :1104-1109).  The sparse variant's mask is 0 at a row's
// top-k positions and -inf elsewhere.  The reference scatters it into a float [AB, ASq, Sk] tensor
// on the host side (:1380-1445); here the kernel takes the index list itself and keeps the row's
// membership as one bit per key in LDS, so that tensor is never written or read.  Entries outside
// [0, Sk) select nothing.  An additive float mask of the same shape is accepted as well.
//
// One workgroup per (b, sq): the head-averaged probabilities of the row live in LDS, a thread owns
// keys j = tid, tid + 256, ... and walks their key rows with 16-byte loads; fp32 arithmetic on
// bf16 / fp16 / fp32 inputs.

#include "common.h"

namespace cm {
namespace {

constexpr int kThreads = 256;
constexpr float kEps = 1e-10f;
constexpr float kSentinel = -3.4028234663852886e38f;

struct LossParams {
  const void* q;             // [ASq, AB, AH, AD]
  const void* k;             // [Sk, AB, AH, AD]
  const float* index_scores; // [AB, ASq, Sk]
  const float* mask;         // [AB, ASq, Sk] or NULL
  const void* topk_idx;      // [AB, ASq, topk] or NULL
  int topk, index_dtype;
  float* loss;               // [AB, ASq]
  int in_dtype;
  int ASq, AB, AH, AD, Sk;
  float scale;
};

__device__ __forceinline__ float block_reduce(float v, bool take_max, float* red) {
  const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
  v = take_max ? wave_max(v) : wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) r = take_max ? fmaxf(r, red[w]) : r + red[w];
  return r;
}

__global__ __launch_bounds__(kThreads) void dsa_indexer_loss_kernel(const LossParams p) {
  extern __shared__ __align__(16) float lds[];           // [Sk] p accumulators, [Sk] scores of one head, [AD] q row, [8] reduce
  float* pacc = lds;
  float* sc = lds + p.Sk;
  float* qs = sc + p.Sk;
  float* red = qs + p.AD;
  unsigned* bits = reinterpret_cast<unsigned*>(red + 8);   // [ceil(Sk / 32)] membership of the row's index list
  const int tid = (int)threadIdx.x;
  const int b = (int)(blockIdx.x % p.AB);
  const int sq = (int)(blockIdx.x / p.AB);
  const int n = min(sq + 1, p.Sk);                        // keys 0 .. n-1 are causally visible
  const size_t row = ((size_t)b * p.ASq + sq) * (size_t)p.Sk;
  for (int j = tid; j < n; j += kThreads) pacc[j] = 0.0f;
  if (p.topk_idx) {
    for (int w = tid; w < (p.Sk + 31) / 32; w += kThreads) bits[w] = 0u;
    __syncthreads();
    const size_t list = ((size_t)b * p.ASq + sq) * (size_t)p.topk;
    for (int t = tid; t < p.topk; t += kThreads) {
      const long long c = p.index_dtype == CPPMEGA_MI355_I64 ? static_cast<const long long*>(p.topk_idx)[list + t]
                                                             : (long long)static_cast<const int*>(p.topk_idx)[list + t];
      if (c >= 0 && c < p.Sk) atomicOr(&bits[c >> 5], 1u << (c & 31));
    }
  }
  auto mask_at = [&](int j) -> float {
    float mv = p.mask ? p.mask[row + j] : 0.0f;
    if (p.topk_idx && !((bits[j >> 5] >> (j & 31)) & 1u)) mv = -INFINITY;
    return mv;
  };

  for (int h = 0; h < p.AH; ++h) {
    __syncthreads();                                      // qs and sc are free again
    for (int d = tid; d < p.AD; d += kThreads)
      qs[d] = load_as(p.q, (((size_t)sq * p.AB + b) * p.AH + h) * (size_t)p.AD + d, p.in_dtype);
    __syncthreads();
    float m = kSentinel;
    for (int j = tid; j < n; j += kThreads) {
      const size_t base = (((size_t)j * p.AB + b) * p.AH + h) * (size_t)p.AD;
      float acc = 0.0f;
      if (p.in_dtype != CPPMEGA_MI355_F32 && (p.AD & 7) == 0) {
        const uint4* kr = reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(p.k) + base);
        for (int d8 = 0; d8 < p.AD / 8; ++d8) {
          const uint4 w = kr[d8];
          const unsigned u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const unsigned short lo = (unsigned short)(u[e] & 0xffffu), hi = (unsigned short)(u[e] >> 16);
            const float f0 = p.in_dtype == CPPMEGA_MI355_BF16 ? bf16_bits_to_f32(lo) : f16_bits_to_f32(lo);
            const float f1 = p.in_dtype == CPPMEGA_MI355_BF16 ? bf16_bits_to_f32(hi) : f16_bits_to_f32(hi);
            acc = fmaf(qs[d8 * 8 + 2 * e], f0, acc);
            acc = fmaf(qs[d8 * 8 + 2 * e + 1], f1, acc);
          }
        }
      } else if (p.in_dtype == CPPMEGA_MI355_F32 && (p.AD & 3) == 0) {
        const float4* kr = reinterpret_cast<const float4*>(static_cast<const float*>(p.k) + base);
        for (int d4 = 0; d4 < p.AD / 4; ++d4) {
          const float4 w = kr[d4];
          acc = fmaf(qs[d4 * 4], w.x, acc); acc = fmaf(qs[d4 * 4 + 1], w.y, acc);
          acc = fmaf(qs[d4 * 4 + 2], w.z, acc); acc = fmaf(qs[d4 * 4 + 3], w.w, acc);
        }
      } else {
        for (int d = 0; d < p.AD; ++d) acc = fmaf(qs[d], load_as(p.k, base + d, p.in_dtype), acc);
      }
      float s = acc * p.scale + mask_at(j);
      s = fmaxf(s, kSentinel);                            // (-inf from the mask joins the sentinel)
      sc[j] = s;
      m = fmaxf(m, s);
    }
    m = block_reduce(m, true, red);
    if (m <= kSentinel) m = 0.0f;
    float dsum = 0.0f;
    for (int j = tid; j < n; j += kThreads) {
      const float e = expf(sc[j] - m);
      sc[j] = e;
      dsum += e;
    }
    dsum = block_reduce(dsum, false, red);
    const float inv = 1.0f / (dsum <= 0.0f ? 1.0f : dsum);
    for (int j = tid; j < n; j += kThreads) pacc[j] += sc[j] * inv;
  }

  // index softmax statistics over every key
  float m1 = kSentinel;
  for (int j = tid; j < p.Sk; j += kThreads) {
    const float v = p.index_scores[row + j] + mask_at(j);
    m1 = fmaxf(m1, fmaxf(v, kSentinel));
  }
  m1 = block_reduce(m1, true, red);
  if (m1 <= kSentinel) m1 = 0.0f;
  float d1 = 0.0f;
  for (int j = tid; j < p.Sk; j += kThreads) {
    const float v = p.index_scores[row + j] + mask_at(j);
    d1 += expf(fmaxf(v, kSentinel) - m1);
  }
  d1 = block_reduce(d1, false, red);
  const float inv1 = 1.0f / (d1 <= 0.0f ? 1.0f : d1);

  const float inv_heads = 1.0f / (float)p.AH;
  float kl = 0.0f;
  for (int j = tid; j < n; j += kThreads) {
    const float pj = pacc[j] * inv_heads;
    const float v = p.index_scores[row + j] + mask_at(j);
    const float qj = expf(fmaxf(v, kSentinel) - m1) * inv1;
    kl += pj * (logf(pj + kEps) - logf(qj + kEps));
  }
  kl = block_reduce(kl, false, red);
  if (tid == 0) p.loss[(size_t)b * p.ASq + sq] = kl;
}

}  // namespace

bool dsa_indexer_loss_mfma_supports(const cppmega_mi355_dsa_loss_args_t& a);                    // dsa_indexer_loss_mfma.hip
int dsa_indexer_loss_mfma_launch(const cppmega_mi355_dsa_loss_args_t& a, hipStream_t stream);

int dsa_indexer_loss_launch(const cppmega_mi355_dsa_loss_args_t& a, hipStream_t stream) {
  if (!a.query || !a.key || !a.index_scores || !a.loss) return fail(CPPMEGA_MI355_ERR_NULL, "dsa_indexer_loss: a pointer is NULL");
  if (a.seq_q < 0 || a.batch < 0 || a.heads < 0 || a.head_dim < 0 || a.seq_k < 0)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "dsa_indexer_loss: negative dimension");
  if (a.heads > 128) return fail(CPPMEGA_MI355_ERR_SHAPE, "dsa_indexer_loss: AH > 128 is numerically unsafe (got AH=%d)", a.heads);
  if (a.in_dtype != CPPMEGA_MI355_F32 && a.in_dtype != CPPMEGA_MI355_F16 && a.in_dtype != CPPMEGA_MI355_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "dsa_indexer_loss: query / key must be float32, float16 or bfloat16");
  if ((size_t)a.seq_q * a.batch == 0 || a.heads == 0 || a.head_dim == 0 || a.seq_k == 0) return 0;
  if (a.topk_indices) {
    if (a.topk < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "dsa_indexer_loss: an index list needs topk >= 1 (an empty list masks every key)");
    if (a.index_dtype != CPPMEGA_MI355_I32 && a.index_dtype != CPPMEGA_MI355_I64)
      return fail(CPPMEGA_MI355_ERR_DTYPE, "dsa_indexer_loss: topk_indices must be int32 or int64");
  }
  if (dsa_indexer_loss_mfma_supports(a)) return dsa_indexer_loss_mfma_launch(a, stream);    // bfloat16 / float16 rows
  const size_t lds = ((size_t)2 * a.seq_k + a.head_dim + 8 + (a.seq_k + 31) / 32) * sizeof(float);
  if (lds > 160 * 1024) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "dsa_indexer_loss: Sk %d needs %zu bytes of LDS (limit 160 KiB)", a.seq_k, lds);
  if ((size_t)a.seq_q * a.batch > 0x7fffffffull) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "dsa_indexer_loss: too many rows for one launch");
  LossParams p;
  p.q = a.query; p.k = a.key; p.index_scores = a.index_scores; p.mask = a.index_mask; p.loss = a.loss;
  p.in_dtype = a.in_dtype; p.ASq = a.seq_q; p.AB = a.batch; p.AH = a.heads; p.AD = a.head_dim; p.Sk = a.seq_k;
  p.scale = a.softmax_scale;
  p.topk_idx = a.topk_indices; p.topk = a.topk; p.index_dtype = a.index_dtype;
  if (lds > 64 * 1024)
    CM_HIP_CHECK(hipFuncSetAttribute((const void*)dsa_indexer_loss_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(dsa_indexer_loss_kernel, dim3((unsigned)((size_t)a.seq_q * a.batch)), dim3(kThreads), lds, stream, p);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
