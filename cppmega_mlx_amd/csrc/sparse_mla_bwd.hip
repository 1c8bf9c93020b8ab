// Sparse MLA backward for float carriers and per-token FP8 operands (gfx950).
//
// Gradients of out = softmax(sm_scale * q . K_sel^T) . K_sel[:, :d_v] with respect to q and the
// KV rows, for one cotangent d_out; the reference's sparse_mla_bwd_direct
// (cppmega_mlx/nn/_tilelang/sparse_mla_path_c.py:2644-2816), kernel(d_out, dkv, dq, indices, kv,
// q, sm_scale_buf) with dkv float32 accumulated by atomic adds and cleared beforehand (:3163-3230):
//
//   s_k  = sm_scale * q . kv[i_k]            p = softmax(s) over the selected, valid keys
//   dp_k = d_out . kv[i_k][:d_v]             ds_k = p_k * (dp_k - sum_j p_j dp_j)
//   dq   = sm_scale * sum_k ds_k kv[i_k]
//   dkv[i_k] += sm_scale * ds_k * q  (+ p_k * d_out on the first d_v channels)
//
// One workgroup per (batch, query, head).  Scores and dp come from the same pass over the
// selected rows (a wavefront per key, lanes across channels, so a row is read with coalesced
// loads); p, dp and ds stay in LDS; dq is a thread per channel walking the keys; the scatter into
// dkv is a thread per (key, channel) with float32 atomic adds (rows selected by several queries
// or heads meet there, in no fixed order: results agree to rounding, not bit for bit).  fp32
// arithmetic throughout, like the reference.
//
// The per-token FP8 form, fp8_sparse_mla_bwd_kernel(q_fp8, q_scale, kv_fp8, kv_scale, d_out,
// indices, sm_scale_buf, dq_dequant, dkv_dequant) (sparse_mla_fp8_path_c.py:1966-2214), is the
// same arithmetic on the dequantised values q = dec(byte) * q_scale[b,s,h],
// kv = dec(byte) * kv_scale[b,t,g]; the gradients are with respect to those values.

#include "common.h"

namespace cm {
namespace {

constexpr int kThreads = 256;

struct BwdParams {
  const void* q;
  const void* kv;
  const void* d_out;
  const void* indices;
  const float* q_scale;      // per (b, s, h) when q is e4m3, else NULL
  const float* kv_scale;     // per (b, t, g) when kv is e4m3, else NULL
  const float* sm_scale_dev;
  void* dq;
  float* dkv;
  int q_dtype, kv_dtype, do_dtype, dq_dtype, index_dtype;
  int B, S, H, G, Skv, topk, D, d_v;
  float sm_scale;
};

__global__ __launch_bounds__(kThreads) void fill_zero_kernel(float* dst, size_t n) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t j = i; j < n; j += stride) dst[j] = 0.0f;
}

__device__ __forceinline__ float block_reduce(float v, bool take_max, float* red) {
  const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
  v = take_max ? wave_max(v) : wave_sum(v);
  __syncthreads();                                      // red is free again
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < kThreads / 64; ++w) r = take_max ? fmaxf(r, red[w]) : r + red[w];
  return r;
}

__global__ __launch_bounds__(kThreads) void sparse_mla_bwd_kernel(const BwdParams p) {
  extern __shared__ __align__(16) float lds[];          // [topk] p, [topk] dp (then ds), [topk] rows (as int), [D] q, [d_v] d_out, [8] reduce
  float* pk = lds;
  float* dpk = lds + p.topk;
  int* rows = reinterpret_cast<int*>(lds + 2 * p.topk);
  float* qs = lds + 3 * p.topk;
  float* dos = qs + p.D;
  float* red = dos + p.d_v;
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t bsh = blockIdx.x;
  const int h = (int)(bsh % p.H);
  const size_t bs = bsh / p.H;
  const int b = (int)(bs / p.S);
  const int g = h / (p.H / p.G);
  const float sm_scale = p.sm_scale_dev ? *p.sm_scale_dev : p.sm_scale;
  const size_t idx_base = (bs * p.G + g) * (size_t)p.topk;

  const float q_sc = p.q_scale ? p.q_scale[bsh] : 1.0f;
  for (int d = tid; d < p.D; d += kThreads) qs[d] = load_as(p.q, bsh * p.D + d, p.q_dtype) * q_sc;
  for (int d = tid; d < p.d_v; d += kThreads) dos[d] = load_as(p.d_out, bsh * p.d_v + d, p.do_dtype);
  for (int k = tid; k < p.topk; k += kThreads) {
    const long long i = p.index_dtype == CPPMEGA_MI355_I64 ? ((const long long*)p.indices)[idx_base + k]
                                                          : (long long)((const int*)p.indices)[idx_base + k];
    rows[k] = (i >= 0 && i < p.Skv) ? (int)i : -1;
  }
  __syncthreads();

  // ---- scores and dp: a wavefront per key ----
  for (int k = wave; k < p.topk; k += kThreads / 64) {
    const int r = rows[k];
    float s = 0.0f, dp = 0.0f;
    if (r >= 0) {                                       // (uniform in the wavefront)
      const size_t krow = ((size_t)b * p.Skv + (size_t)r) * p.G + g;
      const size_t base = krow * (size_t)p.D;
      const float k_sc = p.kv_scale ? p.kv_scale[krow] : 1.0f;
      for (int d = lane; d < p.D; d += 64) {
        const float kvv = load_as(p.kv, base + d, p.kv_dtype) * k_sc;
        s = fmaf(qs[d], kvv, s);
        if (d < p.d_v) dp = fmaf(dos[d], kvv, dp);
      }
      s = wave_sum(s) * sm_scale;
      dp = wave_sum(dp);
    }
    if (lane == 0) {
      pk[k] = r >= 0 ? s : -INFINITY;
      dpk[k] = dp;
    }
  }
  __syncthreads();

  // ---- softmax over the valid keys ----
  float m = -INFINITY;
  for (int k = tid; k < p.topk; k += kThreads) m = fmaxf(m, pk[k]);
  m = block_reduce(m, true, red);
  float sum = 0.0f;
  for (int k = tid; k < p.topk; k += kThreads) {
    const float e = (rows[k] >= 0) ? expf(pk[k] - m) : 0.0f;
    pk[k] = e;
    sum += e;
  }
  sum = block_reduce(sum, false, red);
  const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
  float dot = 0.0f;
  for (int k = tid; k < p.topk; k += kThreads) {
    const float pv = pk[k] * inv;
    pk[k] = pv;
    dot = fmaf(pv, dpk[k], dot);
  }
  dot = block_reduce(dot, false, red);
  for (int k = tid; k < p.topk; k += kThreads) dpk[k] = pk[k] * (dpk[k] - dot);   // ds
  __syncthreads();

  // ---- dq: a thread per channel ----
  for (int d = tid; d < p.D; d += kThreads) {
    float acc = 0.0f;
    for (int k = 0; k < p.topk; ++k) {
      const int r = rows[k];
      if (r >= 0) {
        const size_t krow = ((size_t)b * p.Skv + (size_t)r) * p.G + g;
        const float k_sc = p.kv_scale ? p.kv_scale[krow] : 1.0f;
        acc = fmaf(dpk[k] * k_sc, load_as(p.kv, krow * (size_t)p.D + d, p.kv_dtype), acc);
      }
    }
    store_as(p.dq, bsh * p.D + d, p.dq_dtype, acc * sm_scale);
  }

  // ---- dkv: a thread per (key, channel), atomic accumulation ----
  const long long total = (long long)p.topk * p.D;
  for (long long kd = tid; kd < total; kd += kThreads) {
    const int k = (int)(kd / p.D), d = (int)(kd % p.D);
    const int r = rows[k];
    if (r < 0) continue;
    float v = sm_scale * dpk[k] * qs[d];
    if (d < p.d_v) v = fmaf(pk[k], dos[d], v);
    atomicAdd(&p.dkv[(((size_t)b * p.Skv + (size_t)r) * p.G + g) * (size_t)p.D + d], v);
  }
}

bool float_carrier(int dt) { return dt == CPPMEGA_MI355_F32 || dt == CPPMEGA_MI355_F16 || dt == CPPMEGA_MI355_BF16; }
bool operand_dtype(int dt) { return float_carrier(dt) || dt == CPPMEGA_MI355_E4M3; }

}  // namespace

bool sparse_mla_bwd_mfma_supports(const cppmega_mi355_sparse_mla_bwd_args_t& a);                    // sparse_mla_bwd_mfma.hip
int sparse_mla_bwd_mfma_launch(const cppmega_mi355_sparse_mla_bwd_args_t& a, hipStream_t stream);

int sparse_mla_bwd_launch(const cppmega_mi355_sparse_mla_bwd_args_t& a, hipStream_t stream) {
  if (!a.q || !a.kv || !a.d_out || !a.indices || !a.dq || !a.dkv) return fail(CPPMEGA_MI355_ERR_NULL, "sparse_mla_bwd: a pointer is NULL");
  if (a.batch < 0 || a.seq_q < 0 || a.heads < 1 || a.kv_groups < 1 || a.seq_kv < 0 || a.topk < 0 || a.d_qk < 1)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "sparse_mla_bwd: negative or empty dimension");
  if (a.heads % a.kv_groups != 0) return fail(CPPMEGA_MI355_ERR_SHAPE, "heads %d not divisible by kv_group %d", a.heads, a.kv_groups);
  if (a.d_v <= 0 || a.d_v > a.d_qk) return fail(CPPMEGA_MI355_ERR_SHAPE, "d_v must be in (0, %d], got %d", a.d_qk, a.d_v);
  if (!operand_dtype(a.q_dtype) || !operand_dtype(a.kv_dtype) || !float_carrier(a.d_out_dtype) || !float_carrier(a.dq_dtype))
    return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla_bwd: q / kv must be float32, float16, bfloat16 or e4m3; d_out and dq a float carrier");
  if ((a.q_dtype == CPPMEGA_MI355_E4M3 && !a.q_scale) || (a.kv_dtype == CPPMEGA_MI355_E4M3 && !a.kv_scale))
    return fail(CPPMEGA_MI355_ERR_NULL, "sparse_mla_bwd: e4m3 operands need their per-token scales");
  if (a.index_dtype != CPPMEGA_MI355_I32 && a.index_dtype != CPPMEGA_MI355_I64)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla_bwd: indices must be int32 or int64");
  const bool on_matrix_cores = sparse_mla_bwd_mfma_supports(a);      // bfloat16 / float16 (or per-token e4m3) operands
  const size_t lds = ((size_t)3 * a.topk + a.d_qk + a.d_v + 8) * sizeof(float);
  if (!on_matrix_cores && lds > 160 * 1024) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla_bwd: topk %d with d_qk %d needs %zu bytes of LDS (limit 160 KiB)", a.topk, a.d_qk, lds);
  const size_t n_dkv = (size_t)a.batch * a.seq_kv * a.kv_groups * a.d_qk;
  if (a.clear_dkv && n_dkv) {
    size_t blocks = (n_dkv + kThreads * 8 - 1) / (kThreads * 8);
    if (blocks > 65535u * 16) blocks = 65535u * 16;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, stream, a.dkv, n_dkv);
  }
  const size_t lanes = (size_t)a.batch * a.seq_q * a.heads;
  if (lanes == 0) return 0;
  if (on_matrix_cores) return sparse_mla_bwd_mfma_launch(a, stream);
  if (lanes > 0x7fffffffull) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla_bwd: too many (batch, query, head) rows for one launch");
  BwdParams p;
  p.q = a.q; p.kv = a.kv; p.d_out = a.d_out; p.indices = a.indices; p.sm_scale_dev = a.sm_scale_dev; p.dq = a.dq; p.dkv = a.dkv;
  p.q_scale = a.q_dtype == CPPMEGA_MI355_E4M3 ? a.q_scale : nullptr;
  p.kv_scale = a.kv_dtype == CPPMEGA_MI355_E4M3 ? a.kv_scale : nullptr;
  p.q_dtype = a.q_dtype; p.kv_dtype = a.kv_dtype; p.do_dtype = a.d_out_dtype; p.dq_dtype = a.dq_dtype; p.index_dtype = a.index_dtype;
  p.B = a.batch; p.S = a.seq_q; p.H = a.heads; p.G = a.kv_groups; p.Skv = a.seq_kv; p.topk = a.topk; p.D = a.d_qk; p.d_v = a.d_v;
  p.sm_scale = a.sm_scale;
  if (lds > 64 * 1024)
    CM_HIP_CHECK(hipFuncSetAttribute((const void*)sparse_mla_bwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(sparse_mla_bwd_kernel, dim3((unsigned)lanes), dim3(kThreads), lds, stream, p);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
