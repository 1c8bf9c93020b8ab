// Sparse index producers (gfx950): the index lists the sparse-attention kernels consume when
// no indexer scores exist -- a causal window, or the newest valid keys of an explicit mask.
//
//   causal   indices[b, s, g, j] = query_offset + s - j if in [0, key_length), else -1.
//            One thread per output element; pure index arithmetic, write-bound.
//   mask     per (b, s, g): the newest n = min(topk, key_length) valid keys of the mask row,
//            ascending, right-aligned, -1 in front.  One wavefront per row: count the valid
//            keys (the validity bits of up to 16384 keys stay in registers, longer rows are
//            read a second time), then place key number r (ascending among the valid ones, V
//            in all) at slot n - V + r if that is >= 0.  A lane reads 16 mask bytes (boolean
//            masks) or 16 floats per step; ranks come from popcounts and a wavefront prefix
//            sum; the kept keys of a step pass through LDS so that they leave coalesced.

#include "common.h"

namespace cm {
namespace {

struct CausalParams {
  void* out;
  long long total;          // B * S * G * topk
  int S, G, topk, wide;
  long long qoff, klen;
};

__global__ __launch_bounds__(256) void causal_indices_kernel(const CausalParams p) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < p.total; i += (long long)gridDim.x * 256) {
    const int j = (int)(i % p.topk);
    const int s = (int)((i / ((long long)p.topk * p.G)) % p.S);
    const long long pos = p.qoff + s - j;
    const long long v = (pos >= 0 && pos < p.klen) ? pos : -1;
    if (p.wide) ((long long*)p.out)[i] = v;
    else ((int*)p.out)[i] = (int)v;
  }
}

// int32 output, topk a multiple of 4: a thread writes four consecutive window slots (16 bytes);
// total / 4 fits 32 bits (checked on the host), so the index arithmetic is 32-bit
__global__ __launch_bounds__(256) void causal_indices_vec4_kernel(const CausalParams p) {
  const unsigned quads = (unsigned)(p.total >> 2), per_row = (unsigned)p.topk >> 2;
  for (unsigned q = blockIdx.x * 256u + threadIdx.x; q < quads; q += gridDim.x * 256u) {
    const unsigned row = q / per_row;                      // (b * S + s) * G + g
    const int j0 = (int)(q - row * per_row) * 4;
    const int s = (int)((row / (unsigned)p.G) % (unsigned)p.S);
    const long long pos0 = p.qoff + s - j0;
    int4 v;
    v.x = (pos0 >= 0 && pos0 < p.klen) ? (int)pos0 : -1;
    v.y = (pos0 - 1 >= 0 && pos0 - 1 < p.klen) ? (int)(pos0 - 1) : -1;
    v.z = (pos0 - 2 >= 0 && pos0 - 2 < p.klen) ? (int)(pos0 - 2) : -1;
    v.w = (pos0 - 3 >= 0 && pos0 - 3 < p.klen) ? (int)(pos0 - 3) : -1;
    reinterpret_cast<int4*>(p.out)[q] = v;
  }
}

struct MaskParams {
  const void* mask;
  long long sb, sg, ss;
  int* out;
  int B, S, G, n, K, dtype;
};

__device__ __forceinline__ bool finite_bits32(unsigned u) { return (u & 0x7f800000u) != 0x7f800000u; }

// exclusive prefix sum over the wavefront + the total
__device__ __forceinline__ int wave_exclusive(int v, int lane, int& total) {
  int x = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int y = __shfl_up(x, off, 64);
    if (lane >= off) x += y;
  }
  total = __shfl(x, 63, 64);
  return x - v;
}

// validity bits of the (up to) 16 keys k0 .. k0+15 of this lane
template <int DT>
__device__ __forceinline__ unsigned valid16(const MaskParams& p, const unsigned char* row, long long k0, bool vec_ok) {
  unsigned bits = 0;
  if (DT == CPPMEGA_MI355_MASK_BOOL) {
    if (vec_ok && k0 + 16 <= p.K) {
      const uint4 t = *reinterpret_cast<const uint4*>(row + k0);
      const unsigned w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // non-zero byte -> 0x01 per byte (x | x>>1 | .. folded into bit 0), then the four bit 0s gathered by a multiply (byte i -> bit 24 + i)
        unsigned x = w[d];
        x |= x >> 4; x |= x >> 2; x |= x >> 1;
        x &= 0x01010101u;
        bits |= (((x * 0x01020408u) >> 24) & 0xfu) << (4 * d);
      }
    } else {
      for (int i = 0; i < 16 && k0 + i < p.K; ++i) bits |= (row[k0 + i] ? 1u : 0u) << i;
    }
  } else {
    for (int i = 0; i < 16 && k0 + i < p.K; ++i) {
      bool ok;
      if (DT == CPPMEGA_MI355_MASK_F32) ok = finite_bits32(((const unsigned*)row)[k0 + i]);
      else if (DT == CPPMEGA_MI355_MASK_F16) ok = (((const unsigned short*)row)[k0 + i] & 0x7c00u) != 0x7c00u;
      else ok = (((const unsigned short*)row)[k0 + i] & 0x7f80u) != 0x7f80u;
      bits |= (ok ? 1u : 0u) << i;
    }
  }
  return bits;
}

template <int DT>
__global__ __launch_bounds__(256) void mask_indices_kernel(const MaskParams p) {
  const int lane = lane_id();
  // (32-bit arithmetic, the launcher checks that the row count fits: the 64-bit divisions were
  // several hundred instructions per wavefront)
  const unsigned r32 = blockIdx.x * 4u + (threadIdx.x >> 6);                    // (b * S + s) * G + g
  if (r32 >= (unsigned)p.B * (unsigned)p.S * (unsigned)p.G) return;
  const unsigned bs = r32 / (unsigned)p.G;
  const int g = (int)(r32 - bs * (unsigned)p.G);
  const int b = (int)(bs / (unsigned)p.S), s = (int)(bs - (unsigned)b * (unsigned)p.S);
  const long long r = r32;
  constexpr int ES = DT == CPPMEGA_MI355_MASK_BOOL ? 1 : (DT == CPPMEGA_MI355_MASK_F32 ? 4 : 2);
  const unsigned char* row = (const unsigned char*)p.mask + ((long long)b * p.sb + (long long)g * p.sg + (long long)s * p.ss) * ES;
  const bool vec_ok = (((size_t)row) & 15) == 0;
  int* out = p.out + r * p.n;
  __shared__ int strips[4][1024];
  int* strip = strips[threadIdx.x >> 6];
  // pass 1: validity bits (kept in registers for rows of up to 16384 keys) and their number
  constexpr int kKeep = 16;
  unsigned kept[kKeep];
  int mine = 0;
  {
    int st = 0;
    for (long long k0 = (long long)lane * 16; k0 < p.K; k0 += 64 * 16, ++st) {
      const unsigned bits = valid16<DT>(p, row, k0, vec_ok);
      if (st < kKeep) kept[st] = bits;
      mine += __popc(bits);
    }
  }
  int V;
  (void)wave_exclusive(mine, lane, V);
  // leading -1 slots
  const int lead = max(p.n - V, 0);
  for (int i = lane; i < lead; i += 64) out[i] = -1;
  // pass 2: place the newest n; key number r (ascending among the valid ones) goes to slot n - V + r
  const int first = V - p.n;                                                    // ranks below this are dropped
  int before = 0;                                                               // valid keys in earlier steps
  int st = 0;
  for (long long base = 0; base < p.K; base += 64 * 16, ++st) {
    const long long k0 = base + (long long)lane * 16;
    unsigned bits = 0u;
    if (k0 < p.K) bits = st < kKeep ? kept[st] : valid16<DT>(p, row, k0, vec_ok);
    const int cnt = __popc(bits);
    int step_total;
    int rank = before + wave_exclusive(cnt, lane, step_total);
    before += step_total;
    if (before <= first) continue;                                              // (uniform) nothing of this step is kept
    // the step's kept keys go through this wavefront's LDS strip in rank order and leave as
    // whole 256-byte stores (a lane's keys are consecutive ranks: direct stores would scatter)
    const int step_rank0 = before - step_total;                                 // rank of the step's first valid key
    if (step_total == 64 * 16) {
      // every key of the step is valid (the body of a causal mask): rank = position within the step,
      // so the kept keys are the consecutive numbers base + lo .. base + 1023 and need no strip
      const int lo = max(first - step_rank0, 0);
      for (int e = lo + lane; e < 64 * 16; e += 64) out[step_rank0 + e - first] = (int)(base + e);
      continue;
    }
    unsigned rest = bits;
    int rloc = rank - step_rank0;                                               // 0 .. 1023
    while (rest) {
      const int i = __builtin_ctz(rest);
      rest &= rest - 1;
      strip[rloc++] = (int)(k0 + i);
    }
    __builtin_amdgcn_wave_barrier();
    const int lo = max(first - step_rank0, 0);                                  // first kept entry of the strip
    for (int e = lo + lane; e < step_total; e += 64) out[step_rank0 + e - first] = strip[e];
    __builtin_amdgcn_wave_barrier();
  }
}

}  // namespace

int causal_indices_launch(const cppmega_mi355_causal_indices_args_t& a, hipStream_t stream) {
  if (a.batch < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "batch_size must be positive, got %d", a.batch);
  if (a.seq < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "seq_length must be positive, got %d", a.seq);
  if (a.groups < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "kv_group must be positive, got %d", a.groups);
  if (a.topk < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk must be positive, got %d", a.topk);
  if (a.query_offset < 0) return fail(CPPMEGA_MI355_ERR_SHAPE, "query_offset must be non-negative, got %lld", (long long)a.query_offset);
  if (a.key_length < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "key_length must be positive, got %lld", (long long)a.key_length);
  if (a.index_dtype != CPPMEGA_MI355_I32 && a.index_dtype != CPPMEGA_MI355_I64)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "causal_sparse_indices: index dtype %d", a.index_dtype);
  if (!a.indices) return fail(CPPMEGA_MI355_ERR_NULL, "causal_sparse_indices: indices is NULL");
  CausalParams p;
  p.out = a.indices; p.S = a.seq; p.G = a.groups; p.topk = a.topk; p.wide = a.index_dtype == CPPMEGA_MI355_I64;
  p.qoff = a.query_offset; p.klen = a.key_length;
  p.total = (long long)a.batch * a.seq * a.groups * a.topk;
  if (!p.wide && a.topk % 4 == 0 && (((size_t)a.indices) & 15) == 0 && (p.total >> 2) < 0xffffffffll) {
    const unsigned blocks = (unsigned)min(((p.total >> 2) + 255) / 256, (long long)256 * 32);
    hipLaunchKernelGGL(causal_indices_vec4_kernel, dim3(blocks), dim3(256), 0, stream, p);
  } else {
    const unsigned blocks = (unsigned)min((p.total + 255) / 256, (long long)256 * 32);
    hipLaunchKernelGGL(causal_indices_kernel, dim3(blocks), dim3(256), 0, stream, p);
  }
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

int mask_indices_launch(const cppmega_mi355_mask_indices_args_t& a, hipStream_t stream) {
  if (a.batch < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "batch_size must be positive, got %d", a.batch);
  if (a.seq < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "seq_length must be positive, got %d", a.seq);
  if (a.groups < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "kv_group must be positive, got %d", a.groups);
  if (a.topk < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk must be positive, got %d", a.topk);
  if (a.key_length < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "key_length must be positive, got %d", a.key_length);
  if (a.mask_dtype < CPPMEGA_MI355_MASK_BOOL || a.mask_dtype > CPPMEGA_MI355_MASK_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "mask_sparse_indices: mask dtype %d", a.mask_dtype);
  if (!a.mask || !a.indices) return fail(CPPMEGA_MI355_ERR_NULL, "mask_sparse_indices: mask / indices is NULL");
  MaskParams p;
  p.mask = a.mask; p.sb = a.stride_b; p.sg = a.stride_g; p.ss = a.stride_s; p.out = a.indices;
  p.B = a.batch; p.S = a.seq; p.G = a.groups; p.K = a.key_length; p.n = min(a.topk, a.key_length); p.dtype = a.mask_dtype;
  const long long rows = (long long)a.batch * a.seq * a.groups;
  if (rows > 0x7fffffffll) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_indices_from_attention_mask: %lld rows in one call", rows);
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  switch (a.mask_dtype) {
    case CPPMEGA_MI355_MASK_BOOL: hipLaunchKernelGGL(mask_indices_kernel<CPPMEGA_MI355_MASK_BOOL>, grid, block, 0, stream, p); break;
    case CPPMEGA_MI355_MASK_F32: hipLaunchKernelGGL(mask_indices_kernel<CPPMEGA_MI355_MASK_F32>, grid, block, 0, stream, p); break;
    case CPPMEGA_MI355_MASK_F16: hipLaunchKernelGGL(mask_indices_kernel<CPPMEGA_MI355_MASK_F16>, grid, block, 0, stream, p); break;
    default: hipLaunchKernelGGL(mask_indices_kernel<CPPMEGA_MI355_MASK_BF16>, grid, block, 0, stream, p); break;
  }
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
