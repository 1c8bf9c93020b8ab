// DSA indexer KL loss on the matrix cores, bfloat16 / float16 query and key (gfx950).
//
// Same result as dsa_indexer_loss.hip (the reference's two stages,
// cppmega_mlx/nn/_tilelang/dsa_splitk_indexer_loss.py:398-656 and :855-1165) with the attention
// scores of 16 query positions at a time on v_mfma_f32_16x16x32_{bf16,f16}:
//
//   workgroup = (batch, 16 consecutive query positions), 8 wavefronts; the causally visible keys
//   are cut into tiles of 32 and dealt to the wavefronts round robin, so a workgroup's keys are
//   read once per pass and the wavefronts never wait for each other inside a pass;
//   S^T[key, query] = K_h[key, :] . Q_h[query, :]^T per head h: the key rows are the A operand and
//   the query rows the B operand; the key fragments are fetched from memory in operand order
//   (16-byte loads, the next head's while the current one is reduced), the 16 query rows sit in
//   LDS when all their heads fit there (else they are fetched like the keys); a lane then holds
//   4 consecutive keys of one query per 16-key block, which is also how it reads the index
//   scores.
//
//   prologue  membership bits of the 16 index lists in LDS (sparse loss); max and sum of the index
//             softmax of each row over all keys;
//   pass 1    per (head, query): running max and sum of exp over the wavefront's tiles, kept in
//             LDS per wavefront, merged across the wavefronts at the end;
//   pass 2    the same scores again; p = mean over heads of exp(s - m_h) / d_h accumulates in
//             registers over the head loop of a tile, then sum of p * (log(p + eps) - log(q + eps)).
//
// Longest rows first: the workgroups of the last query positions are launched first.

#include "common.h"
#include "mfma_util.h"

namespace cm {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kRows = 16;              // query positions per workgroup
constexpr int kTile = 32;              // keys per wavefront step
constexpr float kEps = 1e-10f;

struct LossMfmaParams {
  const unsigned short* q;   // [ASq, AB, AH, AD]
  const unsigned short* k;   // [Sk, AB, AH, AD]
  const float* index_scores; // [AB, ASq, Sk]
  const float* mask;         // [AB, ASq, Sk] or NULL
  const void* topk_idx;      // [AB, ASq, topk] or NULL
  float* loss;               // [AB, ASq]
  int topk, index_dtype;
  int ASq, AB, AH, AD, Sk;
  int nblocks;               // ceil(ASq / 16)
  float scale;
};

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

template <bool F16>
__device__ __forceinline__ f32x4 mfma16(const __attribute__((ext_vector_type(4))) unsigned a, const __attribute__((ext_vector_type(4))) unsigned b, const f32x4 c) {
  if (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

constexpr int kQPad = 8;              // bfloat16 elements of padding per query row in LDS

// K_LDS (head sizes 64 and 128): the 32 key rows of a step are fetched with neighbouring lanes on
// neighbouring 16-byte pieces of a row (loads whose lanes each point into another row move a quarter
// of the bytes per clock) and reach operand order through a private LDS tile whose 16-byte slots are
// XOR-swizzled by the row.
template <bool F16, int KSTEPS, bool Q_LDS, bool K_LDS>
__global__ __launch_bounds__(kThreads) void dsa_indexer_loss_mfma_kernel(const LossMfmaParams p) {
  extern __shared__ __align__(16) float lds[];
  float* wstat = lds;                                     // [kWaves][AH][16][2]: running max, sum
  float* stat = wstat + kWaves * p.AH * 32;               // [AH][16][2]: max, 1 / sum
  float* idxstat = stat + p.AH * 32;                      // [16][2]: max, 1 / sum of the index softmax
  float* klred = idxstat + 32;                            // [kWaves][16]
  unsigned* bits = reinterpret_cast<unsigned*>(klred + kWaves * 16);   // [16][words] (sparse loss only)
  const int words = (p.Sk + 31) / 32;
  const int qpitch = p.AH * p.AD + kQPad;                 // elements per query row in LDS
  unsigned short* qs = reinterpret_cast<unsigned short*>(bits + (p.topk_idx ? kRows * ((words + 3) & ~3) : 0));   // [16][qpitch]
  constexpr int PPR = 4 * KSTEPS;                         // 16-byte pieces per key row of one head
  constexpr int RP = PPR >= 16 ? 1 : 16 / PPR;            // rows per 256 bytes
  unsigned char* kstage = reinterpret_cast<unsigned char*>(qs + (Q_LDS ? kRows * qpitch : 0)) + (threadIdx.x >> 6) * (32 * PPR * 16);

  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kg = lane >> 4;
  const int b = (int)(blockIdx.x % p.AB);
  const int blk = p.nblocks - 1 - (int)(blockIdx.x / p.AB);
  const int sq0 = blk * kRows;
  const int my_sq = sq0 + l16;                            // this lane's query position (as a B column)
  const bool my_row = my_sq < p.ASq;
  const int n_wg = min(sq0 + kRows, p.Sk);                // keys any row of the block can see
  const int ntiles = (n_wg + kTile - 1) / kTile;
  const bool sparse = p.topk_idx != nullptr;
  const size_t my_idx_row = ((size_t)b * p.ASq + (my_row ? my_sq : 0)) * (size_t)p.Sk;

  // ---- prologue ---------------------------------------------------------------------------
  if (sparse) {
    for (int w = tid; w < kRows * words; w += kThreads) bits[w] = 0u;
    __syncthreads();
    for (int e = tid; e < kRows * p.topk; e += kThreads) {
      const int r = e / p.topk, t = e - r * p.topk;
      if (sq0 + r < p.ASq) {
        const size_t at = ((size_t)b * p.ASq + sq0 + r) * (size_t)p.topk + t;
        const long long c = p.index_dtype == CPPMEGA_MI355_I64 ? static_cast<const long long*>(p.topk_idx)[at]
                                                               : (long long)static_cast<const int*>(p.topk_idx)[at];
        if (c >= 0 && c < p.Sk) atomicOr(&bits[r * words + (int)(c >> 5)], 1u << (c & 31));
      }
    }
    __syncthreads();
  }
  for (int r = wave; r < kRows; r += kWaves) {            // index softmax statistics of row r
    float m = -INFINITY, d = 0.0f;
    if (sq0 + r < p.ASq) {
      const size_t row = ((size_t)b * p.ASq + sq0 + r) * (size_t)p.Sk;
      for (int j = lane; j < p.Sk; j += 64) {
        float v = p.index_scores[row + j];
        if (p.mask) v += p.mask[row + j];
        if (sparse && !((bits[r * words + (j >> 5)] >> (j & 31)) & 1u)) v = -INFINITY;
        if (v > -INFINITY) {                              // (NaN scores are skipped as well)
          const float mn = fmaxf(m, v);
          d = d * __expf(m - mn) + __expf(v - mn);
          m = mn;
        }
      }
    }
    const float M = wave_max(m);
    float dsum = wave_sum(m > -INFINITY ? d * __expf(m - M) : 0.0f);
    if (lane == 0) {
      idxstat[r * 2] = M > -INFINITY ? M : 0.0f;
      idxstat[r * 2 + 1] = 1.0f / (dsum > 0.0f ? dsum : 1.0f);
    }
  }
  if (Q_LDS) {
    const int per_row = p.AH * p.AD / 8;                  // 16-byte pieces of one position's heads
    for (int piece = tid; piece < kRows * per_row; piece += kThreads) {
      const int r = piece / per_row, c8 = piece - r * per_row;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (sq0 + r < p.ASq)
        v = *reinterpret_cast<const uint4*>(p.q + ((size_t)(sq0 + r) * p.AB + b) * (size_t)p.AH * p.AD + c8 * 8);
      *reinterpret_cast<uint4*>(qs + r * qpitch + c8 * 8) = v;
    }
  }
  for (int e = lane; e < p.AH * 16; e += 64) {
    wstat[(wave * p.AH * 16 + e) * 2] = -INFINITY;
    wstat[(wave * p.AH * 16 + e) * 2 + 1] = 0.0f;
  }
  __syncthreads();

  const size_t head_stride = (size_t)p.AD;                // elements between heads of one position
  const size_t pos_stride = (size_t)p.AB * p.AH * p.AD;   // elements between positions
  const unsigned short* q_lane = p.q + (size_t)(my_row ? my_sq : 0) * pos_stride + (size_t)b * p.AH * p.AD + 8 * kg;

  // operand fragments of one (tile, head): two 16-key blocks of K and the query block
  typedef __attribute__((ext_vector_type(4))) unsigned u4;
  struct Frag { u4 ka[2 * KSTEPS]; u4 qb[Q_LDS ? 1 : KSTEPS]; };   // ka: [sub][step] in operand order, or the pieces in load order (K_LDS)
  const unsigned short* q_lds = qs + l16 * qpitch + 8 * kg;
  auto load_frag = [&](Frag& f, int key0, int h) {
    if (K_LDS) {
#pragma unroll
      for (int t = 0; t < 2 * KSTEPS; ++t) {
        const int P = lane + 64 * t, row = P / PPR, c = P % PPR;
        f.ka[t] = *reinterpret_cast<const u4*>(
            p.k + (size_t)min(key0 + row, p.Sk - 1) * pos_stride + ((size_t)b * p.AH + h) * head_stride + 8 * c);
      }
    } else {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const int key = key0 + 16 * sub + l16;
        const unsigned short* src = p.k + (size_t)min(key, p.Sk - 1) * pos_stride + ((size_t)b * p.AH + h) * head_stride + 8 * kg;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) f.ka[sub * KSTEPS + kk] = *reinterpret_cast<const u4*>(src + 32 * kk);
      }
    }
    if (!Q_LDS) {
#pragma unroll
      for (int kk = 0; kk < KSTEPS; ++kk) f.qb[kk] = *reinterpret_cast<const u4*>(q_lane + (size_t)h * head_stride + 32 * kk);
    }
  };
  // scores of this lane: s[sub][i] = key key0 + 16 * sub + 4 * kg + i against query my_sq
  auto scores = [&](const Frag& f, int h, float (&s)[2][4]) {
    u4 qb[KSTEPS];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk)
      qb[kk] = Q_LDS ? *reinterpret_cast<const u4*>(q_lds + h * p.AD + 32 * kk) : f.qb[Q_LDS ? 0 : kk];
    if (K_LDS) {                                          // load order -> the wavefront's LDS tile
#pragma unroll
      for (int t = 0; t < 2 * KSTEPS; ++t) {
        const int P = lane + 64 * t, row = P / PPR, c = P % PPR;
        *reinterpret_cast<u4*>(kstage + (row * PPR + (c ^ ((row / RP) % PPR))) * 16) = f.ka[t];
      }
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KSTEPS; ++kk) {
        u4 ka = f.ka[sub * KSTEPS + kk];
        if (K_LDS) {
          const int row = 16 * sub + l16, c = 4 * kk + kg;
          ka = *reinterpret_cast<const u4*>(kstage + (row * PPR + (c ^ ((row / RP) % PPR))) * 16);
        }
        acc = mfma16<F16>(ka, qb[kk], acc);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) s[sub][i] = acc[i] * p.scale;
    }
  };
  // which of the lane's 8 keys count, and the additive mask on them
  auto tile_mask = [&](int key0, bool (&ok)[2][4], float (&add)[2][4]) {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int kb = key0 + 16 * sub + 4 * kg;
      unsigned w = 0xffffffffu;
      if (sparse && kb < p.Sk) w = bits[l16 * words + (kb >> 5)] >> (kb & 31);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = kb + i;
        ok[sub][i] = my_row && key <= my_sq && key < p.Sk && ((w >> i) & 1u);
        add[sub][i] = 0.0f;
        if (p.mask && ok[sub][i]) {
          add[sub][i] = p.mask[my_idx_row + key];
          if (!(add[sub][i] > -INFINITY)) ok[sub][i] = false;
        }
      }
    }
  };

  // ---- pass 1: max and sum of exp per (head, query) -------------------------------------------
  for (int t = wave; t < ntiles; t += kWaves) {
    const int key0 = t * kTile;
    bool ok[2][4];
    float add[2][4];
    tile_mask(key0, ok, add);
    Frag cur, nxt;
    load_frag(cur, key0, 0);
    for (int h = 0; h < p.AH; ++h) {
      if (h + 1 < p.AH) load_frag(nxt, key0, h + 1);
      float s[2][4];
      scores(cur, h, s);
      float tmax = -INFINITY;
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[sub][i] = ok[sub][i] ? s[sub][i] + add[sub][i] : -INFINITY;
          tmax = fmaxf(tmax, s[sub][i]);
        }
      tmax = fmaxf(tmax, xor16(tmax));
      tmax = fmaxf(tmax, xor32(tmax));
      float* st = wstat + ((wave * p.AH + h) * 16 + l16) * 2;
      const float m_old = st[0], d_old = st[1];
      const float m_new = fmaxf(m_old, tmax);
      float esum = 0.0f;
      if (m_new > -INFINITY) {
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
          for (int i = 0; i < 4; ++i) esum += __expf(s[sub][i] - m_new);
      }
      esum += xor16(esum);
      esum += xor32(esum);
      if (kg == 0 && m_new > -INFINITY) {
        st[0] = m_new;
        st[1] = d_old * __expf(m_old - m_new) + esum;
      }
      if (h + 1 < p.AH) cur = nxt;
    }
  }
  __syncthreads();
  for (int e = tid; e < p.AH * 16; e += kThreads) {
    float M = -INFINITY;
    for (int w = 0; w < kWaves; ++w) M = fmaxf(M, wstat[(w * p.AH * 16 + e) * 2]);
    float dsum = 0.0f;
    if (M > -INFINITY)
      for (int w = 0; w < kWaves; ++w) {
        const float mw = wstat[(w * p.AH * 16 + e) * 2];
        if (mw > -INFINITY) dsum += wstat[(w * p.AH * 16 + e) * 2 + 1] * __expf(mw - M);
      }
    stat[e * 2] = M > -INFINITY ? M : 0.0f;
    stat[e * 2 + 1] = 1.0f / (dsum > 0.0f ? dsum : 1.0f);
  }
  __syncthreads();

  // ---- pass 2: the divergence -------------------------------------------------------------------
  const float m1 = idxstat[l16 * 2], inv1 = idxstat[l16 * 2 + 1];
  const bool idx_vec = (p.Sk & 3) == 0 && (reinterpret_cast<uintptr_t>(p.index_scores) & 15) == 0;
  const float inv_heads = 1.0f / (float)p.AH;
  float kl = 0.0f;
  for (int t = wave; t < ntiles; t += kWaves) {
    const int key0 = t * kTile;
    bool ok[2][4];
    float add[2][4];
    tile_mask(key0, ok, add);
    float pacc[2][4];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int i = 0; i < 4; ++i) pacc[sub][i] = 0.0f;
    Frag cur, nxt;
    load_frag(cur, key0, 0);
    for (int h = 0; h < p.AH; ++h) {
      if (h + 1 < p.AH) load_frag(nxt, key0, h + 1);
      float s[2][4];
      scores(cur, h, s);
      const float mh = stat[(h * 16 + l16) * 2], invd = stat[(h * 16 + l16) * 2 + 1];
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (ok[sub][i]) pacc[sub][i] += __expf(s[sub][i] + add[sub][i] - mh) * invd;
      if (h + 1 < p.AH) cur = nxt;
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int kb = key0 + 16 * sub + 4 * kg;
      // the lane's four index scores: one 16-byte load where the row allows it
      float iv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (my_row && kb <= my_sq && kb < p.Sk) {
        if (idx_vec) {
          const f32x4 t = *reinterpret_cast<const f32x4*>(p.index_scores + my_idx_row + kb);
          iv[0] = t[0]; iv[1] = t[1]; iv[2] = t[2]; iv[3] = t[3];
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (kb + i < p.Sk) iv[i] = p.index_scores[my_idx_row + kb + i];
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = kb + i;
        if (my_row && key <= my_sq && key < p.Sk) {       // causal keys; masked ones carry p = 0
          const float pj = pacc[sub][i] * inv_heads;
          float qj = 0.0f;
          if (ok[sub][i]) {
            const float v = iv[i] + add[sub][i];
            if (v > -INFINITY) qj = __expf(v - m1) * inv1;
          }
          kl += pj * (__logf(pj + kEps) - __logf(qj + kEps));
        }
      }
    }
  }
  kl += xor16(kl);
  kl += xor32(kl);
  if (kg == 0) klred[wave * 16 + l16] = kl;
  __syncthreads();
  if (tid < kRows && sq0 + tid < p.ASq) {
    float total = 0.0f;
    for (int w = 0; w < kWaves; ++w) total += klred[w * 16 + tid];
    p.loss[(size_t)b * p.ASq + sq0 + tid] = total;
  }
}

size_t lds_base_bytes(int AH, int Sk, bool sparse) {
  return ((size_t)kWaves * AH * 32 + (size_t)AH * 32 + 32 + kWaves * 16) * 4 + (sparse ? (size_t)kRows * ((((Sk + 31) / 32) + 3) & ~3) * 4 : 0);
}
size_t q_lds_bytes(int AH, int AD) { return (size_t)kRows * (AH * AD + kQPad) * 2; }

}  // namespace

bool dsa_indexer_loss_mfma_supports(const cppmega_mi355_dsa_loss_args_t& a) {
  if (a.in_dtype != CPPMEGA_MI355_BF16 && a.in_dtype != CPPMEGA_MI355_F16) return false;
  if (a.head_dim != 32 && a.head_dim != 64 && a.head_dim != 96 && a.head_dim != 128) return false;
  return lds_base_bytes(a.heads, a.seq_k, a.topk_indices != nullptr) <= 160 * 1024;
}

int dsa_indexer_loss_mfma_launch(const cppmega_mi355_dsa_loss_args_t& a, hipStream_t stream) {
  LossMfmaParams p;
  p.q = static_cast<const unsigned short*>(a.query);
  p.k = static_cast<const unsigned short*>(a.key);
  p.index_scores = a.index_scores; p.mask = a.index_mask; p.topk_idx = a.topk_indices; p.loss = a.loss;
  p.topk = a.topk; p.index_dtype = a.index_dtype;
  p.ASq = a.seq_q; p.AB = a.batch; p.AH = a.heads; p.AD = a.head_dim; p.Sk = a.seq_k;
  p.nblocks = (a.seq_q + kRows - 1) / kRows;
  p.scale = a.softmax_scale;
  const size_t grid = (size_t)p.nblocks * a.batch;
  if (grid > 0x7fffffffull) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "dsa_indexer_loss: too many rows for one launch");
  size_t lds = lds_base_bytes(a.heads, a.seq_k, a.topk_indices != nullptr);
  const bool q_lds = lds + q_lds_bytes(a.heads, a.head_dim) <= 64 * 1024;      // the query rows too, while two workgroups still fit a CU
  if (q_lds) lds += q_lds_bytes(a.heads, a.head_dim);
  const size_t k_bytes = (size_t)kWaves * 32 * (a.head_dim / 8) * 16;          // a 32-row key tile per wavefront
  const bool k_lds = (a.head_dim == 64 || a.head_dim == 128) && lds + k_bytes <= 160 * 1024;
  if (k_lds) lds += k_bytes;
  const bool f16 = a.in_dtype == CPPMEGA_MI355_F16;
  const void* fn = nullptr;
#define CM_PICK2(KS, KL)                                                                                                \
  fn = f16 ? (q_lds ? (const void*)dsa_indexer_loss_mfma_kernel<true, KS, true, KL> : (const void*)dsa_indexer_loss_mfma_kernel<true, KS, false, KL>) \
           : (q_lds ? (const void*)dsa_indexer_loss_mfma_kernel<false, KS, true, KL> : (const void*)dsa_indexer_loss_mfma_kernel<false, KS, false, KL>)
  switch (a.head_dim / 32) {
    case 1: CM_PICK2(1, false); break;
    case 2: if (k_lds) { CM_PICK2(2, true); } else { CM_PICK2(2, false); } break;
    case 3: CM_PICK2(3, false); break;
    default: if (k_lds) { CM_PICK2(4, true); } else { CM_PICK2(4, false); } break;
  }
#undef CM_PICK2
  if (lds > 64 * 1024) CM_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  void* kargs[] = {(void*)&p};
  CM_HIP_CHECK(hipLaunchKernel(fn, dim3((unsigned)grid), dim3(kThreads), kargs, lds, stream));
  return 0;
}

}  // namespace cm
