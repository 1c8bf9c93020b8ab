// Sparse MLA forward over an FP8 latent KV cache on the matrix cores (gfx950):
// 64 or 128 heads share every gathered key row.
//
// Shapes served: bf16 queries of 576 = 512 latent + 64 rope channels, d_v = 512,
// keys as e4m3 latent [512] with fp32 scales (per 128 / 256 / 512 channels, or
// per row, or none) plus a bf16 rope tail [64]; at least 33 heads per KV group.
//
// Workgroup = (query, KV group, chunk of 32*HG heads, key split), 4 wavefronts,
// key tiles of 32 rows.
//
//   HBM -> LDS   Rows travel as raw bytes (e4m3 latent, bf16 rope, fp32 scales)
//                straight into a ring of four LDS tile slots by the load unit
//                (global_load_lds), three tiles ahead.  Nothing is ever
//                rewritten in LDS: both matrix products dequantise in the
//                operand path, in registers.  The 16-byte chunk c of row r lives
//                at chunk c ^ (r & 7), which makes both access patterns below
//                conflict-free; the swizzle costs nothing because each lane of
//                a load instruction picks which source chunk it fetches.
//   S^T = K.Q^T  Wavefront w owns 32 heads (their Q^T fragments stay in 144
//                VGPRs) and HG/2 sub-tiles of 16 keys.  A K fragment is one
//                16-byte LDS read of e4m3 bytes, converted to bf16 by
//                v_cvt_scalef32_pk_bf16_fp8 with the power-of-two part of the
//                block scale (exact); the mantissa part of the scale multiplies
//                the fp32 partial sum of that 128-channel block.  The contraction
//                order inside a 64-channel step is permuted (the same way for K
//                and Q) so that one 16-byte read feeds two MFMA k-steps.
//   softmax      base 2, running maximum per (wavefront, head) moved lazily.
//                P is written to LDS as bf16 in the B-operand layout of the
//                second product, once per scale block with V's block scale
//                folded in (so V itself is converted unscaled, exactly).
//   O^T += V^T.P^T  Wavefront w owns value channels 128w..128w+127 for all heads
//                of the workgroup: V^T fragments are transposing 8-byte LDS reads
//                (ds_read_b64_tr_b8) of the raw tile.  Accumulators are kept per
//                producing wavefront (its running maximum is private), 256 AGPRs
//                in all, so the key loop needs one barrier per tile and no
//                agreement on maxima; the two accumulator sets of a head (HG = 2)
//                are merged once at the end, in registers.
//   pipeline     iteration t: barrier; issue tile t+3; QK + softmax of tile t+1;
//                PV of tile t.
//
// Key splits write their accumulators (rounded to bf16) to the workspace exactly as the lanes
// hold them (512 B per store), plus (max, sum) per head; sparse_mla_latent_combine_kernel merges the
// splits and does the transposition to [head][channel] that the single-split path does in LDS.

#include <cstdlib>

#include "sparse_mla_common.h"
#include "mfma_util.h"

namespace cm {
namespace {

constexpr int kLat = 512;
constexpr int kRope = 64;
constexpr int kDqk = kLat + kRope;
constexpr int kTK = 32;                         // keys per tile
constexpr int kRing = 4;                        // tile slots
constexpr int kLatBytes = kTK * kLat;           // 16384
constexpr int kRopeBytes = kTK * kRope * 2;     // 4096
constexpr int kScaleBytes = kTK * 4 * 4;        // 512: up to four fp32 scales per row
constexpr int kSlotBytes = kLatBytes + kRopeBytes + kScaleBytes;   // 20992
constexpr int kRingBytes = kRing * kSlotBytes;  // 83968
constexpr int kMaxKeys = 2048;                  // keys of one split (their rows are staged in LDS)
constexpr int kKeyInts = kMaxKeys + 4 * kTK;    // + the tiles the pipeline prefetches past the end
constexpr int kXPitch = 132;                    // floats per head row of the output transpose (128 + 4)
constexpr int kPartFloats = 4 * 16 * 64 * 4;         // partial values (bf16) of one 32-head group: [4 wavefronts][16 rows][64 lanes][4]
constexpr float kLazy = 8.0f;                   // move a running maximum only when it grows by > 2^8

template <int HG>
struct Geo {
  static constexpr int kSpw = HG / 2;                       // 16-key sub-tiles per wavefront and tile
  static constexpr int kSlots = 2 * HG;                     // (k-step, head group) pairs of a tile
  static constexpr int kPBytes = 4 * kSlots * 1024;         // one parity: 4 scale variants
  static constexpr int kPOff = kRingBytes;
  static constexpr int kFacOff = kPOff + 2 * kPBytes;       // [parity][4 producers][32 heads] fp32
  static constexpr int kFlagOff = kFacOff + 2 * 4 * 32 * 4; // [parity][4 producers] int
  static constexpr int kStatOff = kFlagOff + 2 * 4 * 4;     // [4 producers][32 heads][2] fp32
  static constexpr int kKeyOff = kStatOff + 4 * 32 * 2 * 4;
  static constexpr int kSmem = kKeyOff + kKeyInts * 4;
  static_assert(kSmem <= 160 * 1024, "LDS budget");
  static_assert(4 * 32 * kXPitch * 4 <= kRingBytes, "the output transpose reuses the ring");
};

// 2^x by the hardware instruction alone (x <= ~8 here; tiny results may flush to zero)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ bf16x8 cvt8(unsigned w0, unsigned w1, float pow2_scale) {
  const unsigned o0 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w0, pow2_scale, false));
  const unsigned o1 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w0, pow2_scale, true));
  const unsigned o2 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w1, pow2_scale, false));
  const unsigned o3 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w1, pow2_scale, true));
  return __builtin_bit_cast(bf16x8, make_uint4(o0, o1, o2, o3));
}

// scale = pow2 * mant: pow2 keeps the exponent field (what the converter applies, exactly),
// mant the sign and mantissa.  A zero or denormal scale comes out as ~2^-127 (its products
// vanish either way); inf / nan scales stay non-finite.
__device__ __forceinline__ float scale_pow2(float s) { return __uint_as_float(__float_as_uint(s) & 0x7f800000u); }
__device__ __forceinline__ float scale_mant(float s) {
  return __uint_as_float((__float_as_uint(s) & 0x807fffffu) | 0x3f800000u);
}

// The score product uses the compiler's own MFMA (this file is built with
// -mllvm -amdgpu-mfma-vgpr-form, so its accumulators are ordinary VGPRs): the compiler then
// knows the instruction's latency and pads its hazards exactly.  The value product keeps the
// inline form: its 256 accumulator registers must be AGPRs.
__device__ __forceinline__ void mfma_s(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}

// HG: 32-head groups per workgroup (2 or 4); NBLK: fp32 scales per key row (1, 2 or 4)
template <int HG, int NBLK>
__global__ __launch_bounds__(256, 1) void sparse_mla_latent_kernel(const MlaParams p) {
  using G_ = Geo<HG>;
  constexpr int SPW = G_::kSpw;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = (int)threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- which (query, KV group, head chunk, split).  Workgroup ids that are equal modulo 8 run on
  //      the same XCD and share its L2: every workgroup of one (query, KV group) gets such ids, so
  //      its query rows are fetched from HBM once (all key splits read them) and the head chunks
  //      of a split find the gathered key rows of their sibling in cache ----
  const int chunks = (p.heads_per_group + 32 * HG - 1) / (32 * HG);
  const long long per_q = (long long)p.num_splits * chunks;    // workgroups of one (query, KV group)
  const long long nq = (long long)p.B * p.S * p.G;
  const long long nq8 = nq & ~7ll;
  long long qg;
  int chunk, split;
  {
    const long long id = blockIdx.x;
    long long r;
    if (id < nq8 * per_q) {
      const long long slot = id >> 3;
      qg = (slot / per_q) * 8 + (id & 7);
      r = slot % per_q;
    } else {
      const long long rest = id - nq8 * per_q;
      qg = nq8 + rest / per_q;
      r = rest % per_q;
    }
    split = (int)(r / chunks);
    chunk = (int)(r % chunks);
  }
  const int g = (int)(qg % p.G);
  const size_t bs = (size_t)(qg / p.G);           // b*S + s
  const int b = (int)(bs / p.S);
  const int head0 = g * p.heads_per_group + chunk * 32 * HG;
  const int heads_here = min(32 * HG, p.heads_per_group - chunk * 32 * HG);
  const size_t idx_base = (bs * p.G + g) * (size_t)p.topk;
  const int key_begin = split * p.keys_per_split;
  const int key_end = min(p.topk, key_begin + p.keys_per_split);
  const int n_keys = max(0, key_end - key_begin);
  const int list_tiles = (n_keys + kTK - 1) / kTK;   // tiles the index list spans; trailing all-skipped tiles are dropped below

  constexpr int nblk = NBLK;
  const bool has_scale = p.kv_scale_kind != CPPMEGA_MI355_SCALE_NONE;   // otherwise the scale area holds ones

  // roles: this wavefront produces scores for head group hgq and sub-tiles sub0.., and
  // accumulates value channels 128*wave.. for every head group
  const int hgq = wave % HG;
  const int sub0 = (wave / HG) * SPW;

  int* keys = reinterpret_cast<int*>(smem + G_::kKeyOff);
  float* facbuf = reinterpret_cast<float*>(smem + G_::kFacOff);
  int* flagbuf = reinterpret_cast<int*>(smem + G_::kFlagOff);
  float* stats = reinterpret_cast<float*>(smem + G_::kStatOff);

  // The first index entries are requested before the (much larger) query fragments: loads return
  // in order, and the key rows can only be fetched once the indices are known.  Every load of
  // this prologue is unconditional (positions and heads are clamped instead): only then can
  // the compiler wait for the index words by count and leave the query loads in flight.
  int early_lo[2], early_hi[2];
  {
    const bool wide = p.index_dtype == CPPMEGA_MI355_I64;
    const int* words = (const int*)p.indices;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const size_t at = idx_base + (size_t)min(key_begin + tid + 256 * e, p.topk - 1);
      const size_t w0 = wide ? 2 * at : at;
      early_lo[e] = words[w0];
      early_hi[e] = words[w0 + (wide ? 1 : 0)];
    }
  }

  // ---- Q^T fragments: lane (head n = lane%16, kq = lane/16), heads n and 16+n of group hgq.
  //      latent step ks (64 channels): fragments 2ks, 2ks+1 hold channels 64ks + 16kq + {0..7}, {8..15};
  //      rope step r: fragment 16+r holds channels 512 + 32r + 8kq + {0..7} ----
  bf16x8 qf[2][18];
  {
    const int n = lane & 15, kq = lane >> 4;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int h = 32 * hgq + hh * 16 + n;
      // heads past the end of the group repeat head 0: their columns stay finite and are never stored
      const unsigned short* qrow = (const unsigned short*)p.q + (bs * p.H + head0 + (h < heads_here ? h : 0)) * (size_t)kDqk;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const uint4 t0 = *reinterpret_cast<const uint4*>(qrow + 64 * ks + 16 * kq);
        const uint4 t1 = *reinterpret_cast<const uint4*>(qrow + 64 * ks + 16 * kq + 8);
        qf[hh][2 * ks] = __builtin_bit_cast(bf16x8, t0);
        qf[hh][2 * ks + 1] = __builtin_bit_cast(bf16x8, t1);
      }
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const uint4 t = *reinterpret_cast<const uint4*>(qrow + kLat + 32 * r + 8 * kq);
        qf[hh][16 + r] = __builtin_bit_cast(bf16x8, t);
      }
    }
  }
  // ---- cache rows of this split's keys -> LDS (-1 = skipped) ----
  int* last_valid = reinterpret_cast<int*>(smem);          // (ring memory, not yet in use)
  if (tid == 0) *last_valid = -1;
  __syncthreads();
  {
    int mine = -1;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int i = tid + 256 * e;
      if (i < list_tiles * kTK + 4 * kTK) {
        const long long k = p.index_dtype == CPPMEGA_MI355_I64
                                ? (long long)(((unsigned long long)(unsigned)early_hi[e] << 32) | (unsigned)early_lo[e])
                                : (long long)early_lo[e];
        const bool ok = i < n_keys && k >= 0 && k < p.Skv;
        keys[i] = ok ? (int)k : -1;
        if (ok) mine = i;
      }
    }
    for (int i = tid + 512; i < list_tiles * kTK + 4 * kTK; i += 256) {
      int row = -1;
      if (i < n_keys) {
        const long long k = load_index(p, idx_base + key_begin + i);
        if (k >= 0 && k < p.Skv) { row = (int)k; mine = i; }
      }
      keys[i] = row;
    }
    mine = max(mine, __shfl_xor(mine, 1, 64));
    mine = max(mine, __shfl_xor(mine, 2, 64));
    mine = max(mine, __shfl_xor(mine, 4, 64));
    mine = max(mine, __shfl_xor(mine, 8, 64));
    mine = max(mine, __shfl_xor(mine, 16, 64));
    mine = max(mine, __shfl_xor(mine, 32, 64));
    if (lane == 0 && mine >= 0) atomicMax(last_valid, mine);
  }

  if (!has_scale) {                               // no scales in memory: every slot's scale area is 1.0 for good
    for (int i = tid; i < kRing * kTK; i += 256)
      reinterpret_cast<float*>(smem + (i / kTK) * kSlotBytes + kLatBytes + kRopeBytes)[i % kTK] = 1.0f;
  }
  __syncthreads();                                // keys[] is complete
  // causal padding puts the skipped (-1) slots at the end of a list: tiles past the last valid key do nothing
  const int n_tiles = __builtin_amdgcn_readfirstlane((*last_valid + kTK) / kTK);
  __syncthreads();                                // everyone has read it before the ring is written

  // ---- HBM -> LDS: this wavefront brings rows 8*wave .. 8*wave+7 of a tile.  A skipped key
  //      fetches cache row 0 instead (its probability is zero), so every wavefront issues
  //      the same number of loads for every tile and the in-order load counter can be
  //      waited on by count. ----
  // Row numbers fit 32 bits (checked on the host).  The loads are written as inline assembly:
  // the compiler would otherwise order every later LDS read behind them (vmcnt(0)), which
  // serialises the pipeline this kernel is built around.
  //   latent : instruction i of wavefront w carries rows 8i+2w (lanes 0..31) and 8i+2w+1, so a
  //            lane's swizzle term (row & 7) is the same for all i
  //   rope   : one instruction, rows 8w + lane/8
  //   scales : element 64w + lane of [32 rows][nblk]
  const bool scale_op = has_scale && 64 * wave < kTK * nblk;
  const size_t group_row0 = ((size_t)b * p.Skv) * p.G + g;     // cache row of key 0; key k is G rows further per step
  const int lat_row = 2 * wave + (lane >> 5);                 // + 8i
  const int rope_row = 8 * wave + (lane >> 3);
  const int sc_elem = 64 * wave + lane;
  const int sc_row = min(sc_elem / nblk, kTK - 1);
  const unsigned char* lat_src = (const unsigned char*)p.kv + group_row0 * kLat + (((lane & 31) ^ (lat_row & 7)) << 4);
  const unsigned char* rope_src = (const unsigned char*)p.rope + group_row0 * (kRope * 2) + (((lane & 7) ^ (rope_row & 7)) << 4);
  const unsigned char* sc_src = (const unsigned char*)p.kv_scale + (group_row0 * nblk + (unsigned)(sc_elem % nblk)) * 4;
  const unsigned lat_step = (unsigned)p.G * kLat, rope_step = (unsigned)p.G * (kRope * 2), sc_step = (unsigned)p.G * nblk * 4;
  auto dma16 = [&](const unsigned char* src, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "memory", "m0");
  };
  auto dma4 = [&](const unsigned char* src, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_addr), "v"(src) : "memory", "m0");
  };
  const unsigned smem_base = (unsigned)(size_t)(lds_void*)smem;                 // LDS byte address of the ring
  auto issue_tile = [&](int tau) {
    const unsigned slot = smem_base + (unsigned)(tau & (kRing - 1)) * kSlotBytes;
    const int* tk = keys + tau * kTK;
    int rows[6];
#pragma unroll
    for (int i = 0; i < 4; ++i) rows[i] = tk[8 * i + lat_row];
    rows[4] = tk[rope_row];
    rows[5] = scale_op ? tk[sc_row] : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      dma16(lat_src + (size_t)(unsigned)max(rows[i], 0) * lat_step, slot + (8 * i + 2 * wave) * kLat);
    dma16(rope_src + (size_t)(unsigned)max(rows[4], 0) * rope_step, slot + kLatBytes + 8 * wave * (kRope * 2));
    if (scale_op) {
      if (sc_elem < kTK * nblk)
        dma4(sc_src + (size_t)(unsigned)max(rows[5], 0) * sc_step, slot + kLatBytes + kRopeBytes + 256 * wave);
    }
  };
  auto wait_tiles_but_one = [&]() {               // everything but the most recently issued tile has landed
    if (scale_op) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  };

  // ---- score side state ----
  float m_run[2] = {-INFINITY, -INFINITY};        // base-2 running reference of heads n and 16+n
  float l_run[2] = {0.0f, 0.0f};                  // this lane's share of the denominators
  const float qk_scale = p.sm_scale * kLog2e;

  // S^T of tile tau for this wavefront's head group and sub-tiles
  auto qk_tile = [&](int tau, f32x4 (&st)[SPW][2]) {
    const unsigned char* slot = smem + (tau & (kRing - 1)) * kSlotBytes;
    const int m = lane & 15, kq = lane >> 4;
#pragma unroll
    for (int sj = 0; sj < SPW; ++sj) {
      const int r = 16 * (sub0 + sj) + m;         // tile row of this lane's K fragment
      const int r7 = r & 7;
      const unsigned char* lat0 = slot + r * kLat + ((kq ^ r7) << 4);
      const unsigned char* lat1 = slot + r * kLat + (((4 + kq) ^ r7) << 4);
      const unsigned char* rope = slot + kLatBytes + r * (kRope * 2);
      const float* scl = reinterpret_cast<const float*>(slot + kLatBytes + kRopeBytes) + r * nblk;
      // the power-of-two part of a key's scale goes into the conversion of its K fragment (this
      // lane's row r); the mantissa part multiplies the partial sums, which this lane holds for
      // keys 4*(lane/16) + i
      const float* sclc = reinterpret_cast<const float*>(slot + kLatBytes + kRopeBytes) + (16 * (sub0 + sj) + 4 * kq) * nblk;
      auto load_k = [&](int ks) {                 // raw bytes of the 64-channel step ks
        return *reinterpret_cast<const uint4*>(((ks & 1) ? lat1 : lat0) + 128 * (ks >> 1));
      };
      uint4 raw_a = load_k(0), raw_b = load_k(1);
      float pw[4];
      bool plain = true;                          // every scale of this row is a power of two
#pragma unroll
      for (int grp = 0; grp < 4; ++grp) {
        const float sc = scl[(grp * nblk) >> 2];
        pw[grp] = scale_pow2(sc);
        plain = plain && (pw[grp] == sc);
      }
      const bool all_plain = __ballot(!plain) == 0ull;     // (uniform) no mantissa factors in this sub-tile
      f32x4 tot0 = {0.f, 0.f, 0.f, 0.f}, tot1 = {0.f, 0.f, 0.f, 0.f};
      f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
      // software pipeline: step ks multiplies fragments converted during step ks-1 from bytes
      // read during step ks-2
      bf16x8 f0 = cvt8(raw_a.x, raw_a.y, pw[0]), f1 = cvt8(raw_a.z, raw_a.w, pw[0]);
      bf16x8 rf0 = f0, rf1 = f0;                  // rope fragments (read during the last two steps)
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        uint4 raw_c = raw_b;
        if (ks + 2 < 8) raw_c = load_k(ks + 2);
        else if (ks == 6) rf0 = *reinterpret_cast<const bf16x8*>(rope + ((kq ^ r7) << 4));
        else rf1 = *reinterpret_cast<const bf16x8*>(rope + (((4 + kq) ^ r7) << 4));
        bf16x8 n0 = f0, n1 = f1;
        if (ks + 1 < 8) {
          n0 = cvt8(raw_b.x, raw_b.y, pw[(ks + 1) >> 1]);
          n1 = cvt8(raw_b.z, raw_b.w, pw[(ks + 1) >> 1]);
        }
        mfma_s(a0, f0, qf[0][2 * ks]);
        mfma_s(a1, f0, qf[1][2 * ks]);
        mfma_s(a0, f1, qf[0][2 * ks + 1]);
        mfma_s(a1, f1, qf[1][2 * ks + 1]);
        // one LDS read, then MFMA and conversion pairs alternating
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
        }
        if ((ks & 1) && !all_plain) {             // end of a 128-channel block: apply its mantissa factors
          const int grp = ks >> 1;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float mant = scale_mant(sclc[i * nblk + ((grp * nblk) >> 2)]);
            tot0[i] += mant * a0[i];
            tot1[i] += mant * a1[i];
            a0[i] = 0.0f;
            a1[i] = 0.0f;
          }
        }
        f0 = n0; f1 = n1;
        raw_b = raw_c;
      }
      mfma_s(a0, rf0, qf[0][16]);
      mfma_s(a1, rf0, qf[1][16]);
      mfma_s(a0, rf1, qf[0][17]);
      mfma_s(a1, rf1, qf[1][17]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        tot0[i] += a0[i];
        tot1[i] += a1[i];
      }
      st[sj][0] = tot0;
      st[sj][1] = tot1;
    }
  };

  // ---- value side state: o[4*dvb + producer] = O^T[32 channels x 32 heads] ----
  f32x16 o[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) o[i][j] = 0.0f;
  const int pvar = (wave * nblk) >> 2;                         // scale block of channels 128*wave..
  int pv_off[4];                                               // transposing-read offsets per 32-channel block
  {
    const int t = lane & 15, half = (lane >> 4) & 1, kq2 = lane >> 5;
    const int r = 8 * kq2 + (t >> 1);                          // row within a 16-key step (r & 7 = t >> 1)
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb) {
      const int c = 8 * wave + 2 * dvb + half;                 // 16-byte chunk of the row
      pv_off[dvb] = r * kLat + ((c ^ (r & 7)) << 4) + 8 * (t & 1);
    }
  }
  // One pipeline stage: the value product of tile tv (8 steps of one V^T fragment and HG MFMAs)
  // with the softmax of tile ts cut into pieces that run in the shadow of those MFMAs.
  // do_s / do_v are uniform.
  auto stage = [&](int tv, bool do_v, int ts, bool do_s) {
    typedef __attribute__((ext_vector_type(2))) int i32x2;
    const int n = lane & 15, gq = lane >> 4;
    const unsigned char* vslot = smem + (tv & (kRing - 1)) * kSlotBytes;
    const unsigned char* sslot = smem + (ts & (kRing - 1)) * kSlotBytes;
    const int vpar = tv & 1, spar = ts & 1;
    f32x4 st[SPW][2];
    const unsigned char* pfrag = smem + G_::kPOff + vpar * G_::kPBytes + (pvar * G_::kSlots * 64 + lane) * 16;
    unsigned char* pdst = smem + G_::kPOff + spar * G_::kPBytes;
    float sv[SPW][2][4];
    float pr[2][4];
    float mx[2] = {-INFINITY, -INFINITY};
    // V's block scales of this lane's keys (4gq + i of each sub-tile) and their validity: read once, up front
    // (with two sub-tiles per wavefront there are no registers to spare: those read when needed)
    constexpr bool kHoist = SPW == 1;
    float vsc[SPW][4][nblk];
    int4 kvalid[SPW];
    auto read_scales = [&](int sj) {
      const float* scl = reinterpret_cast<const float*>(sslot + kLatBytes + kRopeBytes) + (16 * (sub0 + sj) + 4 * gq) * nblk;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (nblk == 4) {
          const float4 v4 = *reinterpret_cast<const float4*>(scl + 4 * i);
          vsc[sj][i][0] = v4.x; vsc[sj][i][1 % nblk] = v4.y; vsc[sj][i][2 % nblk] = v4.z; vsc[sj][i][3 % nblk] = v4.w;
        } else if (nblk == 2) {
          const float2 v2 = *reinterpret_cast<const float2*>(scl + 2 * i);
          vsc[sj][i][0] = v2.x; vsc[sj][i][1 % nblk] = v2.y;
        } else {
          vsc[sj][i][0] = scl[i];
        }
      }
    };
    if (do_v) {                                   // producers moved their reference: rescale (rare)
      const int4 fl = *reinterpret_cast<const int4*>(flagbuf + vpar * 4);
      if (__builtin_amdgcn_readfirstlane(fl.x | fl.y | fl.z | fl.w) != 0) {
        mfma_settle_acc(o);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          // one accumulator block at a time: the values pass through ordinary VGPRs
          const float fsc = facbuf[(vpar * 4 + (i & 3)) * 32 + (lane & 31)];
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int j = 0; j < 16; ++j) o[i][j] *= fsc;
          asm volatile("" : "+a"(o[i]));
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma_settle_acc(o);
      }
    }
    bf16x8 pb[HG];
    i32x2 vraw = {0, 0};
    auto load_v = [&](int i) {                    // V^T fragment of step i = (k-step i/4, channel block i%4)
      return __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) i32x2*)(vslot + 16 * (i >> 2) * kLat + pv_off[i & 3]));
    };
    auto load_p = [&](int kstep) {
#pragma unroll
      for (int hg = 0; hg < HG; ++hg) pb[hg] = *reinterpret_cast<const bf16x8*>(pfrag + (kstep * HG + hg) * 1024);
    };
    auto probs = [&](int sj) {                    // pr = exp2(score - reference), denominators
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          pr[hh][i] = (sv[sj][hh][i] == -INFINITY) ? 0.0f : fast_exp2(sv[sj][hh][i] - m_run[hh]);
          l_run[hh] += pr[hh][i];
        }
    };
    // P (x V's block scale) -> LDS in the B-operand layout of the 32x32x16 product: lane
    // (head, key/8) owns 16 bytes = 8 keys; this lane holds keys 4gq..4gq+3 of sub-tile sj
    auto write_p = [&](int sj, int v0, int v1) {
      const int slot_id = (sub0 + sj) * HG + hgq;
#pragma unroll
      for (int v = v0; v < v1; ++v) {
        if (v >= nblk) break;
        float sc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) sc[i] = vsc[sj][i][v % nblk];
        unsigned char* dst = pdst + ((v * G_::kSlots + slot_id) * 64 + (gq >> 1) * 32) * 16 + (gq & 1) * 8;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          const uint2 w = make_uint2(pack_bf16(pr[hh][0] * sc[0], pr[hh][1] * sc[1]),
                                     pack_bf16(pr[hh][2] * sc[2], pr[hh][3] * sc[3]));
          *reinterpret_cast<uint2*>(dst + (hh * 16 + n) * 16) = w;
        }
      }
    };
    auto softmax_piece = [&](int i) {
      if (i == 0) {                               // mask, scale, local maxima
#pragma unroll
        for (int sj = 0; sj < SPW; ++sj) {
          const int4 kk = kHoist ? kvalid[sj] : *reinterpret_cast<const int4*>(keys + ts * kTK + 16 * (sub0 + sj) + 4 * gq);
          const bool ok[4] = {kk.x >= 0, kk.y >= 0, kk.z >= 0, kk.w >= 0};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            sv[sj][0][e] = ok[e] ? st[sj][0][e] * qk_scale : -INFINITY;
            sv[sj][1][e] = ok[e] ? st[sj][1][e] * qk_scale : -INFINITY;
            mx[0] = fmaxf(mx[0], sv[sj][0][e]);
            mx[1] = fmaxf(mx[1], sv[sj][1][e]);
          }
        }
      } else if (i == 1) {                        // maxima across the four key quarters; lazy reference
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          mx[hh] = fmaxf(mx[hh], xor16(mx[hh]));
          mx[hh] = fmaxf(mx[hh], xor32(mx[hh]));
        }
        const bool grow = (mx[0] > m_run[0] + kLazy) || (mx[1] > m_run[1] + kLazy);
        const bool any_grow = __ballot(grow) != 0ull;
        // accumulators of a head whose reference was -inf are still zero: nothing to rescale
        const bool rescale = (mx[0] > m_run[0] + kLazy && m_run[0] != -INFINITY) || (mx[1] > m_run[1] + kLazy && m_run[1] != -INFINITY);
        const bool any_rescale = __ballot(rescale) != 0ull;
        if (any_grow) {                           // consumers rescale their accumulators by fac first
          float fac[2];
#pragma unroll
          for (int hh = 0; hh < 2; ++hh) {
            const float m_new = (mx[hh] > m_run[hh] + kLazy) ? mx[hh] : m_run[hh];
            fac[hh] = (m_run[hh] == -INFINITY) ? 1.0f : exp2f(m_run[hh] - m_new);
            l_run[hh] *= fac[hh];
            m_run[hh] = m_new;
          }
          if (any_rescale && lane < 16) {
            facbuf[(spar * 4 + wave) * 32 + n] = fac[0];
            facbuf[(spar * 4 + wave) * 32 + 16 + n] = fac[1];
          }
        }
        if (!any_rescale && lane < 32) facbuf[(spar * 4 + wave) * 32 + lane] = 1.0f;
        if (lane == 0) flagbuf[spar * 4 + wave] = any_rescale ? 1 : 0;
      } else if (i == 2) {
        if (!kHoist) read_scales(0);
        probs(0);
      } else if (i == 3) {
        write_p(0, 0, 2);
      } else if (i == 4) {
        write_p(0, 2, 4);
      } else if (SPW == 2) {
        if (i == 5) { read_scales(1); probs(1); }
        else if (i == 6) write_p(1, 0, 2);
        else write_p(1, 2, 4);
      }
    };
    if (do_s) qk_tile(ts, st);
    __builtin_amdgcn_sched_barrier(0);
    if (do_s && kHoist) {
#pragma unroll
      for (int sj = 0; sj < SPW; ++sj) {
        kvalid[sj] = *reinterpret_cast<const int4*>(keys + ts * kTK + 16 * (sub0 + sj) + 4 * gq);
        read_scales(sj);
      }
    }
    if (do_v) {
      load_p(0);
      vraw = load_v(0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_barrier(0);
      i32x2 vnext = vraw;
      if (do_v && i < 7) vnext = load_v(i + 1);
      if (do_s) softmax_piece(i);
      if (do_v) {
        const bf16x8 a = cvt8((unsigned)vraw[0], (unsigned)vraw[1], 1.0f);
        const int kstep = i >> 2, dvb = i & 3;
#pragma unroll
        for (int hg = 0; hg < HG; ++hg) {
          const int prod = HG == 4 ? hg : hg + 2 * kstep;      // the wavefront that produced this P
          mfma_pv(o[4 * dvb + prod], a, pb[hg]);
        }
        if (i == 3) load_p(1);
      }
      vraw = vnext;
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- pipeline ----
  issue_tile(0);
  issue_tile(1);
  issue_tile(2);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  stage(0, false, 0, true);
  for (int t = 0; t < n_tiles; ++t) {
    wait_tiles_but_one();                         // tile t+1 (issued two iterations ago) has landed
    __syncthreads();                              // ... for every wavefront; P(t) is complete; PV(t-1) is done
    issue_tile(t + 3);                            // into the slot of tile t-1
    __builtin_amdgcn_sched_barrier(0);
    stage(t, true, t + 1, t + 1 < n_tiles);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the prefetches past the end
  mfma_settle_acc(o);

  // ---- epilogue ----
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {                // a head's denominator is spread over lanes n, n+16, n+32, n+48
    l_run[hh] += xor16(l_run[hh]);
    l_run[hh] += xor32(l_run[hh]);
  }
  if (lane < 16) {
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      stats[(wave * 32 + hh * 16 + lane) * 2 + 0] = m_run[hh];
      stats[(wave * 32 + hh * 16 + lane) * 2 + 1] = l_run[hh];
    }
  }
  __syncthreads();                                // statistics are visible; the ring is free

  const int hd = lane & 31, gq2 = lane >> 5;
  const bool direct = p.num_splits == 1;
  float* xbuf = reinterpret_cast<float*>(smem) + wave * 32 * kXPitch;     // private to this wavefront
  const size_t q_index = bs;
  // key-split partials: one block per (query, KV group, head chunk, split)
  const size_t part_block = (size_t)(((long long)bs * p.G + g) * chunks + chunk) * p.num_splits + split;
  const size_t part_blocks_total = (size_t)p.B * p.S * p.G * chunks * p.num_splits;
#pragma unroll
  for (int hg = 0; hg < HG; ++hg) {
    float m_all, l_all;
    if (HG == 4) {
      m_all = stats[(hg * 32 + hd) * 2];
      l_all = stats[(hg * 32 + hd) * 2 + 1];
    } else {                                      // two producers per head group: hg and hg + 2
      const float ma = stats[(hg * 32 + hd) * 2], la = stats[(hg * 32 + hd) * 2 + 1];
      const float mb = stats[((hg + 2) * 32 + hd) * 2], lb = stats[((hg + 2) * 32 + hd) * 2 + 1];
      m_all = fmaxf(ma, mb);
      const float fa = (ma == -INFINITY) ? 0.0f : exp2f(ma - m_all);
      const float fb = (mb == -INFINITY) ? 0.0f : exp2f(mb - m_all);
      l_all = la * fa + lb * fb;
#pragma unroll
      for (int dvb = 0; dvb < 4; ++dvb) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 16; ++j) o[4 * dvb + hg][j] = o[4 * dvb + hg][j] * fa + o[4 * dvb + hg + 2][j] * fb;
        asm volatile("" : "+a"(o[4 * dvb + hg]));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    const int h_local = 32 * hg + hd;
    float out_scale = 1.0f, lse_val = 0.0f;
    if (direct) {
      float m_fin = m_all, l_fin = l_all;
      if (p.sinks && h_local < heads_here) {
        const float sk = p.sinks[head0 + h_local] * kLog2e;
        const float m2 = fmaxf(m_fin, sk);
        const float keep = (m_fin == -INFINITY) ? 0.0f : exp2f(m_fin - m2);
        l_fin = l_fin * keep + exp2f(sk - m2);
        out_scale = keep;
        m_fin = m2;
      }
      if (l_fin > 0.0f) {
        out_scale = out_scale / l_fin;
        lse_val = (m_fin + log2f(l_fin)) * kLn2;
      } else {
        out_scale = 0.0f;
      }
    }
    if (!direct) {
      // key split: the unnormalised accumulators leave exactly as the lanes hold them (1 KiB per
      // store instruction); the combine kernel knows the layout and does the transposition
      // (bf16: the values are relative to the split's own maximum, so their range is that of
      // the output times the split's probability mass; the rounding is 2^-9 relative)
      unsigned short* blk = (unsigned short*)p.workspace + part_block * (size_t)(HG * kPartFloats) +
                            ((size_t)((wave * HG + hg) * 16) * 64 + lane) * 4;
#pragma unroll
      for (int dvb = 0; dvb < 4; ++dvb) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const f32x16& acc = o[4 * dvb + hg];
          *reinterpret_cast<uint2*>(blk + (size_t)(dvb * 4 + j) * 256) =
              make_uint2(pack_bf16(acc[4 * j], acc[4 * j + 1]), pack_bf16(acc[4 * j + 2], acc[4 * j + 3]));
        }
      }
      if (wave == 0 && lane < 32) {
        float* ml = (float*)((unsigned short*)p.workspace + part_blocks_total * (size_t)(HG * kPartFloats)) + (part_block * (32 * HG) + h_local) * 2;
        ml[0] = m_all;
        ml[1] = l_all;
      }
      continue;
    }
    // transpose through LDS: lane (head hd, gq2) holds channels 32dvb + 8j + 4gq2 + (0..3) in o[.][4j..4j+3]
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x16& acc = o[4 * dvb + hg];
        const float4 v = make_float4(acc[4 * j] * out_scale, acc[4 * j + 1] * out_scale, acc[4 * j + 2] * out_scale,
                                     acc[4 * j + 3] * out_scale);
        *reinterpret_cast<float4*>(xbuf + hd * kXPitch + 32 * dvb + 8 * j + 4 * gq2) = v;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // rows of 128 channels leave coalesced: 32 lanes x 4 channels, two heads per step
#pragma unroll 4
    for (int it = 0; it < 16; ++it) {
      const int row = 2 * it + gq2;
      const int hl = 32 * hg + row;
      if (hl >= heads_here) continue;
      const float4 v = *reinterpret_cast<const float4*>(xbuf + row * kXPitch + hd * 4);
      const size_t off = (q_index * p.H + head0 + hl) * (size_t)kLat + 128 * wave + hd * 4;
      if (p.out_dtype == CPPMEGA_MI355_F32) {
        *reinterpret_cast<float4*>((float*)p.out + off) = v;
      } else if (p.out_dtype == CPPMEGA_MI355_BF16) {
        *reinterpret_cast<uint2*>((unsigned short*)p.out + off) = make_uint2(pack_bf16(v.x, v.y), pack_bf16(v.z, v.w));
      } else {
        unsigned short* dst = (unsigned short*)p.out + off;
        dst[0] = f32_to_f16_bits(v.x); dst[1] = f32_to_f16_bits(v.y);
        dst[2] = f32_to_f16_bits(v.z); dst[3] = f32_to_f16_bits(v.w);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (wave == 0 && lane < 32 && h_local < heads_here && p.lse) p.lse[q_index * p.H + head0 + h_local] = lse_val;
  }
}

// Merges the key splits written by sparse_mla_latent_kernel.  A partial block holds, per
// (wavefront w = 128 value channels, head group hg), 16 rows of 64 lanes x float4 exactly as the
// accumulator registers held them: row 4*dvb + j, lane (head hd = lane%32, half = lane/32), element e
// is channel 128w + 32dvb + 8j + 4half + e of head 32hg + hd.  One workgroup per (query, KV group,
// head chunk, w, hg): coalesced 1 KiB row reads, weights per head, transposition through LDS,
// coalesced output rows.
template <int HG>
__global__ __launch_bounds__(256) void sparse_mla_latent_combine_kernel(const MlaParams p) {
  __shared__ float x[32][kXPitch];
  const int tid = (int)threadIdx.x, lane = tid & 63, r4 = tid >> 6;
  const int chunks = (p.heads_per_group + 32 * HG - 1) / (32 * HG);
  const int w = (int)blockIdx.y / HG, hg = (int)blockIdx.y % HG;
  const size_t unit = blockIdx.x;                              // (b*S + s, g, chunk)
  const int chunk = (int)(unit % chunks);
  const size_t qg = unit / chunks;
  const int g = (int)(qg % p.G);
  const size_t bs = qg / p.G;
  const int head0 = g * p.heads_per_group + chunk * 32 * HG;
  const int heads_here = min(32 * HG, p.heads_per_group - chunk * 32 * HG);
  const int hd = lane & 31, half = lane >> 5;
  const int h_local = 32 * hg + hd;
  const size_t blocks_total = (size_t)p.B * p.S * p.G * chunks * p.num_splits;
  const float* ml = (const float*)((const unsigned short*)p.workspace + blocks_total * (size_t)(HG * kPartFloats));
  const size_t block0 = unit * p.num_splits;
  // all (max, sum) pairs first, then the partial rows four splits at a time, so that the loads
  // of a group are in flight together (the split count is at most 16)
  float ms[16], ls[16];
  float m_all = -INFINITY;
#pragma unroll
  for (int s = 0; s < 16; ++s) {
    ms[s] = -INFINITY;
    ls[s] = 0.0f;
    if (s < p.num_splits) {
      const float2 t = *reinterpret_cast<const float2*>(ml + ((block0 + s) * (32 * HG) + h_local) * 2);
      ms[s] = t.x;
      ls[s] = t.y;
    }
    m_all = fmaxf(m_all, ms[s]);
  }
  float m_fin = m_all, l_fin = 0.0f;
  if (p.sinks && h_local < heads_here) {
    const float sk = p.sinks[head0 + h_local] * kLog2e;
    m_fin = fmaxf(m_all, sk);
    l_fin = exp2f(sk - m_fin);
  }
  float4 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  const unsigned short* src0 = (const unsigned short*)p.workspace + block0 * (size_t)(HG * kPartFloats) +
                               ((size_t)((w * HG + hg) * 16 + 4 * r4) * 64 + lane) * 4;
#pragma unroll
  for (int s0 = 0; s0 < 16; s0 += 4) {
    if (s0 >= p.num_splits) break;                            // (uniform)
    uint2 raw[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = min(s0 + u, p.num_splits - 1);             // a repeated last split gets weight 0
#pragma unroll
      for (int i = 0; i < 4; ++i)
        raw[u][i] = *reinterpret_cast<const uint2*>(src0 + (size_t)s * (HG * kPartFloats) + (size_t)i * 256);
    }
    float4 v[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[u][i] = make_float4(__uint_as_float(raw[u][i].x << 16), __uint_as_float(raw[u][i].x & 0xffff0000u),
                              __uint_as_float(raw[u][i].y << 16), __uint_as_float(raw[u][i].y & 0xffff0000u));
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float f = (s0 + u < p.num_splits && ms[s0 + u] != -INFINITY) ? exp2f(ms[s0 + u] - m_fin) : 0.0f;
      l_fin += ls[s0 + u] * f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i].x += v[u][i].x * f; acc[i].y += v[u][i].y * f; acc[i].z += v[u][i].z * f; acc[i].w += v[u][i].w * f;
      }
    }
  }
  const float inv = l_fin > 0.0f ? 1.0f / l_fin : 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {                                // row 4*r4 + i = (dvb = r4, j = i)
    *reinterpret_cast<float4*>(&x[hd][32 * r4 + 8 * i + 4 * half]) =
        make_float4(acc[i].x * inv, acc[i].y * inv, acc[i].z * inv, acc[i].w * inv);
  }
  if (p.lse && w == 0 && r4 == 0 && half == 0 && h_local < heads_here)
    p.lse[bs * p.H + head0 + h_local] = l_fin > 0.0f ? (m_fin + log2f(l_fin)) * kLn2 : 0.0f;
  __syncthreads();
  // thread -> head tid/8, 16 channels (tid%8)*16
  const int row = tid >> 3, c0 = (tid & 7) * 16;
  if (32 * hg + row < heads_here) {
    const size_t off = (bs * p.H + head0 + 32 * hg + row) * (size_t)kLat + 128 * w + c0;
    float v[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float4 t = *reinterpret_cast<const float4*>(&x[row][c0 + 4 * i]);
      v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
    }
    if (p.out_dtype == CPPMEGA_MI355_BF16) {
      uint4 a, b;
      a = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
      b = make_uint4(pack_bf16(v[8], v[9]), pack_bf16(v[10], v[11]), pack_bf16(v[12], v[13]), pack_bf16(v[14], v[15]));
      *reinterpret_cast<uint4*>((unsigned short*)p.out + off) = a;
      *reinterpret_cast<uint4*>((unsigned short*)p.out + off + 8) = b;
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) store_as(p.out, off + i, p.out_dtype, v[i]);
    }
  }
}

}  // namespace

bool sparse_mla_latent_supported(const MlaParams& p) {
  if (p.q_dtype != CPPMEGA_MI355_BF16 || p.q_scale_kind != CPPMEGA_MI355_SCALE_NONE) return false;
  if (p.d_qk != kDqk || p.d_v != kLat || p.d_kv != kLat) return false;
  if (p.kv_dtype != CPPMEGA_MI355_E4M3) return false;
  if (p.rope_dim != kRope || p.rope_dtype != CPPMEGA_MI355_BF16) return false;
  if (p.kv_scale_kind == CPPMEGA_MI355_SCALE_F32_BLOCK) {
    if (p.kv_scale_block != 128 && p.kv_scale_block != 256 && p.kv_scale_block != 512) return false;
  } else if (p.kv_scale_kind != CPPMEGA_MI355_SCALE_PER_TOKEN && p.kv_scale_kind != CPPMEGA_MI355_SCALE_NONE) {
    return false;
  }
  if (p.heads_per_group <= 32) return false;      // a single 32-head group gains nothing from sharing
  if (p.topk < 1 || (size_t)p.B * p.S == 0) return false;
  if (((uintptr_t)p.q | (uintptr_t)p.kv | (uintptr_t)p.rope) & 15) return false;
  if (p.kv_scale && ((uintptr_t)p.kv_scale & 3)) return false;
  if ((unsigned long long)p.B * p.Skv * p.G >= 0x7fffffffull) return false;   // cache rows are counted in 32 bits
  return true;
}

// heads per workgroup (in units of 32) and the key-split factor
static int latent_splits(const MlaParams& p, int hg, long long* wgs) {
  const int chunks = (p.heads_per_group + 32 * hg - 1) / (32 * hg);
  const long long base = (long long)p.B * p.S * p.G * chunks;
  int splits = 1;
  while (base * splits < 256 && p.topk / (splits * 2) >= 4 * kTK && splits < 16) splits *= 2;
  while ((p.topk + splits - 1) / splits > kMaxKeys) splits *= 2;
  *wgs = base * splits;
  return splits;
}

void sparse_mla_latent_plan(MlaParams& p) {
  // 128 heads per workgroup reuse every gathered row the most; 64 only when that is what it takes
  // to cover the device (few queries, short key lists)
  int hg = p.heads_per_group > 64 ? 4 : 2;
  long long wgs4 = 0, wgs2 = 0;
  if (hg == 4) {
    latent_splits(p, 4, &wgs4);
    latent_splits(p, 2, &wgs2);
    if (wgs4 < 256 && wgs2 > wgs4) hg = 2;
  }
  if (const char* env = getenv("CPPMEGA_MI355_MLA_HEADS_PER_WG")) {
    const int v = atoi(env);
    if (v == 64) hg = 2;
    if (v == 128) hg = 4;
  }
  p.heads_per_wg = 32 * hg;
  long long wgs = 0;
  const int splits = latent_splits(p, hg, &wgs);
  const int tiles = (p.topk + kTK - 1) / kTK;
  const int tiles_per_split = (tiles + splits - 1) / splits;
  p.num_splits = splits;
  p.keys_per_split = tiles_per_split * kTK;
}

int sparse_mla_latent_launch(const MlaParams& p, hipStream_t stream) {
  const int hg = p.heads_per_wg / 32;
  const int chunks = (p.heads_per_group + 32 * hg - 1) / (32 * hg);
  const long long wgs = (long long)p.B * p.S * p.G * p.num_splits * chunks;
  if (wgs > 0x7fffffffll || p.keys_per_split > kMaxKeys) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse MLA: launch too large");
  const dim3 grid((unsigned)wgs), block(256);
  const int nblk = p.kv_scale_kind == CPPMEGA_MI355_SCALE_F32_BLOCK ? kLat / p.kv_scale_block : 1;
#define CM_LAUNCH_LATENT(HG_, NB_)                                                                                      \
  do {                                                                                                                  \
    CM_HIP_CHECK(hipFuncSetAttribute((const void*)sparse_mla_latent_kernel<HG_, NB_>,                                    \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, Geo<HG_>::kSmem));                      \
    hipLaunchKernelGGL((sparse_mla_latent_kernel<HG_, NB_>), grid, block, Geo<HG_>::kSmem, stream, p);                   \
  } while (0)
  if (hg == 4) {
    if (nblk == 4) CM_LAUNCH_LATENT(4, 4);
    else if (nblk == 2) CM_LAUNCH_LATENT(4, 2);
    else CM_LAUNCH_LATENT(4, 1);
  } else {
    if (nblk == 4) CM_LAUNCH_LATENT(2, 4);
    else if (nblk == 2) CM_LAUNCH_LATENT(2, 2);
    else CM_LAUNCH_LATENT(2, 1);
  }
#undef CM_LAUNCH_LATENT
  CM_HIP_CHECK(hipGetLastError());
  if (p.num_splits > 1) {
    const dim3 cgrid((unsigned)((size_t)p.B * p.S * p.G * chunks), (unsigned)(4 * hg));
    if (hg == 4) hipLaunchKernelGGL(sparse_mla_latent_combine_kernel<4>, cgrid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(sparse_mla_latent_combine_kernel<2>, cgrid, dim3(256), 0, stream, p);
  }
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

// the combine step alone (partials in the layout of hg 32-head groups per workgroup)
int sparse_mla_latent_combine_launch(const MlaParams& p, int hg, hipStream_t stream) {
  const int chunks = (p.heads_per_group + 32 * hg - 1) / (32 * hg);
  const dim3 cgrid((unsigned)((size_t)p.B * p.S * p.G * chunks), (unsigned)(4 * hg));
  if (hg == 4) hipLaunchKernelGGL(sparse_mla_latent_combine_kernel<4>, cgrid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(sparse_mla_latent_combine_kernel<2>, cgrid, dim3(256), 0, stream, p);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

size_t sparse_mla_latent_workspace_bytes(const MlaParams& p) {
  if (p.num_splits <= 1) return 0;
  const int hg = p.heads_per_wg / 32;
  const int chunks = (p.heads_per_group + 32 * hg - 1) / (32 * hg);
  const size_t blocks = (size_t)p.B * p.S * p.G * chunks * p.num_splits;
  return blocks * ((size_t)hg * kPartFloats * sizeof(unsigned short) + 32 * hg * 2 * sizeof(float));
}

}  // namespace cm
