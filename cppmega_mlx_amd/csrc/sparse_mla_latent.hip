// Sparse MLA forward over an FP8 latent KV cache on the matrix cores (gfx950), with the
// wavefronts of a workgroup split into score producers and value consumers.
//
// Shapes served: bf16 queries of 576 = 512 latent + 64 rope channels, d_v = 512, keys as e4m3
// latent [512] with fp32 scales (per 128 / 256 / 512 channels, per row, or none) plus a bf16
// rope tail [64]; more than 32 heads per KV group.
//
// Workgroup = (query, KV group, chunk of 64 heads, key split), 8 wavefronts, key tiles of 32
// rows in a ring of five LDS slots filled by the load unit (global_load_lds) three tiles ahead.
// Two wavefronts share a SIMD: one producer and one consumer, so the matrix passes of one run
// under the vector instructions of the other.
//
//   producers (wavefronts 0..3): producer p owns heads 16p..16p+15 of the chunk.
//     S^T = K.Q^T on v_mfma_scale_f32_16x16x128_f8f6f4: the key bytes are the A operand as they
//     lie in the tile (no conversion instructions, operand exponent 2^0); every 128-channel block is
//     accumulated from zero and enters the score times its keys' fp32 block scales.  Q^T is
//     split once per workgroup into two e4m3 planes hi + lo (hi + lo = the bf16 value, one
//     exponent per head and 128 channels), kept in registers.  The rope tail is a bf16 product.
//     Softmax in base 2 with a lazily moved private running maximum per head; P goes to LDS as
//     bf16 in the B-operand layout of the value product, one plane per scale block: plane b is P
//     times the keys' scales of block b (one fp32 product, rounded once).
//   consumers (wavefronts 4..7): consumer c owns value channels 128c..128c+127 (= scale block c
//     when there are four) for all 64 heads: O^T += V^T.P_c^T on v_mfma_f32_32x32x16_bf16, V^T
//     fragments by transposing LDS reads of the raw tile, converted unscaled (exactly), P_c the
//     plane of its block.  They also issue the row loads.
//   pipeline  iteration t: barrier; producers: scores and P of tile t+1; consumers: issue tile
//             t+4, value product of tile t.  One barrier per tile.
//
// Key splits write their accumulators (rounded to bf16) to the workspace as the lanes hold them
// plus (max, sum) per head; sparse_mla_latent_combine_kernel merges them and does the transposition
// to [head][channel] that the single-split path does in LDS.

#include <type_traits>

#include "sparse_mla_common.h"
#include "mfma_util.h"

namespace cm {

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr int kLat = 512;
constexpr int kRope = 64;
constexpr int kDqk = kLat + kRope;
constexpr int kTK = 32;                         // keys per tile
constexpr int kRing = 5;                        // tile slots
constexpr int kAhead = kRing - 1;               // tiles issued ahead of the value product
// A tile slot holds the rows in matrix-operand order.  Latent: for sub-tile sj (16 keys) and
// 128-channel block blk, two planes j of 64 lanes x 16 bytes: lane (key n = lane % 16, kg = lane / 16)
// of plane j holds channels 128 blk + 32 kg + 16 j .. + 15 of key 16 sj + n.  A plane is what one
// load instruction writes (the load unit stores lane after lane) and what one 16-byte-per-lane
// LDS read of a K operand fetches, contiguously.  Plane 1 starts 128 bytes after the end of plane
// 0, so that the two neighbouring chunks a V^T read takes from eight rows fall on different banks.
// Rope: for sub-tile sj and 32-channel step s one plane: lane (n, kq) holds channels 32 s + 8 kq .. + 7.
constexpr int kPlane = 1024 + 128;              // bytes from plane 0 to plane 1 of a pair
constexpr int kPair = 2 * kPlane;               // one (sub-tile, block)
constexpr int kLatBytes = 8 * kPair;            // 18432
constexpr int kRopeBytes = 4 * 1024;            // [sj][s] planes
constexpr int kScaleBytes = kTK * 4 * 4;        // up to four fp32 scales per row: [row][block]
constexpr int kSlotBytes = kLatBytes + kRopeBytes + kScaleBytes;   // 23552
constexpr int kRingBytes = kRing * kSlotBytes;  // 104960
constexpr int kMaxKeys = 2048;                  // keys of one split (their rows are staged in LDS)
constexpr int kKeyInts = kMaxKeys + kTK;
constexpr int kHeadsWg = 64;
constexpr int kXPitch = 132;                    // floats per head row of the output transpose (128 + 4)
constexpr int kPartFloats = 4 * 16 * 64 * 4;    // partial values of one 32-head group: [4 consumers][8 row pairs][64 lanes][8]
constexpr float kLazy = 8.0f;                   // move a running maximum only when it grows by > 2^8

constexpr int kPPlane = 2 * 2 * 1024;           // one plane of P of one tile: [k-step][head block][64 lanes x 16 B]
constexpr int kPBytes = 4 * kPPlane;            // up to four planes per tile: P times V's scale of block b
constexpr int kPOff = kRingBytes;
constexpr int kFacOff = kPOff + 2 * kPBytes;        // [parity][4 producers][16 heads] fp32
constexpr int kFlagOff = kFacOff + 2 * 4 * 16 * 4;  // [parity][4 producers] int
constexpr int kStatOff = kFlagOff + 2 * 4 * 4;      // [4 producers][16 heads][2] fp32
constexpr int kValidOff = kStatOff + 4 * 16 * 2 * 4;  // [tile] int: every key of the tile is valid
constexpr int kKeyOff = kValidOff + (kMaxKeys / kTK) * 4;
constexpr int kSmem = kKeyOff + kKeyInts * 4;
static_assert(kSmem <= 160 * 1024, "LDS budget");
static_assert(4 * 32 * kXPitch * 4 <= kRingBytes, "the output transpose reuses the ring");

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ bf16x8 cvt8(unsigned w0, unsigned w1) {
  const unsigned o0 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w0, 1.0f, false));
  const unsigned o1 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w0, 1.0f, true));
  const unsigned o2 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w1, 1.0f, false));
  const unsigned o3 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w1, 1.0f, true));
  return __builtin_bit_cast(bf16x8, make_uint4(o0, o1, o2, o3));
}

// 16 x 16 x 128 over e4m3 bytes, operands scaled by 2^(byte - 127): the byte is byte SEL of `a_exp`
// for A and of `b_exp` for B, and must be the same in the four lanes of a row (l, l+16, ..).
template <int SEL>
__device__ __forceinline__ void mfma_s8(f32x4& acc, const i32x8& a, const i32x8& b, int a_exp, int b_exp) {
  acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc, 0, 0, SEL, a_exp, SEL, b_exp);
}
__device__ __forceinline__ void mfma_s(f32x4& acc, const bf16x8& a, const bf16x8& b) {
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ void mfma_o(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}

// 32 bf16 (four 16-byte pieces, channel order) of each lane -> e4m3 hi + e4m3 lo with hi + lo = x,
// both in units of 2^(e - 127); returns e, common to lanes l, l^16, l^32, l^48 (one head's 128
// channels).  hi carries the upper four significant bits of a bf16 value and lo the lower four, so
// the pair is exact for every element within ~2^-14 of the largest of the 128 and off by less
// than 2^-18 of that largest one otherwise.
__device__ __forceinline__ int split_q32(const uint4 (&x)[4], i32x8& hi, i32x8& lo) {
  u16x2 top = {0, 0};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const unsigned w[4] = {x[j].x, x[j].y, x[j].z, x[j].w};
#pragma unroll
    for (int d = 0; d < 4; ++d) top = __builtin_elementwise_max(top, __builtin_bit_cast(u16x2, w[d] & 0x7fff7fffu));
  }
  int amax_bits = max((int)top[0], (int)top[1]);             // bf16 bits of the largest magnitude
  amax_bits = max(amax_bits, __float_as_int(xor16(__int_as_float(amax_bits))));
  amax_bits = max(amax_bits, __float_as_int(xor32(__int_as_float(amax_bits))));
  const int e = max((amax_bits >> 7) - 7, 1);                 // |x| / 2^(e-127) < 256
  const float unit = __uint_as_float((unsigned)e << 23);
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
                                                         __uint_as_float(w0 & 0xffff0000u) - d0[1], unit, false);
      l = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(l, __uint_as_float(w1 << 16) - d1[0],
                                                   __uint_as_float(w1 & 0xffff0000u) - d1[1], unit, true);
      hi[2 * j + d] = (int)hw;
      lo[2 * j + d] = __builtin_bit_cast(int, l);
    }
  }
  return e;
}

// v_max_f32 as it is (fmaxf first passes every operand through a canonicalising max with itself).
// Only for operands that ordinary vector instructions produced: never for matrix results, whose
// read-after-write wait states the compiler pads only for instructions it can see.
__device__ __forceinline__ float vmax(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

__device__ __forceinline__ float vmax3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// maximum over lanes l, l^16, l^32, l^48 (every lane gets it): a row swap leaves each value next
// to its partner's
__device__ __forceinline__ float max_rows(float v) {
  unsigned u = __float_as_uint(v);
  u32x2 r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = vmax(__uint_as_float(r[0]), __uint_as_float(r[1]));
  u = __float_as_uint(v);
  r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return vmax(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// NBLK: fp32 scales per key row (1, 2 or 4)
template <int NBLK>
__global__ __launch_bounds__(512, 2) void sparse_mla_latent_kernel(const MlaParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = (int)threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave < 4;
  const int role = wave & 3;                    // producer p / consumer c
  constexpr int nblk = NBLK;

  // ---- which (query, KV group, head chunk, split).  Workgroup ids that are equal modulo 8 run on
  //      the same XCD and share its L2: every workgroup of one (query, KV group) gets such ids, so
  //      the gathered key rows are fetched from HBM once for both head chunks and the query rows
  //      once for all key splits ----
  // (all of it in 32-bit unsigned arithmetic - the launcher checks that the grid fits: the same
  // decoding with 64-bit divisions was a dependent chain of ~1000 scalar instructions in front of
  // the first load of every workgroup)
  const unsigned chunks = (unsigned)(p.heads_per_group + kHeadsWg - 1) / (unsigned)kHeadsWg;
  const unsigned per_q = (unsigned)p.num_splits * chunks;      // workgroups of one (query, KV group)
  const unsigned nq = (unsigned)p.B * (unsigned)p.S * (unsigned)p.G;
  const unsigned nq8 = nq & ~7u;
  unsigned qg;
  int chunk, split;
  {
    // (several queries per sequence: the last ones first - under a causal selection they hold the
    // longest key lists, and the short ones then fill the end of the launch)
    const unsigned id = p.S > 1 ? gridDim.x - 1u - blockIdx.x : blockIdx.x;
    unsigned r;
    if (id < nq8 * per_q) {
      const unsigned slot = id >> 3, sq = slot / per_q;
      qg = sq * 8u + (id & 7u);
      r = slot - sq * per_q;
    } else {
      const unsigned rest = id - nq8 * per_q, rq = rest / per_q;
      qg = nq8 + rq;
      r = rest - rq * per_q;
    }
    split = (int)(r / chunks);
    chunk = (int)(r - (unsigned)split * chunks);
  }
  const unsigned bs32 = qg / (unsigned)p.G;       // b*S + s
  const int g = (int)(qg - bs32 * (unsigned)p.G);
  const size_t bs = bs32;
  const int b = (int)(bs32 / (unsigned)p.S);
  const int head0 = g * p.heads_per_group + chunk * kHeadsWg;
  const int heads_here = min(kHeadsWg, p.heads_per_group - chunk * kHeadsWg);
  const size_t idx_base = (bs * p.G + g) * (size_t)p.topk;
  const int key_begin = split * p.keys_per_split;
  const int key_end = min(p.topk, key_begin + p.keys_per_split);
  const int n_keys = max(0, key_end - key_begin);
  const int list_tiles = (n_keys + kTK - 1) / kTK;

  const bool has_scale = p.kv_scale_kind != CPPMEGA_MI355_SCALE_NONE;   // otherwise the scale area holds ones

  int* keys = reinterpret_cast<int*>(smem + kKeyOff);
  float* facbuf = reinterpret_cast<float*>(smem + kFacOff);
  int* flagbuf = reinterpret_cast<int*>(smem + kFlagOff);
  float* stats = reinterpret_cast<float*>(smem + kStatOff);
  int* tvalid = reinterpret_cast<int*>(smem + kValidOff);

  if (!has_scale) {                               // no scales in memory: every slot's scale area is 1.0 for good
    for (int i = tid; i < kRing * kTK; i += 512)
      reinterpret_cast<float*>(smem + (i / kTK) * kSlotBytes + kLatBytes + kRopeBytes)[i % kTK] = 1.0f;
  }
  // ---- cache rows of this split's keys -> LDS (-1 = skipped) ----
  int* last_valid = reinterpret_cast<int*>(stats);          // [8], one per wavefront (the statistics come much later)
  // thread t takes list entries t, t + 512, ..: every index word is requested before the first one
  // is looked at (one memory round trip), unconditionally, with positions clamped to the list.
  // The producers put their query-row requests between the two halves: the load unit then
  // moves the 74 KB of query rows while the index words are on their way, instead of in front of
  // the first key tile.
  constexpr int kRounds = kMaxKeys / 512;
  const bool wide = p.index_dtype == CPPMEGA_MI355_I64;
  const float sm_scale = mla_sm_scale(p);        // (a uniform load when the scale lives in device memory)
  int idx_lo[kRounds], idx_hi[kRounds];
  {
    const int* words = (const int*)p.indices;
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
      idx_lo[r] = 0; idx_hi[r] = 0;
      if (r * 512 < list_tiles * kTK) {           // (uniform)
        const size_t at = idx_base + (size_t)min(key_begin + tid + 512 * r, p.topk - 1);
        const size_t w0 = wide ? 2 * at : at;
        idx_lo[r] = words[w0];
        idx_hi[r] = words[w0 + (wide ? 1 : 0)];
      }
    }
  }
  auto stage_keys = [&]() {
    const int ctid = tid;
    int* lo = idx_lo; int* hi = idx_hi;
    int mine = -1;
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
      if (r * 512 < list_tiles * kTK) {
        const int i = ctid + 512 * r;
        const long long k = wide ? (long long)(((unsigned long long)(unsigned)hi[r] << 32) | (unsigned)lo[r]) : (long long)lo[r];
        const bool ok = i < n_keys && k >= 0 && k < p.Skv;
        int row = ok ? (int)k : -1;
        if (i < list_tiles * kTK) keys[i] = row;
        if (ok) mine = i;
        // a tile is the 32 consecutive entries of half a wavefront; the masked-key path also serves a
        // non-positive softmax scale (the plain path takes maxima before scaling)
        const unsigned long long okm = __ballot(ok && sm_scale > 0.0f);
        if ((lane & 31) == 0 && i < list_tiles * kTK) tvalid[i / kTK] = (unsigned)(okm >> (lane & 32)) == 0xffffffffu;
      }
    }
    mine = max(mine, __shfl_xor(mine, 1, 64));
    mine = max(mine, __shfl_xor(mine, 2, 64));
    mine = max(mine, __shfl_xor(mine, 4, 64));
    mine = max(mine, __shfl_xor(mine, 8, 64));
    mine = max(mine, __shfl_xor(mine, 16, 64));
    mine = max(mine, __shfl_xor(mine, 32, 64));
    if (lane == 0) last_valid[wave] = mine;
  };
  // causal padding puts the skipped (-1) slots at the end of a list: tiles past the last valid key do nothing
  auto count_tiles = [&]() {
    int m = -1;
#pragma unroll
    for (int w = 0; w < 8; ++w) m = max(m, last_valid[w]);
    return __builtin_amdgcn_readfirstlane((m + kTK) / kTK);
  };
  const size_t q_index = bs;
  // key-split partials: one block per (query, KV group, head chunk, split)
  const size_t part_block = (size_t)(((long long)bs * p.G + g) * chunks + chunk) * p.num_splits + split;
  const size_t part_blocks_total = (size_t)p.B * p.S * p.G * chunks * p.num_splits;

  if (producer) {
    // =====================================================================================
    // producer p = role: heads 16p .. 16p+15 of the chunk
    // =====================================================================================
    const int n = lane & 15, kg = lane >> 4;
    // Q^T operands: lane (head n, kg) holds channels 128 blk + 32 kg .. +31 of the latent and
    // channels 512 + 32 r + 8 kg .. +7 of the rope tail
    // The 16 query rows of this wavefront (18 KB, contiguous when every head exists) are fetched as
    // they lie in memory - piece lane + 64 t, neighbouring lanes on neighbouring 16 bytes; a load whose
    // lanes each point into another row moves a quarter of the bytes per clock - and reach operand
    // order through the ring slot 1 + role, which holds no tile before the first barrier of the
    // pipeline (rows padded by 16 bytes: the 16 lanes of an operand read fall on distinct banks).
    typedef __attribute__((ext_vector_type(4))) unsigned u4;
    constexpr int kQPieces = kDqk / 8;              // 72 pieces of 16 bytes per head row
    constexpr int kQPitch = kDqk * 2 + 16;          // 1168
    static_assert(16 * kQPitch <= kLatBytes + kRopeBytes, "the query rows fit a slot without touching its scale area");
    u4 qload[18];
#pragma unroll
    for (int t = 0; t < 18; ++t) {
      const int P = lane + 64 * t, hl = P / kQPieces, piece = P - hl * kQPieces;
      const int h = 16 * role + hl;
      // heads past the end of the group repeat head 0: their columns stay finite and are never stored
      qload[t] = *reinterpret_cast<const u4*>((const unsigned short*)p.q + (bs * p.H + head0 + (h < heads_here ? h : 0)) * (size_t)kDqk + 8 * piece);
    }
    __builtin_amdgcn_sched_barrier(0);
    stage_keys();
    unsigned char* qstage = smem + (1 + role) * kSlotBytes;
#pragma unroll
    for (int t = 0; t < 18; ++t) {
      const int P = lane + 64 * t, hl = P / kQPieces, piece = P - hl * kQPieces;
      *reinterpret_cast<u4*>(qstage + hl * kQPitch + piece * 16) = qload[t];
    }
    uint4 qraw[4][4];
    bf16x8 qr[2];
#pragma unroll
    for (int blk = 0; blk < 4; ++blk)
#pragma unroll
      for (int j = 0; j < 4; ++j) qraw[blk][j] = *reinterpret_cast<const uint4*>(qstage + n * kQPitch + (16 * blk + 4 * kg + j) * 16);
#pragma unroll
    for (int r = 0; r < 2; ++r) qr[r] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(qstage + n * kQPitch + (64 + 4 * r + kg) * 16));
    __syncthreads();                                // keys[] is complete
    const int n_tiles = count_tiles();
    i32x8 qh[4], ql[4];
    int qexp = 0;
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) qexp |= split_q32(qraw[blk], qh[blk], ql[blk]) << (8 * blk);
    float m_run = -INFINITY;                      // base-2 running reference of head n
    float l_run = 0.0f;                           // this lane's share of its denominator
    const float qk_scale = sm_scale * kLog2e;

    // K operands of a tile -> registers: per sub-tile four 32-byte block fragments and two rope
    // fragments.  The first sub-tile is requested one tile ahead, right after the previous tile's
    // products, so that it lands under its softmax; the second one at the start of the tile, under
    // the first one's products.
    i32x8 kf[2][4];
    bf16x8 rf[2][2];
    // (a tile's slot is passed as its byte offset into the ring, a running value: one address
    // register per slot then reaches every operand of the tile with an immediate offset)
    auto load_k = [&](unsigned slot_off, int sj) {
      const unsigned char* slot = smem + (slot_off + (unsigned)lane * 16u);
      // the lane's 32 bytes of a block are its 16 bytes of the block's two planes
      const unsigned char* lat = slot + sj * (4 * kPair);
      const unsigned char* rope = slot + kLatBytes + sj * 2048;
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
        const uint4 c0 = *reinterpret_cast<const uint4*>(lat + blk * kPair);
        const uint4 c1 = *reinterpret_cast<const uint4*>(lat + blk * kPair + kPlane);
        kf[sj][blk] = i32x8{(int)c0.x, (int)c0.y, (int)c0.z, (int)c0.w, (int)c1.x, (int)c1.y, (int)c1.z, (int)c1.w};
      }
      rf[sj][0] = *reinterpret_cast<const bf16x8*>(rope);
      rf[sj][1] = *reinterpret_cast<const bf16x8*>(rope + 1024);
    };
    constexpr int kOne = 0x7f7f7f7f;                // operand exponent bytes of 2^0: the key bytes enter the products unscaled

    // scores and probabilities of tile tau (the operands of its first sub-tile are in registers) ->
    // P(tau) in LDS.  The common tile - every key valid, no head's maximum above its reference by
    // more than 2^kLazy - is written straight away, a sub-tile's probabilities under the other's
    // products, with its block scales still in registers; the maxima are looked at afterwards, and
    // a tile that moves a reference, or holds skipped keys, is written again the careful way.
    auto produce = [&](int tau, unsigned slot_off, unsigned next_off) {
      const unsigned char* slot = smem + slot_off;
      const int spar = tau & 1;
      const float* scl_base = reinterpret_cast<const float*>(slot + kLatBytes + kRopeBytes);
      const bool all_valid = tvalid[tau] != 0;      // (uniform) no skipped key in this tile
      // "no head of this tile moves its reference": written first, so that the common tile ends
      // without an LDS write the barrier would have to wait for
      if (lane == 0) flagbuf[spar * 4 + role] = 0;
      load_k(slot_off, 1);
      // scales of keys 16 sj + 4 kg + i, one per block: they multiply the block's partial sums here and
      // the probabilities that go to the value product of that block
      auto load_scales = [&](int sj, float (&ksc)[4][nblk]) {
        const float* sclc = scl_base + (16 * sj + 4 * kg) * nblk;
        if (nblk == 4) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float4 v4 = *reinterpret_cast<const float4*>(sclc + 4 * i);
            ksc[i][0] = v4.x; ksc[i][1 % nblk] = v4.y; ksc[i][2 % nblk] = v4.z; ksc[i][3 % nblk] = v4.w;
          }
        } else if (nblk == 2) {
          const float4 a = *reinterpret_cast<const float4*>(sclc), bq = *reinterpret_cast<const float4*>(sclc + 4);
          ksc[0][0] = a.x; ksc[0][1 % nblk] = a.y; ksc[1][0] = a.z; ksc[1][1 % nblk] = a.w;
          ksc[2][0] = bq.x; ksc[2][1 % nblk] = bq.y; ksc[3][0] = bq.z; ksc[3][1 % nblk] = bq.w;
        } else {
          const float4 a = *reinterpret_cast<const float4*>(sclc);
          ksc[0][0] = a.x; ksc[1][0] = a.y; ksc[2][0] = a.z; ksc[3][0] = a.w;
        }
      };
      float ks0[4][nblk], ks1[4][nblk];
      load_scales(0, ks0);
      load_scales(1, ks1);
      // per sub-tile: the rope part first (it needs no scale); then each latent block is accumulated
      // apart, from zero, and enters the score times its keys' block scales.  Two blocks alternate so
      // that a block's scales are applied under the next products.
      f32x4 st[2];
      auto subtile = [&](auto sj_c, const float (&ksc)[4][nblk]) {
        constexpr int sj = decltype(sj_c)::value;
        st[sj] = f32x4{0.f, 0.f, 0.f, 0.f};
        mfma_s(st[sj], rf[sj][0], qr[0]);
        mfma_s(st[sj], rf[sj][1], qr[1]);
        auto pair = [&](auto b_c) {
          constexpr int b0 = decltype(b_c)::value, b1 = b0 + 1;
          f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0;
          mfma_s8<b0>(a0, kf[sj][b0], qh[b0], kOne, qexp);
          mfma_s8<b1>(a1, kf[sj][b1], qh[b1], kOne, qexp);
          mfma_s8<b0>(a0, kf[sj][b0], ql[b0], kOne, qexp);
          mfma_s8<b1>(a1, kf[sj][b1], ql[b1], kOne, qexp);
#pragma unroll
          for (int i = 0; i < 4; ++i) st[sj][i] = __builtin_fmaf(ksc[i][(b0 * nblk) >> 2], a0[i], st[sj][i]);
#pragma unroll
          for (int i = 0; i < 4; ++i) st[sj][i] = __builtin_fmaf(ksc[i][(b1 * nblk) >> 2], a1[i], st[sj][i]);
        };
        pair(std::integral_constant<int, 0>{});
        pair(std::integral_constant<int, 2>{});
      };
      // P -> LDS in the B-operand layout of the 32x32x16 product: lane (head of a 32-head block,
      // key/8) owns 16 bytes = 8 keys; this lane holds keys 4kg..4kg+3.  One plane per scale block:
      // plane b is P times the keys' scales of block b (fp32 product, rounded to bf16 once), so the
      // value product of block b takes V's bytes unscaled.
      unsigned char* pdst = smem + kPOff + spar * kPBytes + ((role >> 1) * 64 + (role & 1) * 16 + n + (kg >> 1) * 32) * 16 + (kg & 1) * 8;
      float l_add = 0.0f;
      auto emit = [&](int sj, const float (&ksc)[4][nblk], float mul, float neg_m) {
        float pr[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          pr[i] = fast_exp2(__builtin_fmaf(st[sj][i], mul, neg_m));
          l_add += pr[i];
        }
#pragma unroll
        for (int pb = 0; pb < nblk; ++pb) {
          *reinterpret_cast<uint2*>(pdst + pb * kPPlane + sj * 2048) =
              make_uint2(pack_bf16(pr[0] * ksc[0][pb], pr[1] * ksc[1][pb]), pack_bf16(pr[2] * ksc[2][pb], pr[3] * ksc[3][pb]));
        }
      };
      // (a head with no valid key yet has m_run = -inf: its tile is always written the careful way)
      const float neg_m0 = -vmax(m_run, -1.0e30f);
      subtile(std::integral_constant<int, 0>{}, ks0);
      subtile(std::integral_constant<int, 1>{}, ks1);
      load_k(next_off, 0);                          // (the fragment registers are free again; a tile that does not exist reads as garbage nobody uses)
      if (all_valid) {
        emit(0, ks0, qk_scale, neg_m0);
        emit(1, ks1, qk_scale, neg_m0);
      }
      // ---- the tile's maxima: this lane holds head n, keys 16 sj + 4 kg + i ----
      float mx;
      float mul = qk_scale;                         // what turns a held sum into a base-2 score
      if (all_valid) {
        // no skipped key: the maximum is taken on the raw sums (qk_scale > 0 on this path)
        mx = vmax3(vmax3(st[0][0], st[0][1], st[0][2]), vmax3(st[0][3], st[1][0], st[1][1]), vmax(st[1][2], st[1][3]));
      } else {
        int4 kk[2];
#pragma unroll
        for (int sj = 0; sj < 2; ++sj) kk[sj] = *reinterpret_cast<const int4*>(keys + tau * kTK + 16 * sj + 4 * kg);
        mx = -INFINITY;
#pragma unroll
        for (int sj = 0; sj < 2; ++sj) {
          const bool ok[4] = {kk[sj].x >= 0, kk[sj].y >= 0, kk[sj].z >= 0, kk[sj].w >= 0};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            st[sj][e] = ok[e] ? st[sj][e] * qk_scale : -INFINITY;
            mx = fmaxf(mx, st[sj][e]);
          }
        }
        mul = 1.0f;
      }
      mx = max_rows(mx) * mul;                 // over the four key quarters (lanes n, n+16, n+32, n+48)
      const bool grow = mx > m_run + kLazy;
      const bool any_grow = __ballot(grow) != 0ull;           // (uniform)
      bool any_rescale = false;
      if (any_grow) {
        // accumulators of a head whose reference was -inf are still zero: nothing to rescale
        any_rescale = __ballot(grow && m_run != -INFINITY) != 0ull;
        float fac = 1.0f;
        if (grow) {
          fac = (m_run == -INFINITY) ? 1.0f : fast_exp2(m_run - mx);
          l_run *= fac;
          m_run = mx;
        }
        if (any_rescale && lane < 16) facbuf[(spar * 4 + role) * 16 + n] = fac;
      }
      if (any_rescale && lane == 0) flagbuf[spar * 4 + role] = 1;
      if (any_grow || !all_valid) {
        // the careful way: exp2(-inf - m) is 0 for a finite m; a head with no valid key yet keeps m_run = -inf
        const float neg_m = -vmax(m_run, -1.0e30f);
        l_add = 0.0f;
        emit(0, ks0, mul, neg_m);
        emit(1, ks1, mul, neg_m);
      }
      l_run += l_add;
    };

    // t = -1: [X] tile 0 has landed.  t >= 0: [B_t] tile t+2 has landed, P(t) is complete, the value
    // product of tile t-1 is done.
    unsigned s_cur = 0, s_nxt = kSlotBytes;       // ring offsets of the tile produced in this round and of the next one
    for (int t = -1; t < n_tiles; ++t) {
      __syncthreads();
      // (the first barrier only promises tile 0: tile 1's operands are read a round late, once)
      if (t <= 0 && t + 1 < n_tiles) load_k(s_cur, 0);
      if (t + 1 < n_tiles) produce(t + 1, s_cur, s_nxt);
      s_cur = s_nxt;
      s_nxt = s_nxt + kSlotBytes == kRingBytes ? 0u : s_nxt + kSlotBytes;
    }
    l_run += xor16(l_run);
    l_run += xor32(l_run);
    if (lane < 16) {
      stats[(role * 16 + lane) * 2 + 0] = m_run;
      stats[(role * 16 + lane) * 2 + 1] = l_run;
    }
    __syncthreads();                              // [E] statistics are visible; the ring is free
    return;
  }

  // =======================================================================================
  // consumer c = role: value channels 128c .. 128c+127 of all 64 heads; also the row loads
  // =======================================================================================
  stage_keys();
  __syncthreads();                                // keys[] is complete
  const int n_tiles = count_tiles();
  // HBM -> LDS.  A skipped key fetches cache row 0 instead (its probability is zero), so every
  // tile is the same six load instructions per wavefront and the in-order load counter can be
  // waited on by count.  The loads are inline assembly (the compiler would otherwise order every
  // later LDS read behind them) with a uniform 64-bit base and a 32-bit byte offset per lane:
  //   latent : block c of both sub-tiles, two planes each: lane (n, kg) of plane j fetches bytes
  //            128 c + 32 kg + 16 j .. + 15 of key 16 sj + n
  //   rope   : plane (sj = c / 2, s = c % 2): lane (n, kq) fetches bytes 64 s + 16 kq .. + 15 of the rope row
  //   scales : elements 8 nblk c .. 8 nblk (c + 1) - 1 of [32 rows][nblk], one per lane (without
  //            scales in memory: a word nobody reads, so that the count stays six)
  const size_t group_row0 = ((size_t)b * p.Skv_pitch) * p.G + g;     // cache row of key 0; key k is G rows further per step
  const unsigned char* lat_base = (const unsigned char*)p.kv + group_row0 * kLat;
  const unsigned char* rope_base = (const unsigned char*)p.rope + group_row0 * (kRope * 2);
  const unsigned char* sc_base = has_scale ? (const unsigned char*)p.kv_scale + group_row0 * nblk * 4 : (const unsigned char*)p.kv;
  const unsigned lat_step = (unsigned)p.G * kLat, rope_step = (unsigned)p.G * (kRope * 2), sc_step = has_scale ? (unsigned)p.G * nblk * 4 : 0u;
  const unsigned lat_lane = 128u * role + 32u * (lane >> 4), rope_lane = 64u * (role & 1) + 16u * (lane >> 4);
  const int sc_elem = 8 * nblk * role + lane;                         // (lanes below 8 nblk)
  const unsigned sc_lane = has_scale ? 4u * (unsigned)(sc_elem % nblk) : 0u;
  const int sc_row = min(sc_elem / nblk, kTK - 1);
  const bool sc_active = lane < 8 * nblk;
  const unsigned sc_dst = kLatBytes + kRopeBytes + (has_scale ? 32u * nblk * role : 256u);
  auto dma16 = [&](const unsigned char* base, unsigned off, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
  };
  auto dma4 = [&](const unsigned char* base, unsigned off, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
  };
  const unsigned smem_base = (unsigned)(size_t)(lds_void*)smem;                 // LDS byte address of the ring
  // prepare computes the lanes' byte offsets of a tile, part(i) issues instruction i of it into the
  // slot at `dma_slot`.  The value product spreads the parts between its matrix instructions:
  // issuing blocks while the load unit's queue is full.
  unsigned dma_slot = 0;                          // (uniform) LDS address of the slot being filled
  unsigned off_l0 = 0, off_l1 = 0, off_r = 0, off_s = 0;
  auto dma_prepare = [&](int tau, unsigned slot_off) {
    dma_slot = smem_base + slot_off;
    const int* tk = keys + tau * kTK;
    const unsigned k0 = (unsigned)max(tk[lane & 15], 0), k1 = (unsigned)max(tk[16 + (lane & 15)], 0);   // this lane's key of sub-tile 0 / 1
    const unsigned ks = (unsigned)max(tk[sc_row], 0);
    off_l0 = __umul24(k0, lat_step) + lat_lane;
    off_l1 = __umul24(k1, lat_step) + lat_lane;
    off_r = __umul24((role >> 1) ? k1 : k0, rope_step) + rope_lane;
    off_s = __umul24(ks, sc_step) + sc_lane;
  };
  auto dma_part = [&](int i) {
    if (i == 0) dma16(lat_base, off_l0, dma_slot + role * kPair);
    else if (i == 1) dma16(lat_base, off_l0 + 16u, dma_slot + role * kPair + kPlane);
    else if (i == 2) dma16(lat_base, off_l1, dma_slot + (4 + role) * kPair);
    else if (i == 3) dma16(lat_base, off_l1 + 16u, dma_slot + (4 + role) * kPair + kPlane);
    else if (i == 4) dma16(rope_base, off_r, dma_slot + kLatBytes + role * 1024);
    else if (sc_active) dma4(sc_base, off_s, dma_slot + sc_dst);
  };
  auto issue_tile = [&](int tau) {
    dma_prepare(tau, (unsigned)(tau % kRing) * kSlotBytes);
#pragma unroll
    for (int i = 0; i < 6; ++i) dma_part(i);
  };

  // ---- value side state: o[dvb][hb] = O^T[32 channels x 32 heads] ----
  f32x16 o[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int hb = 0; hb < 2; ++hb)
#pragma unroll
      for (int j = 0; j < 16; ++j) o[i][hb][j] = 0.0f;
  const int pvar = (role * nblk) >> 2;                         // scale block of channels 128c..
  // transposing reads of V^T: lanes t = 0..15 of a group read 8 bytes each from eight consecutive
  // keys' 16-byte pieces (128 contiguous bytes); half selects the plane, kq2 the upper eight keys of
  // the step; the four 32-channel blocks are 256 bytes apart
  const unsigned char* pv_lane;
  {
    const int t = lane & 15, half = (lane >> 4) & 1, kq2 = lane >> 5;
    const int r = 8 * kq2 + (t >> 1);                          // key within the 16-key step
    pv_lane = smem + role * kPair + half * kPlane + r * 16 + 8 * (t & 1);
  }
  // V^T fragments of one 16-key step (four 32-channel blocks) of the tile in the slot at `slot_off`, raw
  auto load_v = [&](unsigned slot_off, int kstep, i32x2 (&vr)[4]) {
    const unsigned char* vslot = pv_lane + slot_off;
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb)
      vr[dvb] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)(vslot + kstep * (4 * kPair) + dvb * 256));
  };
  const unsigned char* p_lane = smem + kPOff + pvar * kPPlane + lane * 16;
  i32x2 v0[4];                                    // first step of the tile about to be consumed (read ahead of the barrier)
  // value product of tile tv (in the slot at `cur`); NEXT: tile tv+1 exists (in the slot at `nxt`; it
  // has landed: the producers are reading it); DMA: tile tv + kAhead exists and goes to the slot at `prv`
  auto consume = [&](int tv, unsigned cur, unsigned nxt, unsigned prv, auto next_c, auto dma_c) {
    constexpr bool next = decltype(next_c)::value, dma = decltype(dma_c)::value;
    const int vpar = tv & 1;
    if (dma) dma_prepare(tv + kAhead, prv);
    const unsigned char* pfrag = p_lane + vpar * kPBytes;
    bf16x8 pb[2][2];
#pragma unroll
    for (int kstep = 0; kstep < 2; ++kstep)
#pragma unroll
      for (int hb = 0; hb < 2; ++hb) pb[kstep][hb] = *reinterpret_cast<const bf16x8*>(pfrag + (kstep * 2 + hb) * 1024);
    const int4 fl = *reinterpret_cast<const int4*>(flagbuf + vpar * 4);
    i32x2 v1[4];
    load_v(cur, 1, v1);
    __builtin_amdgcn_sched_barrier(0);
    if (__builtin_amdgcn_readfirstlane(fl.x | fl.y | fl.z | fl.w) != 0) {      // producers moved a reference: rescale (rare)
#pragma unroll
      for (int hb = 0; hb < 2; ++hb) {
        const int hd = lane & 31;
        const int fl_p = hb == 0 ? ((hd >> 4) ? fl.y : fl.x) : ((hd >> 4) ? fl.w : fl.z);
        const float fsc = fl_p ? facbuf[(vpar * 4 + 2 * hb + (hd >> 4)) * 16 + (hd & 15)] : 1.0f;
#pragma unroll
        for (int dvb = 0; dvb < 4; ++dvb)
#pragma unroll
          for (int j = 0; j < 16; ++j) o[dvb][hb][j] *= fsc;
      }
    }
    bf16x8 a[4];
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb) a[dvb] = cvt8((unsigned)v0[dvb][0], (unsigned)v0[dvb][1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb) {
      mfma_o(o[dvb][0], a[dvb], pb[0][0]);
      mfma_o(o[dvb][1], a[dvb], pb[0][1]);
      if (dma) dma_part(dvb);
    }
    if (next) load_v(nxt, 0, v0);
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb) a[dvb] = cvt8((unsigned)v1[dvb][0], (unsigned)v1[dvb][1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb) {
      mfma_o(o[dvb][0], a[dvb], pb[1][0]);
      mfma_o(o[dvb][1], a[dvb], pb[1][1]);
      if (dma && dvb < 2) dma_part(4 + dvb);
    }
  };

  // ---- pipeline ----
  // only the first tile is requested ahead of the first barrier (issuing blocks while the load
  // unit's queue is full, and the producers cannot start before this wavefront gets there)
  if (n_tiles > 0) issue_tile(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // tile 0 has landed
  __syncthreads();                                // [X]
#pragma unroll
  for (int tau = 1; tau < kAhead; ++tau)
    if (tau < n_tiles) issue_tile(tau);
  if (n_tiles > 0) load_v(0u, 0, v0);
  // tile 2 has landed (a fourth tile may stay in flight)
  if (n_tiles >= kAhead) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  {
    // slots of tile t, t + 1 and t - 1 (= the slot tile t + kAhead goes to), as byte offsets into the ring
    unsigned cur = 0, nxt = kSlotBytes, prv = (kRing - 1) * kSlotBytes;
    auto advance = [&]() {
      prv = cur;
      cur = nxt;
      nxt = nxt + kSlotBytes == kRingBytes ? 0u : nxt + kSlotBytes;
    };
    const int n_steady = max(n_tiles - kAhead, 0);
    int t = 0;
    for (; t < n_steady; ++t) {
      __syncthreads();                              // [B_t]
      consume(t, cur, nxt, prv, std::true_type{}, std::true_type{});     // (tile t+4 goes into the slot of tile t-1)
      // tile t+3 must have landed before the next barrier; the tile just issued may stay in flight
      asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
      advance();
    }
    for (; t < n_tiles - 1; ++t) {
      __syncthreads();                              // [B_t]
      consume(t, cur, nxt, prv, std::true_type{}, std::false_type{});
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      advance();
    }
    if (t < n_tiles) {
      __syncthreads();                              // [B_t], the last tile
      consume(t, cur, nxt, prv, std::false_type{}, std::false_type{});
    }
  }
  __syncthreads();                                // [E] statistics are visible; the ring is free

  // ---- epilogue ----
  const int hd = lane & 31, gq2 = lane >> 5;
  const bool direct = p.num_splits == 1;
  float* xbuf = reinterpret_cast<float*>(smem) + role * 32 * kXPitch;     // private to this wavefront
#pragma unroll
  for (int hb = 0; hb < 2; ++hb) {
    const float m_all = stats[((2 * hb + (hd >> 4)) * 16 + (hd & 15)) * 2];
    const float l_all = stats[((2 * hb + (hd >> 4)) * 16 + (hd & 15)) * 2 + 1];
    const int h_local = 32 * hb + hd;
    if (!direct) {
      // key split: the unnormalised accumulators leave exactly as the lanes hold them (rounded to
      // bf16: the values are relative to the split's own maximum, so their range is that of the
      // output times the split's probability mass)
      // (two accumulator rows of a lane per 16-byte store: [consumer][head half][dvb][row pair][lane][8])
      unsigned short* blk = (unsigned short*)p.workspace + part_block * (size_t)(2 * kPartFloats) +
                            ((size_t)((role * 2 + hb) * 8) * 64 + lane) * 8;
#pragma unroll
      for (int dvb = 0; dvb < 4; ++dvb) {
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
          const f32x16& acc = o[dvb][hb];
          *reinterpret_cast<uint4*>(blk + (size_t)(dvb * 2 + j2) * 512) =
              make_uint4(pack_bf16(acc[8 * j2], acc[8 * j2 + 1]), pack_bf16(acc[8 * j2 + 2], acc[8 * j2 + 3]),
                         pack_bf16(acc[8 * j2 + 4], acc[8 * j2 + 5]), pack_bf16(acc[8 * j2 + 6], acc[8 * j2 + 7]));
        }
      }
      if (role == 0 && lane < 32) {
        float* ml = (float*)((unsigned short*)p.workspace + part_blocks_total * (size_t)(2 * kPartFloats)) + (part_block * kHeadsWg + h_local) * 2;
        ml[0] = m_all;
        ml[1] = l_all;
      }
      continue;
    }
    float out_scale = 1.0f, lse_val = 0.0f;
    {
      float m_fin = m_all, l_fin = l_all;
      if (mla_has_sinks(p) && h_local < heads_here) {
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
    // transpose through LDS: lane (head hd, gq2) holds channels 32dvb + 8j + 4gq2 + (0..3) in o[.][4j..4j+3]
#pragma unroll
    for (int dvb = 0; dvb < 4; ++dvb) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x16& acc = o[dvb][hb];
        const float4 v = make_float4(acc[4 * j] * out_scale, acc[4 * j + 1] * out_scale, acc[4 * j + 2] * out_scale,
                                     acc[4 * j + 3] * out_scale);
        *reinterpret_cast<float4*>(xbuf + hd * kXPitch + 32 * dvb + 8 * j + 4 * gq2) = v;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // rows of 128 channels leave coalesced: 16 lanes x 8 channels, four heads per step
#pragma unroll 4
    for (int it = 0; it < 8; ++it) {
      const int row = 4 * it + (lane >> 4), c8 = (lane & 15) * 8;
      const int hl = 32 * hb + row;
      if (hl >= heads_here) continue;
      const float4 v = *reinterpret_cast<const float4*>(xbuf + row * kXPitch + c8);
      const float4 u = *reinterpret_cast<const float4*>(xbuf + row * kXPitch + c8 + 4);
      const size_t off = (q_index * p.H + head0 + hl) * (size_t)kLat + 128 * role + c8;
      if (p.out_dtype == CPPMEGA_MI355_F32) {
        *reinterpret_cast<float4*>((float*)p.out + off) = v;
        *reinterpret_cast<float4*>((float*)p.out + off + 4) = u;
      } else if (p.out_dtype == CPPMEGA_MI355_BF16) {
        *reinterpret_cast<uint4*>((unsigned short*)p.out + off) =
            make_uint4(pack_bf16(v.x, v.y), pack_bf16(v.z, v.w), pack_bf16(u.x, u.y), pack_bf16(u.z, u.w));
      } else {
        *reinterpret_cast<uint4*>((unsigned short*)p.out + off) =
            make_uint4(pack_f16(v.x, v.y), pack_f16(v.z, v.w), pack_f16(u.x, u.y), pack_f16(u.z, u.w));
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (role == 0 && lane < 32 && h_local < heads_here && p.lse) p.lse[q_index * p.H + head0 + h_local] = lse_val;
  }
}

// Merges the key splits written by sparse_mla_latent_kernel.  A partial block holds, per
// (consumer w = 128 value channels, 32-head block hg), 16 rows of 64 lanes x float4 exactly as the
// accumulator registers held them: row 4*dvb + j, lane (head hd = lane%32, half = lane/32), element e
// is channel 128w + 32dvb + 8j + 4half + e of head 32hg + hd.  One workgroup per (query, KV group,
// head chunk, w, hg): coalesced 1 KiB row reads, weights per head, transposition through LDS,
// coalesced output rows.
__global__ __launch_bounds__(256) void sparse_mla_latent_combine_kernel(const MlaParams p) {
  constexpr int HG = kHeadsWg / 32;
  __shared__ float x[32][kXPitch];
  const int tid = (int)threadIdx.x, lane = tid & 63, r4 = tid >> 6;
  const int chunks = (p.heads_per_group + 32 * HG - 1) / (32 * HG);
  const int w = (int)blockIdx.y / HG, hg = (int)blockIdx.y % HG;
  const size_t unit = blockIdx.x;                              // (b*S + s, g, chunk)
  const unsigned qg = blockIdx.x / (unsigned)chunks;           // (32-bit divisions: the 64-bit ones are long scalar chains)
  const int chunk = (int)(blockIdx.x - qg * (unsigned)chunks);
  const unsigned bs32 = qg / (unsigned)p.G;
  const int g = (int)(qg - bs32 * (unsigned)p.G);
  const size_t bs = bs32;
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
  if (mla_has_sinks(p) && h_local < heads_here) {
    const float sk = p.sinks[head0 + h_local] * kLog2e;
    m_fin = fmaxf(m_all, sk);
    l_fin = exp2f(sk - m_fin);
  }
  float4 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  const unsigned short* src0 = (const unsigned short*)p.workspace + block0 * (size_t)(HG * kPartFloats) +
                               ((size_t)((w * HG + hg) * 8 + 2 * r4) * 64 + lane) * 8;
#pragma unroll
  for (int s0 = 0; s0 < 16; s0 += 4) {
    if (s0 >= p.num_splits) break;                            // (uniform)
    uint4 raw[4][2];                                           // two accumulator rows per 16-byte load
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = min(s0 + u, p.num_splits - 1);             // a repeated last split gets weight 0
#pragma unroll
      for (int i2 = 0; i2 < 2; ++i2) {                          // (read once: non-temporal, 0.7 us of the decode step)
        typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
        const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src0 + (size_t)s * (HG * kPartFloats) + (size_t)i2 * 512));
        raw[u][i2] = make_uint4(t[0], t[1], t[2], t[3]);
      }
    }
    float4 v[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i2 = 0; i2 < 2; ++i2) {
        v[u][2 * i2] = make_float4(__uint_as_float(raw[u][i2].x << 16), __uint_as_float(raw[u][i2].x & 0xffff0000u),
                                   __uint_as_float(raw[u][i2].y << 16), __uint_as_float(raw[u][i2].y & 0xffff0000u));
        v[u][2 * i2 + 1] = make_float4(__uint_as_float(raw[u][i2].z << 16), __uint_as_float(raw[u][i2].z & 0xffff0000u),
                                       __uint_as_float(raw[u][i2].w << 16), __uint_as_float(raw[u][i2].w & 0xffff0000u));
      }
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
  if ((unsigned long long)p.B * p.Skv_pitch * p.G >= 0x7fffffffull) return false;   // cache rows are counted in 32 bits
  // a lane's byte offset from the first row of its batch is a 24-bit row number times a 24-bit step, below 2^31
  if ((unsigned long long)p.Skv_pitch * p.G * kLat >= (1ull << 31) || p.Skv_pitch >= (1 << 24) || (long long)p.G * kLat >= (1 << 24)) return false;
  if (p.topk > 16 * kMaxKeys) return false;       // the combine step merges at most 16 key splits
  return true;
}

void sparse_mla_latent_plan(MlaParams& p) {
  const int chunks = (p.heads_per_group + kHeadsWg - 1) / kHeadsWg;
  const long long base = (long long)p.B * p.S * p.G * chunks;
  int splits = 1;
  while (base * splits < 256 && p.topk / (splits * 2) >= 4 * kTK && splits < 16) splits *= 2;
  while ((p.topk + splits - 1) / splits > kMaxKeys && splits < 16) splits *= 2;
  p.heads_per_wg = kHeadsWg;
  const int tiles = (p.topk + kTK - 1) / kTK;
  const int tiles_per_split = (tiles + splits - 1) / splits;
  p.num_splits = splits;
  p.keys_per_split = tiles_per_split * kTK;
}

int sparse_mla_latent_launch(const MlaParams& p, hipStream_t stream) {
  const int chunks = (p.heads_per_group + kHeadsWg - 1) / kHeadsWg;
  const long long wgs = (long long)p.B * p.S * p.G * p.num_splits * chunks;
  if (wgs > 0x7fffffffll || p.keys_per_split > kMaxKeys || p.num_splits > 16)
    return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse MLA: launch too large");
  const dim3 grid((unsigned)wgs), block(512);
  const int nblk = p.kv_scale_kind == CPPMEGA_MI355_SCALE_F32_BLOCK ? kLat / p.kv_scale_block : 1;
#define CM_LAUNCH_PC(NB_)                                                                                          \
  do {                                                                                                             \
    CM_HIP_CHECK(hipFuncSetAttribute((const void*)sparse_mla_latent_kernel<NB_>,                                 \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kSmem));                           \
    hipLaunchKernelGGL((sparse_mla_latent_kernel<NB_>), grid, block, kSmem, stream, p);                          \
  } while (0)
  if (nblk == 4) CM_LAUNCH_PC(4);
  else if (nblk == 2) CM_LAUNCH_PC(2);
  else CM_LAUNCH_PC(1);
#undef CM_LAUNCH_PC
  CM_HIP_CHECK(hipGetLastError());
  if (p.num_splits > 1) {
    const dim3 cgrid((unsigned)((size_t)p.B * p.S * p.G * chunks), (unsigned)(4 * (kHeadsWg / 32)));
    hipLaunchKernelGGL(sparse_mla_latent_combine_kernel, cgrid, dim3(256), 0, stream, p);
    CM_HIP_CHECK(hipGetLastError());
  }
  return 0;
}

size_t sparse_mla_latent_workspace_bytes(const MlaParams& p) {
  if (p.num_splits <= 1) return 0;
  const int chunks = (p.heads_per_group + kHeadsWg - 1) / kHeadsWg;
  const size_t blocks = (size_t)p.B * p.S * p.G * chunks * p.num_splits;
  return blocks * ((size_t)2 * kPartFloats * sizeof(unsigned short) + kHeadsWg * 2 * sizeof(float));
}

}  // namespace cm
