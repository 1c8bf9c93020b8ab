// Sparse MLA forward on the matrix cores (gfx950): 32 heads share one gathered
// latent KV stream.
//
// Shapes served: d_qk = 576 = 512 latent + 64 rope, d_v = 512, bf16 queries;
// the latent is e4m3 with one fp32 scale per 128 channels (or per row) plus a
// bf16 rope tail, or a packed bf16 row of 576.  float16 queries with float16
// rows of 576 run the same kernel on the float16 matrix instructions.
// Everything else goes to the scalar kernel.
//
// Decomposition
//   workgroup = (batch*query, group of 32 heads, key split); 4 wavefronts.
//   Each wavefront owns all 32 heads for its own interleaved stream of 16-key
//   tiles, so wavefronts never synchronise inside the key loop; their partial
//   results are merged once at the end through LDS, and the key splits of a
//   query are merged by a second, small kernel.
//
// Per tile (16 gathered keys)
//   stage   the 16 rows (fetched one tile ahead into registers) go e4m3 -> bf16
//           with their block scale (two bytes per instruction when the scale is
//           a power of two, an fp32 multiply otherwise) into a swizzled
//           [16][576] bf16 tile private to the wavefront;
//   QK^T    S^T[16 keys x 32 heads] = K . Q^T as 2 x 18 v_mfma_f32_16x16x32_bf16;
//           K fragments are 16-byte LDS reads, Q^T fragments stay in registers
//           for the whole kernel (144 VGPRs);
//   softmax base-2, running max updated lazily (only when it grows by more
//           than 2^8), so the 256 accumulator registers are rescaled rarely;
//   P.V     O^T[512 x 32 heads] += V^T . P^T as 16 v_mfma_f32_32x32x16_bf16;
//           V^T fragments come from the same tile through the LDS transpose
//           read (ds_read_b64_tr_b16); P^T goes from the S^T accumulators to
//           the B operand with one v_permlane16_swap, never through memory.

#include "sparse_mla_common.h"
#include "mfma_util.h"

namespace cm {
namespace {

constexpr int kLat = 512;          // latent channels (= d_v)
constexpr int kRope = 64;
constexpr int kDqk = kLat + kRope; // 576
constexpr int kTile = 16;          // keys per tile
constexpr int kRowBytes = kDqk * 2;             // 1152: one bf16 key row in LDS
constexpr int kTileBytes = kTile * kRowBytes;   // 18432: the bf16 tile of a wavefront
constexpr int kRawLat = kTile * kLat;           // 8192: the same 16 rows as fetched (e4m3)
constexpr int kRawRope = kTile * kRope * 2;     // 2048
constexpr int kMaxBlocks = 8;                   // scale blocks per row the raw area holds
constexpr int kRawScale = kTile * kMaxBlocks * 4;   // 512
constexpr int kWaveBytes = kTileBytes + kRawLat + kRawRope + kRawScale;   // 29184 per wavefront
constexpr int kHeads = 32;         // heads per workgroup
constexpr int kWaves = 4;
constexpr int kKSteps = kDqk / 32; // 18 MFMA k-steps of 32 channels
constexpr int kXPitch = 260;       // floats per head row of the merge buffer (256 + 4 pad)
constexpr int kXBytes = kWaves * kHeads * kXPitch * 4;    // 133120
constexpr int kStatOff = kXBytes;                         // [4 waves][32 heads][2] floats
constexpr int kSmemBytes = kXBytes + kWaves * kHeads * 2 * 4;
static_assert(kWaves * kWaveBytes <= kXBytes, "the merge buffer reuses the tile area");
// 16-bit rows need no conversion: a wavefront owns two tiles, and the load unit writes the
// next one in its final (swizzled) layout while the current one computes
constexpr int kRowsWaveBytes = 2 * kTileBytes;                            // 36864 per wavefront
constexpr int kRowsStatOff = kWaves * kRowsWaveBytes > kXBytes ? kWaves * kRowsWaveBytes : kXBytes;   // 147456
constexpr int kRowsSmemBytes = kRowsStatOff + kWaves * kHeads * 2 * 4;   // 148480 of the 160 KB
constexpr int kRowsKscOff = kRowsSmemBytes;                              // shared FP8 rows: [2 rounds][64 keys] fp32 row scales
constexpr int kRowsFp8SmemBytes = kRowsKscOff + 2 * kWaves * kTile * 4;  // 148992
static_assert(kRowsFp8SmemBytes <= 160 * 1024, "two 16-bit tiles per wavefront fit the LDS of a CU");
constexpr float kLazy = 8.0f;      // rescale when the running max grows by more than 2^8

// 16-byte chunk q of row r lives at chunk (q with its low 3 bits xor f(r)):
// 8 consecutive rows hit 8 different bank groups for the same q (16-byte
// fragment reads), and 4 consecutive rows x 2 adjacent chunks hit all 8
// (transpose reads).
__device__ __forceinline__ int swz(int q, int r) {
  const int f = ((r & 3) << 1) | ((r >> 2) & 1);
  return (q & ~7) | ((q & 7) ^ f);
}

__device__ __forceinline__ bf16x8 lds_read_b128(const unsigned char* base, int byte_off) {
  return *reinterpret_cast<const bf16x8*>(base + byte_off);
}

__device__ __forceinline__ bf16x4 lds_read_tr16_b64(const unsigned char* addr) {
  typedef __attribute__((ext_vector_type(4))) short s16x4;
  const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)addr);
  return __builtin_bit_cast(bf16x4, v);
}

// KV_FP8: latent e4m3 + fp32 scales (+ bf16 rope tail); otherwise a 16-bit row of 576 (or 512 + rope
// tail) in the queries' type: bf16, or float16 with F16 (the float-carrier kernels of
// cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py compute on float16 rows)
// SHARE (16-bit rows, more than 32 heads per KV group): the 4 wavefronts take 4 groups of 32
// heads and walk the same keys - every wavefront fetches one tile of a round of 4 and all compute
// on all 4, so a gathered row is read from the cache once per 128 heads instead of once per 32.
// ROWS (with KV_FP8): key rows of 576 e4m3 codes and e4m3 queries, the prepared buffers of
//   1: cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py - one fp32 scale per row and per (query,
//      head).  Codes become bfloat16 exactly; the two scales multiply the scores (and the key's
//      scale its probability on the way into P.V), so no operand is rounded;
//   2: cppmega_mlx/nn/_tilelang/sparse_mla_blockscaled_path_c.py - one E8M0 byte per 32 channels
//      on both sides.  A power of two times an e4m3 code is a bfloat16, so the scaled values enter
//      the products exactly as well.
template <bool KV_FP8, bool F16 = false, bool SHARE = false, int ROWS = 0>
__global__ __launch_bounds__(kWaves * 64, 1) void sparse_mla_mfma_kernel(const MlaParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr bool STAGED = KV_FP8 && !SHARE;      // rows arrive in a raw area and are converted from there
  unsigned char* tile = smem + wave * (STAGED ? kWaveBytes : kRowsWaveBytes);
  unsigned char* raw_lat = tile + kTileBytes;
  unsigned char* raw_rope = raw_lat + kRawLat;
  unsigned char* raw_sc = raw_rope + kRawRope;
  constexpr bool TOK = ROWS == 1, E8 = ROWS == 2, R576 = ROWS != 0;
  constexpr int kE8Row = kDqk / 32;              // 18 scale bytes per row

  // ---- which (query, head group, split) ------------------------------------
  const int groups_per_kv = (p.heads_per_group + kHeads - 1) / kHeads;
  const int units = SHARE ? (groups_per_kv + kWaves - 1) / kWaves : groups_per_kv;   // workgroups per KV group
  const int hg = (int)blockIdx.x % (p.G * units);
  const size_t bs = blockIdx.x / (p.G * units);                  // b*S + s
  const int split = (int)blockIdx.y;
  const int g = hg / units;
  // the 32 heads of this wavefront (SHARE) or of the whole workgroup; a wavefront past the last
  // head group has none and only fetches
  const int head0 = g * p.heads_per_group + (SHARE ? (hg % units) * kWaves + wave : hg % units) * kHeads;
  const int heads_here = max(0, min(kHeads, (g + 1) * p.heads_per_group - head0));
  const int b = (int)(bs / p.S);
  const size_t idx_base = (bs * p.G + g) * (size_t)p.topk;
  const int key_begin = split * p.keys_per_split;
  const int key_end = min(p.topk, key_begin + p.keys_per_split);
  const int n_tiles = (key_end - key_begin + kTile - 1) / kTile;  // tiles of this split

  // ---- Q^T fragments: lane (head n = lane%16, kq = lane/16) for both head halves ----
  bf16x8 qf[2][kKSteps];
  {
    const int n = lane & 15, kq = lane >> 4;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int h = hh * 16 + n;
      const bool live = h < heads_here;
      const unsigned short* qrow = (const unsigned short*)p.q + (bs * p.H + head0 + (live ? h : 0)) * (size_t)kDqk;
      const unsigned char* qcodes = (const unsigned char*)p.q + (bs * p.H + head0 + (live ? h : 0)) * (size_t)kDqk;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        uint4 t = make_uint4(0, 0, 0, 0);
        if (E8) {
          uint2 c = make_uint2(0, 0);
          float sc = 0.0f;
          if (live) {
            c = *reinterpret_cast<const uint2*>(qcodes + 32 * ks + 8 * kq);
            sc = e8m0_to_f32(((const unsigned char*)p.q_scale)[(bs * p.H + head0 + h) * (size_t)kE8Row + ks]);
          }
          const f32x2 v0 = e4m3x2_lo(c.x), v1 = e4m3x2_hi(c.x), v2 = e4m3x2_lo(c.y), v3 = e4m3x2_hi(c.y);
          t = make_uint4(pack_bf16(v0[0] * sc, v0[1] * sc), pack_bf16(v1[0] * sc, v1[1] * sc),
                         pack_bf16(v2[0] * sc, v2[1] * sc), pack_bf16(v3[0] * sc, v3[1] * sc));
        } else if (TOK) {
          uint2 c = make_uint2(0, 0);
          if (live) c = *reinterpret_cast<const uint2*>(qcodes + 32 * ks + 8 * kq);
          t.x = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c.x, 1.0f, false));
          t.y = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c.x, 1.0f, true));
          t.z = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c.y, 1.0f, false));
          t.w = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c.y, 1.0f, true));
        } else if (live) {
          t = *reinterpret_cast<const uint4*>(qrow + 32 * ks + 8 * kq);
        }
        qf[hh][ks] = __builtin_bit_cast(bf16x8, t);
      }
    }
  }

  f32x16 o[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) o[i][j] = 0.0f;
  float m_run[2] = {-INFINITY, -INFINITY};   // base-2 running reference of heads (lane%16) and 16+(lane%16)
  float l_run[2] = {0.0f, 0.0f};             // this lane's share of the denominators
  const float qk_scale = mla_sm_scale(p) * kLog2e;
  float sfac[2] = {qk_scale, qk_scale};      // what a raw score of heads (lane%16), 16+(lane%16) is multiplied with
  if (TOK) {
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int h = hh * 16 + (lane & 15);
      sfac[hh] = h < heads_here ? qk_scale * ((const float*)p.q_scale)[bs * p.H + head0 + h] : 0.0f;
    }
  }

  // ---- staging ---------------------------------------------------------------------
  // The gathered rows travel HBM -> LDS by the load unit itself (no registers are held
  // while they are in flight): lane l of a 16-byte load instruction lands at base + 16*l.
  //   latent : instruction it (0..7) carries rows 2it, 2it+1  (32 lanes x 16 bytes each)
  //   rope   : instruction it (0..1) carries rows 8it .. 8it+7 (8 lanes x 16 bytes each)
  //   scales : one 4-byte load per (row, block)
  // A lane whose row is invalid issues nothing; what the raw area holds there is finite
  // (zeroed at start, later only real rows) and meets a zero probability.
  const int nblk = KV_FP8 ? (p.kv_scale_kind == CPPMEGA_MI355_SCALE_F32_BLOCK ? kLat / p.kv_scale_block : 1) : 1;
  const bool has_scale = KV_FP8 && p.kv_scale_kind != CPPMEGA_MI355_SCALE_NONE;

  auto key_row = [&](int key_pos) -> int {       // cache row of list position key_pos, or -1
    if (key_pos >= key_end) return -1;
    const long long k = load_index(p, idx_base + key_pos);
    return (k >= 0 && k < p.Skv) ? (int)k : -1;
  };
  const int my_tiles = n_tiles > wave ? (n_tiles - wave + kWaves - 1) / kWaves : 0;
  auto tile_key = [&](int t) -> int {            // lane l reports key (l % 16) of tile t
    return t < my_tiles ? key_row(key_begin + (t * kWaves + wave) * kTile + (lane & 15)) : -1;
  };
  unsigned short e8n[3] = {0, 0, 0};              // E8: scale bytes of the tile in flight
  auto issue_dma = [&](int keyv) {                // keyv: this lane's tile_key() of the tile to fetch
    const bool upper = lane >= 32;
    int rows[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {              // rows 2it (lanes 0..31) and 2it+1 (lanes 32..63)
      const int ra = __builtin_amdgcn_readlane(keyv, 2 * it), rb = __builtin_amdgcn_readlane(keyv, 2 * it + 1);
      rows[it] = upper ? rb : ra;
    }
    const int rope_r0 = __shfl(keyv, lane >> 3, 64), rope_r1 = __shfl(keyv, 8 + (lane >> 3), 64);
    const size_t row_base = (size_t)b * p.Skv_pitch;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      if (rows[it] >= 0) {
        const size_t krow = (row_base + (size_t)rows[it]) * p.G + g;
        const unsigned char* src = (const unsigned char*)p.kv + krow * (R576 ? kDqk : kLat) + (lane & 31) * 16;
        __builtin_amdgcn_global_load_lds((glb_void*)src, (lds_void*)(raw_lat + it * 1024), 16, 0, 0);
      }
    }
    if (R576) {                                   // the last 64 codes of all 16 rows: 4 lanes x 16 bytes each
      const int r = __shfl(keyv, lane >> 2, 64);
      if (r >= 0) {
        const size_t krow = (row_base + (size_t)r) * p.G + g;
        const unsigned char* src = (const unsigned char*)p.kv + krow * kDqk + kLat + (lane & 3) * 16;
        __builtin_amdgcn_global_load_lds((glb_void*)src, (lds_void*)raw_rope, 16, 0, 0);
      }
    }
#pragma unroll
    for (int it = 0; it < (R576 ? 0 : 2); ++it) {
      const int r = it ? rope_r1 : rope_r0;
      if (r >= 0) {
        const size_t krow = (row_base + (size_t)r) * p.G + g;
        const unsigned short* src = (const unsigned short*)p.rope + krow * kRope + (lane & 7) * 8;
        __builtin_amdgcn_global_load_lds((glb_void*)src, (lds_void*)(raw_rope + it * 1024), 16, 0, 0);
      }
    }
    if (E8) {
      // 16 rows x 18 scale bytes as 144 two-byte pieces (a row's bytes start on an even address
      // only), through registers: written to the raw area when the tile is staged
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        const int P = lane + 64 * i;
        const int r = __shfl(keyv, (P / 9) & 15, 64);
        e8n[i] = 0;
        if (P < kTile * 9 && r >= 0) {
          const size_t krow = (row_base + (size_t)r) * p.G + g;
          e8n[i] = *reinterpret_cast<const unsigned short*>((const unsigned char*)p.kv_scale + krow * kE8Row + (P % 9) * 2);
        }
      }
    } else if (has_scale) {
      for (int e0 = 0; e0 < kTile * nblk; e0 += 64) {   // uniform trip count (1 or 2)
        const int e = e0 + lane;
        const int r = __shfl(keyv, (e / nblk) & 15, 64);
        if (e < kTile * nblk && r >= 0) {
          const size_t krow = (row_base + (size_t)r) * p.G + g;
          const float* src = (const float*)p.kv_scale + krow * nblk + (e % nblk);
          __builtin_amdgcn_global_load_lds((glb_void*)src, (lds_void*)(raw_sc + e0 * 4), 4, 0, 0);
        }
      }
    }
  };
  auto stage = [&]() {                            // raw rows -> swizzled bf16 tile
    const int c = lane & 31;
    const int blk = (c * 16) / (kLat / nblk);
    const int hi_row = lane >> 5;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint4 raw[4];
      float sc[4];
      bool all_pow2 = true;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int it = half * 4 + i;
        raw[i] = *reinterpret_cast<const uint4*>(raw_lat + it * 1024 + lane * 16);
        // (TOK: the row's scale goes onto its score and its probability instead)
        if (E8) sc[i] = e8m0_to_f32(raw_sc[(2 * it + hi_row) * kE8Row + (c >> 1)]);
        else sc[i] = has_scale && !TOK ? *reinterpret_cast<const float*>(raw_sc + ((2 * it + hi_row) * nblk + blk) * 4) : 1.0f;
        all_pow2 = all_pow2 && scale_is_pow2(sc[i]);
      }
      const bool fast = __ballot(!all_pow2) == 0ull;      // uniform
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 2 * (half * 4 + i) + hi_row;
        uint4 lo, hi;
        if (fast) dequant16<true>(raw[i], sc[i], lo, hi);
        else dequant16<false>(raw[i], sc[i], lo, hi);
        *reinterpret_cast<uint4*>(tile + r * kRowBytes + swz(2 * c, r) * 16) = lo;
        *reinterpret_cast<uint4*>(tile + r * kRowBytes + swz(2 * c + 1, r) * 16) = hi;
      }
    }
    if (R576) {
      const int r = lane >> 2, c = lane & 3;
      const uint4 raw = *reinterpret_cast<const uint4*>(raw_rope + lane * 16);
      const float sc = E8 ? e8m0_to_f32(raw_sc[r * kE8Row + 16 + (c >> 1)]) : 1.0f;
      uint4 lo, hi;
      if (__ballot(!scale_is_pow2(sc)) == 0ull) dequant16<true>(raw, sc, lo, hi);
      else dequant16<false>(raw, sc, lo, hi);
      *reinterpret_cast<uint4*>(tile + r * kRowBytes + swz(64 + 2 * c, r) * 16) = lo;
      *reinterpret_cast<uint4*>(tile + r * kRowBytes + swz(64 + 2 * c + 1, r) * 16) = hi;
    }
#pragma unroll
    for (int it = 0; it < (R576 ? 0 : 2); ++it) {
      const int r = 8 * it + (lane >> 3);
      const uint4 v = *reinterpret_cast<const uint4*>(raw_rope + it * 1024 + lane * 16);
      *reinterpret_cast<uint4*>(tile + r * kRowBytes + swz(64 + (lane & 7), r) * 16) = v;
    }
  };
  // 16-bit rows: 18 load instructions carry the 16 rows of 1152 bytes straight into a tile.
  // Instruction t fills the tile's bytes [1024t, 1024t + 1024): lane l owns slot P = 64t + l of
  // the tile = slot P % 72 of row P / 72, which holds chunk swz(slot, row) of that row (the
  // swizzle is an exclusive-or, hence its own inverse) - the swizzle is applied on the source side.
  // keyv: lane first + r holds the cache row of the tile's key r (first is uniform)
  // Source of slot 64t + lane, or null for an invalid key.  An instruction touches two rows at most;
  // their addresses are wave-uniform (scalar 64-bit products), a lane only selects and adds.
  auto slot_source = [&](int keyv, int first, int t) -> const unsigned short* {
    const int r0 = (64 * t) / 72;                               // first row the instruction touches
    const int P = 64 * t + lane;
    const bool second = P >= 72 * (r0 + 1);                     // ... and lanes past its end are in row r0 + 1
    const int ra = __builtin_amdgcn_readlane(keyv, first + r0), rb = __builtin_amdgcn_readlane(keyv, first + ((r0 + 1) & 15));
    const size_t row_base = (size_t)b * p.Skv_pitch;
    const size_t ka = (row_base + (size_t)max(ra, 0)) * p.G + g, kb = (row_base + (size_t)max(rb, 0)) * p.G + g;
    const unsigned short* kv_a = (const unsigned short*)p.kv + ka * (size_t)p.d_kv;
    const unsigned short* kv_b = (const unsigned short*)p.kv + kb * (size_t)p.d_kv;
    const unsigned short* rope_a = (const unsigned short*)p.rope + ka * kRope - p.d_kv;
    const unsigned short* rope_b = (const unsigned short*)p.rope + kb * kRope - p.d_kv;
    const int r = second ? r0 + 1 : r0;
    const int c = swz(P - 72 * r, r);
    const bool tail = c * 8 >= p.d_kv;
    const unsigned short* base = second ? (tail ? rope_b : kv_b) : (tail ? rope_a : kv_a);
    return (second ? rb : ra) >= 0 ? base + c * 8 : nullptr;
  };
  auto issue_rows = [&](int keyv, int first, unsigned char* dst) {
#pragma unroll 1
    for (int t = 0; t < kTileBytes / 1024; ++t) {
      const unsigned short* src = slot_source(keyv, first, t);
      if (src) __builtin_amdgcn_global_load_lds((glb_void*)src, (lds_void*)(dst + t * 1024), 16, 0, 0);
    }
  };
  // SHARE: after the first round the rows travel through registers instead: each step fetches a
  // quarter of the wavefront's tile of the next round before its products and writes it to LDS
  // after them.
  // Measured (16-bit rows, 128 heads x 4096 queries x 2048 keys; rows resident in the L2 or not
  // makes no difference, nor do four hot rows that stay in the L1: 3.71 against 3.86 ms in one
  // run): 3.7 ms, of which 2.83 ms remain with the fetches taken out.  A wavefront
  // that is alone on its SIMD issues in order, and what it spends on issuing a load the matrix
  // products do not hide.  Forms that were slower: loads whose lanes straddle two rows with
  // per-lane 64-bit address products, 18 per tile in four uneven shares, 4.09 - 4.25 ms; the same
  // as LDS-writing loads 4.55 ms, all 18 at the start of the round 4.87 ms; the loads of a step
  // spread one at a time between its matrix products 4.2 ms (4.8 ms with the heavier addresses);
  // the four wavefronts fetching at four different points of the step 5.7 ms.
  // Step j of a round fetches rows 4j .. 4j + 3 of the wavefront's tile of the next round:
  //   16-bit rows: four loads of a row's first 64 slots (wave-uniform row address + 16 bytes per
  //     lane) and one load of the last 8 slots of the four rows (32 lanes);
  //   FP8 rows of 576 codes: two loads of the first 512 codes of two rows each (32 lanes a row) and
  //     one of the last 64 codes of the four rows (16 lanes); a lane's 16 codes become 16 bfloat16
  //     (two slots) on their way into the tile.  E8M0: the lane also fetches the scale byte of
  //     its 16 codes.  Per token: step 0 fetches the 16 row scales for the array the four
  //     wavefronts read.
  // Every step has the same shape, so the address of a load is a handful of scalar instructions.
  typedef __attribute__((ext_vector_type(4))) unsigned u4;
  constexpr int kPerStep = R576 ? 3 : 5;
  unsigned char* dma_dst = smem;                  // this wavefront's tile of the next round
  float* ksc_dst = reinterpret_cast<float*>(smem + kRowsKscOff);   // ... and its 16 row scales
  bool dma_on = false;
  int key_dma = -1;                               // lane 16 * wave + r: cache row of key r of that tile
  u4 stg[kPerStep];
  unsigned char stg_e8[kPerStep];
  float stg_ksc = 0.0f;
  // row r of the cache as this (batch, KV group) sees it starts at base + r * stride
  const size_t krow0 = (size_t)b * p.Skv_pitch * p.G + g;
  const unsigned row_bytes = R576 ? (unsigned)kDqk : (unsigned)p.d_kv * 2u;
  const unsigned kv_stride = (unsigned)p.G * row_bytes;
  const unsigned char* kv0 = (const unsigned char*)p.kv + krow0 * row_bytes;
  const bool packed = R576 || p.d_kv == kDqk;     // the last 64 channels sit in the row itself, not in p.rope
  const unsigned char* tail0 = packed ? kv0 + (R576 ? kLat : kLat * 2) : (const unsigned char*)p.rope + krow0 * (kRope * 2);
  const unsigned tail_stride = packed ? kv_stride : (unsigned)p.G * (kRope * 2);
  const unsigned sc_stride = (unsigned)p.G * (E8 ? (unsigned)kE8Row : 4u);
  const unsigned char* sc0 = R576 ? (const unsigned char*)p.kv_scale + krow0 * (E8 ? (size_t)kE8Row : 4) : nullptr;
  auto fetch_one = [&](int j, int i) {            // load i of step j (j uniform, i a constant)
    if (i >= kPerStep) return;
    const int first = 16 * __builtin_amdgcn_readfirstlane(wave) + 4 * j;
    stg[i] = u4{0u, 0u, 0u, 0u};
    stg_e8[i] = 127;                              // scale 1
    if (!dma_on) return;
    if (R576) {
      if (i < 2) {
        const int ra = __builtin_amdgcn_readlane(key_dma, first + 2 * i), rb = __builtin_amdgcn_readlane(key_dma, first + 2 * i + 1);
        const int key = lane < 32 ? ra : rb;
        if (key >= 0) {
          stg[i] = *reinterpret_cast<const u4*>(kv0 + (size_t)key * kv_stride + (lane & 31) * 16);
          if (E8) stg_e8[i] = sc0[(size_t)key * sc_stride + ((lane & 31) >> 1)];
        }
        if (TOK && i == 0 && j == 0) {            // lane r < 16: the scale of the tile's key r
          const int kr = __shfl(key_dma, first + (lane & 15), 64);
          stg_ksc = 0.0f;
          if (kr >= 0) stg_ksc = *reinterpret_cast<const float*>(sc0 + (size_t)kr * sc_stride);
        }
      } else {
        const int key = __shfl(key_dma, first + ((lane >> 2) & 3), 64);
        if (lane < 16 && key >= 0) {
          stg[2] = *reinterpret_cast<const u4*>(tail0 + (size_t)key * tail_stride + (lane & 3) * 16);
          if (E8) stg_e8[2] = sc0[(size_t)key * sc_stride + 16 + ((lane & 3) >> 1)];
        }
      }
    } else if (i < 4) {
      const int key = __builtin_amdgcn_readlane(key_dma, first + i);
      if (key >= 0) stg[i] = *reinterpret_cast<const u4*>(kv0 + (size_t)key * kv_stride + lane * 16);   // uniform branch
    } else {
      const int key = __shfl(key_dma, first + ((lane >> 3) & 3), 64);
      if (lane < 32 && key >= 0) stg[4] = *reinterpret_cast<const u4*>(tail0 + (size_t)key * tail_stride + (lane & 7) * 16);
    }
  };
  auto fetch_share = [&](int j) {
#pragma unroll
    for (int i = 0; i < kPerStep; ++i) fetch_one(j, i);
  };
  auto store_share = [&](int j) {
    if (!dma_on) return;
    if (R576) {
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        const int r = 4 * j + (i < 2 ? 2 * i + (lane >> 5) : (lane >> 2) & 3);
        const int c = i < 2 ? 2 * (lane & 31) : 64 + 2 * (lane & 3);         // first of the two slots
        const float sc = E8 ? e8m0_to_f32(stg_e8[i]) : 1.0f;
        const uint4 raw = make_uint4(stg[i][0], stg[i][1], stg[i][2], stg[i][3]);
        uint4 lo, hi;
        if (__ballot(!scale_is_pow2(sc)) == 0ull) dequant16<true>(raw, sc, lo, hi);
        else dequant16<false>(raw, sc, lo, hi);
        if (i < 2 || lane < 16) {
          *reinterpret_cast<uint4*>(dma_dst + r * kRowBytes + swz(c, r) * 16) = lo;
          *reinterpret_cast<uint4*>(dma_dst + r * kRowBytes + swz(c + 1, r) * 16) = hi;
        }
      }
      if (TOK && j == 0 && lane < kTile) ksc_dst[lane] = stg_ksc;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 4 * j + i;
        *reinterpret_cast<u4*>(dma_dst + r * kRowBytes + swz(lane, r) * 16) = stg[i];
      }
      const int r = 4 * j + ((lane >> 3) & 3);
      if (lane < 32) *reinterpret_cast<u4*>(dma_dst + r * kRowBytes + swz(64 + (lane & 7), r) * 16) = stg[4];
    }
  };

  if (STAGED) {                                   // the raw area starts out as zeros
    for (int i = lane; i < (kRawLat + kRawRope + kRawScale) / 16; i += 64)
      reinterpret_cast<uint4*>(raw_lat)[i] = make_uint4(0, 0, 0, 0);
  } else {                                        // so do both tiles: rows of invalid keys are never fetched
    for (int i = lane; i < kRowsWaveBytes / 16; i += 64) reinterpret_cast<uint4*>(tile)[i] = make_uint4(0, 0, 0, 0);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if (SHARE) __syncthreads();                     // a wavefront's first tile lands in an area another one cleared
  // lane-constant LDS offsets of the operand fragments (the swizzle leaves two variants each)
  int qk_base0, qk_base1, pv_base0a, pv_base0b, pv_base1a, pv_base1b;
  {
    const int m = lane & 15, kq = lane >> 4;
    qk_base0 = m * kRowBytes + swz(kq, m) * 16;
    qk_base1 = m * kRowBytes + swz(4 + kq, m) * 16;
    // transpose reads: 16-lane group g16 covers columns 16*(g16&1)..+15 of a 32-wide block and
    // rows 8*(lane/32) + {0..3} (first read) / {4..7} (second); lane i of the group supplies
    // row i/4, columns 4*(i%4)..+3
    const int i16 = lane & 15, col_half = (lane >> 4) & 1, kq2 = lane >> 5;
    const int r0 = 8 * kq2 + (i16 >> 2), r1 = r0 + 4;
    const int col = 16 * col_half + (i16 & 3) * 4;          // column within the block
    const int lp = col >> 3, inner = (col & 7) * 2;
    pv_base0a = r0 * kRowBytes + swz(lp, r0) * 16 + inner;
    pv_base0b = r0 * kRowBytes + swz(4 + lp, r0) * 16 + inner;
    pv_base1a = r1 * kRowBytes + swz(lp, r1) * 16 + inner;
    pv_base1b = r1 * kRowBytes + swz(4 + lp, r1) * 16 + inner;
  }
  // software pipeline: tile t+1 is in flight to the raw area, and the keys of tile t+2
  // are being read, while tile t computes
  // SHARE: a round is 64 keys = 4 tiles; lane l reports key l of the round, wavefront w fetches
  // tile w of the round into slot 4 * (round % 2) + w, and every wavefront computes on all four
  const int rounds = (n_tiles + kWaves - 1) / kWaves;
  auto round_keys = [&](int r) -> int { return r < rounds ? key_row(key_begin + r * (kWaves * kTile) + lane) : -1; };
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  int key_cur = SHARE ? round_keys(0) : tile_key(0);
  int key_nxt = SHARE ? round_keys(1) : tile_key(1);
  unsigned long long next_mask = 0ull;
  if (SHARE) {
    if (R576) {                                   // the first round passes through the registers as well
      dma_dst = smem + wave_u * kTileBytes;
      ksc_dst = reinterpret_cast<float*>(smem + kRowsKscOff) + kTile * wave_u;
      dma_on = rounds > 0;
      key_dma = key_cur;
      for (int j = 0; j < kWaves; ++j) {
        fetch_share(j);
        store_share(j);
      }
    } else if (rounds > 0) {
      issue_rows(key_cur, 16 * wave_u, smem + wave_u * kTileBytes);
    }
    next_mask = __ballot(key_cur >= 0);
  } else if (my_tiles > 0) {
    if (KV_FP8) issue_dma(key_cur);
    else issue_rows(key_cur, 0, tile);
  }
  const unsigned char* cur = tile;                // the tile being computed on
  unsigned long long round_mask = 0ull;           // SHARE: validity of the 64 keys of the round

  const int steps = SHARE ? rounds * kWaves : my_tiles;
  for (int t = 0; t < steps; ++t) {
    unsigned vmask;
    f32x4 ksc = {1.0f, 1.0f, 1.0f, 1.0f};
    if (SHARE) {
      const int r = t >> 2, j = t & 3;
      if (j == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's tile of round r has landed
        __syncthreads();                                   // ... so have the others'; round r-1 is read out
        round_mask = next_mask;
        key_dma = key_nxt;                                 // round r+1: its index words arrived with the wait above
        next_mask = __ballot(key_dma >= 0);
        key_nxt = round_keys(r + 2);
        dma_dst = smem + (((r + 1) & 1) * kWaves + wave_u) * kTileBytes;
        ksc_dst = reinterpret_cast<float*>(smem + kRowsKscOff) + (((r + 1) & 1) * kWaves + wave_u) * kTile;
        dma_on = r + 1 < rounds;
      }
      vmask = (unsigned)(round_mask >> (16 * j)) & 0xffffu;
      cur = smem + ((r & 1) * kWaves + j) * kTileBytes;
      if (TOK) ksc = *reinterpret_cast<const f32x4*>(smem + kRowsKscOff + (((r & 1) * kWaves + j) * kTile + 4 * (lane >> 4)) * 4);
      const bool idle = heads_here == 0 || vmask == 0u;    // no products in this step
      fetch_share(j);
      if (idle) {                                          // a wavefront without heads only fetches
        store_share(j);
        continue;
      }
    } else {
    vmask = (unsigned)(__ballot(key_cur >= 0) & 0xffffull);
    if (STAGED) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // tile t has landed in the raw area
      if (E8) {
#pragma unroll
        for (int i = 0; i < 3; ++i)
          if (lane + 64 * i < kTile * 9) *reinterpret_cast<unsigned short*>(raw_sc + (lane + 64 * i) * 2) = e8n[i];
      }
      stage();
      if (TOK) ksc = *reinterpret_cast<const f32x4*>(raw_sc + 16 * (lane >> 4));   // scales of keys 4 (lane / 16) + i
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // raw area fully read before it is refilled
      if (t + 1 < my_tiles) issue_dma(key_nxt);
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // tile t has landed
      cur = tile + (t & 1) * kTileBytes;
      // the other tile was last read by the products of tile t-1, whose results have been consumed
      if (t + 1 < my_tiles) issue_rows(key_nxt, 0, tile + ((t + 1) & 1) * kTileBytes);
    }
    key_cur = key_nxt;
    key_nxt = tile_key(t + 2);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (vmask == 0u) continue;                    // nothing to attend to in this tile (uniform)

    // ---- S^T = K . Q^T ------------------------------------------------------------
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    {
      // chunk 4ks+kq of row m: 128 bytes per pair of k-steps, low bits swizzled -> two lane bases
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        const bf16x8 a = lds_read_b128(cur, ((ks & 1) ? qk_base1 : qk_base0) + 128 * (ks >> 1));
        if (F16) {
          mfma_qk_f16(s0, a, qf[0][ks]);
          mfma_qk_f16(s1, a, qf[1][ks]);
        } else {
          mfma_qk(s0, a, qf[0][ks]);
          mfma_qk(s1, a, qf[1][ks]);
        }
      }
      mfma_settle(s0, s1);
    }
    // lane (n = lane%16, gq = lane/16) holds keys 4*gq + i of heads n (s0) and 16+n (s1)
    const int gq = lane >> 4;
    float sv[2][4];
    float mx[2] = {-INFINITY, -INFINITY};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = (vmask >> (4 * gq + i)) & 1u;
      sv[0][i] = ok ? s0[i] * (TOK ? sfac[0] * ksc[i] : qk_scale) : -INFINITY;
      sv[1][i] = ok ? s1[i] * (TOK ? sfac[1] * ksc[i] : qk_scale) : -INFINITY;
      mx[0] = fmaxf(mx[0], sv[0][i]);
      mx[1] = fmaxf(mx[1], sv[1][i]);
    }
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      mx[hh] = fmaxf(mx[hh], xor16(mx[hh]));
      mx[hh] = fmaxf(mx[hh], xor32(mx[hh]));
    }
    // lazy running reference: move it only when the tile maximum exceeds it by more than kLazy
    const bool grow = (mx[0] > m_run[0] + kLazy) || (mx[1] > m_run[1] + kLazy);
    if (__ballot(grow) != 0ull) {
      float fac[2];
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const float m_new = (mx[hh] > m_run[hh] + kLazy) ? mx[hh] : m_run[hh];
        fac[hh] = (m_run[hh] == -INFINITY) ? 0.0f : exp2f(m_run[hh] - m_new);
        l_run[hh] *= fac[hh];
        m_run[hh] = m_new;
      }
      // accumulator lane l carries head l%32: half (l & 16)
      const float fo = (lane & 16) ? fac[1] : fac[0];
      if (__ballot(fo != 1.0f) != 0ull) {
        mfma_settle_acc(o);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          // one 16-register block at a time: the accumulators pass through ordinary
          // VGPRs for the multiply and only a few of those are free
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int j = 0; j < 16; ++j) o[i][j] *= fo;
          asm volatile("" : "+a"(o[i]));      // back into the accumulation registers right away
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma_settle_acc(o);
      }
    }
    unsigned pk[2][2];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      float pr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pr[i] = exp2f(sv[hh][i] - m_run[hh]);      // -inf -> 0; m_run is finite once any key was valid
        l_run[hh] += pr[i];
        if (TOK) pr[i] *= ksc[i];                  // V = scale x codes
      }
      pk[hh][0] = F16 ? pack_f16(pr[0], pr[1]) : pack_bf16(pr[0], pr[1]);
      pk[hh][1] = F16 ? pack_f16(pr[2], pr[3]) : pack_bf16(pr[2], pr[3]);
    }
    // P^T as the B operand of 32x32x16: lane (head = lane%32, kq = lane/32) needs keys 8kq..8kq+7
    bf16x8 pb;
    {
      const u32x2 w0 = __builtin_amdgcn_permlane16_swap(pk[0][0], pk[1][0], false, false);
      const u32x2 w1 = __builtin_amdgcn_permlane16_swap(pk[0][1], pk[1][1], false, false);
      const uint4 packed = make_uint4(w0[0], w1[0], w0[1], w1[1]);
      pb = __builtin_bit_cast(bf16x8, packed);
    }
    // ---- O^T += V^T . P^T ---------------------------------------------------------
#pragma unroll
    for (int db = 0; db < 16; ++db) {
      const int off = 128 * (db >> 1);
      const bf16x4 a0 = lds_read_tr16_b64(cur + ((db & 1) ? pv_base0b : pv_base0a) + off);
      const bf16x4 a1 = lds_read_tr16_b64(cur + ((db & 1) ? pv_base1b : pv_base1a) + off);
      bf16x8 a;
      a[0] = a0[0]; a[1] = a0[1]; a[2] = a0[2]; a[3] = a0[3];
      a[4] = a1[0]; a[5] = a1[1]; a[6] = a1[2]; a[7] = a1[3];
      if (F16) mfma_pv_f16(o[db], a, pb);
      else mfma_pv(o[db], a, pb);
      // keep the scheduler from hoisting every fragment read of the loop to its top: the
      // query fragments need the registers
      if ((db & 7) == 7) __builtin_amdgcn_sched_barrier(0);
    }
    if (SHARE) store_share(t & 3);
  }

  // ---- merge the four wavefronts ----------------------------------------------------
  mfma_settle_acc(o);
  // denominators: a head's share is spread over lanes n, n+16, n+32, n+48
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {
    l_run[hh] += __shfl_xor(l_run[hh], 16, 64);
    l_run[hh] += __shfl_xor(l_run[hh], 32, 64);
  }
  __syncthreads();                               // every wavefront is done with its tile
  // SHARE: the wavefronts hold different heads, nothing is merged - the same path with the sums
  // over wavefronts reduced to the wavefront's own entry serves as the transpose to channel order
  float* stats = reinterpret_cast<float*>(smem + (STAGED ? kStatOff : kRowsStatOff));
  if (lane < 16) {
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      stats[(wave * kHeads + hh * 16 + lane) * 2 + 0] = m_run[hh];
      stats[(wave * kHeads + hh * 16 + lane) * 2 + 1] = l_run[hh];
    }
  }
  __syncthreads();
  // accumulator lane carries head hd = lane%32
  const int hd = lane & 31;
  float m_all = -INFINITY;
#pragma unroll
  for (int w = 0; w < kWaves; ++w)
    if (!SHARE || w == wave) m_all = fmaxf(m_all, stats[(w * kHeads + hd) * 2]);
  float l_all = 0.0f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    if (SHARE && w != wave) continue;
    const float mw = stats[(w * kHeads + hd) * 2];
    l_all += (mw == -INFINITY) ? 0.0f : stats[(w * kHeads + hd) * 2 + 1] * exp2f(mw - m_all);
  }
  {
    const float mine = stats[(wave * kHeads + hd) * 2];
    const float f = (mine == -INFINITY) ? 0.0f : exp2f(mine - m_all);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 16; ++j) o[i][j] *= f;
      asm volatile("" : "+a"(o[i]));
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // final scale for a single-split launch: fold the sink in and normalise
  float out_scale = 1.0f, lse_val = 0.0f;
  const bool direct = p.num_splits == 1;
  if (direct) {
    float m_fin = m_all, l_fin = l_all;
    if (mla_has_sinks(p) && hd < heads_here) {
      const float sk = p.sinks[head0 + hd] * kLog2e;
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

  float* xbuf = reinterpret_cast<float*>(smem);
  const size_t q_index = bs;                     // b*S + s
  // two rounds of 256 value channels each
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    __syncthreads();
    // writer: lane (head hd, gq = lane/32) holds channels 32*db + 8*j + 4*gq + (0..3) in o[db][4j..4j+3]
    {
      const int gq2 = lane >> 5;
#pragma unroll
      for (int dbl = 0; dbl < 8; ++dbl) {
        const int db = half * 8 + dbl;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int ch = 32 * dbl + 8 * j + 4 * gq2;      // channel within this half
          float4 v = make_float4(o[db][4 * j], o[db][4 * j + 1], o[db][4 * j + 2], o[db][4 * j + 3]);
          *reinterpret_cast<float4*>(xbuf + (wave * kHeads + hd) * kXPitch + ch) = v;
        }
      }
    }
    __syncthreads();
    // reader: wavefront w sums heads 8w..8w+7 (SHARE: reads back its own 32); lane = 4 consecutive channels
#pragma unroll 8
    for (int hh = 0; hh < (SHARE ? kHeads : 8); ++hh) {
      const int h = SHARE ? hh : wave * 8 + hh;
      if (h >= heads_here) break;                // uniform
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        if (SHARE && w != wave) continue;
        const float4 v = *reinterpret_cast<const float4*>(xbuf + (w * kHeads + h) * kXPitch + lane * 4);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
      }
      const int ch = half * 256 + lane * 4;
      if (direct) {
        const float sc = __shfl(out_scale, h, 64);   // lane h carries head h
        const size_t off = (q_index * p.H + head0 + h) * (size_t)kLat + ch;
        if (p.out_dtype == CPPMEGA_MI355_F32) {
          *reinterpret_cast<float4*>((float*)p.out + off) = make_float4(acc.x * sc, acc.y * sc, acc.z * sc, acc.w * sc);
        } else if (p.out_dtype == CPPMEGA_MI355_BF16) {
          *reinterpret_cast<uint2*>((unsigned short*)p.out + off) =
              make_uint2(pack_bf16(acc.x * sc, acc.y * sc), pack_bf16(acc.z * sc, acc.w * sc));
        } else {
          unsigned short* dst = (unsigned short*)p.out + off;
          dst[0] = f32_to_f16_bits(acc.x * sc); dst[1] = f32_to_f16_bits(acc.y * sc);
          dst[2] = f32_to_f16_bits(acc.z * sc); dst[3] = f32_to_f16_bits(acc.w * sc);
        }
      } else {
        // partial: [query][head][split][512] fp32
        float* part = (float*)p.workspace + ((q_index * p.H + head0 + h) * (size_t)p.num_splits + split) * kLat + ch;
        *reinterpret_cast<float4*>(part) = acc;
      }
    }
  }
  if ((SHARE || wave == 0) && lane < heads_here) {
    if (direct) {
      if (p.lse) p.lse[q_index * p.H + head0 + lane] = lse_val;
    } else {
      float* ml = (float*)p.workspace + (size_t)p.B * p.S * p.H * p.num_splits * kLat +
                  ((q_index * p.H + head0 + lane) * (size_t)p.num_splits + split) * 2;
      ml[0] = m_all;
      ml[1] = l_all;
    }
  }
}

// Merges the key splits of every (query, head): one wavefront per (query, head).
__global__ __launch_bounds__(256) void sparse_mla_combine_kernel(const MlaParams p) {
  const int lane = lane_id();
  const size_t qh = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (qh >= (size_t)p.B * p.S * p.H) return;
  const int h = (int)(qh % p.H);
  const float* part = (const float*)p.workspace + qh * (size_t)p.num_splits * kLat;
  const float* ml = (const float*)p.workspace + (size_t)p.B * p.S * p.H * p.num_splits * kLat + qh * (size_t)p.num_splits * 2;
  float m_all = -INFINITY;
  for (int s = 0; s < p.num_splits; ++s) m_all = fmaxf(m_all, ml[2 * s]);
  float m_fin = m_all;
  float sink_term = 0.0f;
  if (mla_has_sinks(p)) {
    const float sk = p.sinks[h] * kLog2e;
    m_fin = fmaxf(m_all, sk);
    sink_term = exp2f(sk - m_fin);
  }
  float l_fin = sink_term;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
  for (int s = 0; s < p.num_splits; ++s) {
    const float ms = ml[2 * s];
    if (ms == -INFINITY) continue;
    const float f = exp2f(ms - m_fin);
    l_fin += ml[2 * s + 1] * f;
    const float4 a = *reinterpret_cast<const float4*>(part + (size_t)s * kLat + lane * 8);
    const float4 c = *reinterpret_cast<const float4*>(part + (size_t)s * kLat + lane * 8 + 4);
    acc[0] += a.x * f; acc[1] += a.y * f; acc[2] += a.z * f; acc[3] += a.w * f;
    acc[4] += c.x * f; acc[5] += c.y * f; acc[6] += c.z * f; acc[7] += c.w * f;
  }
  const float inv = l_fin > 0.0f ? 1.0f / l_fin : 0.0f;
  const size_t off = qh * (size_t)kLat + lane * 8;
  if (p.out_dtype == CPPMEGA_MI355_BF16) {
    *reinterpret_cast<uint4*>((unsigned short*)p.out + off) =
        make_uint4(pack_bf16(acc[0] * inv, acc[1] * inv), pack_bf16(acc[2] * inv, acc[3] * inv),
                   pack_bf16(acc[4] * inv, acc[5] * inv), pack_bf16(acc[6] * inv, acc[7] * inv));
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) store_as(p.out, off + i, p.out_dtype, acc[i] * inv);
  }
  if (p.lse && lane == 0) p.lse[qh] = l_fin > 0.0f ? (m_fin + log2f(l_fin)) * kLn2 : 0.0f;
}

}  // namespace

bool sparse_mla_mfma_supported(const MlaParams& p) {
  if (sparse_mla_latent_supported(p)) return true;
  if (p.q_dtype == CPPMEGA_MI355_E4M3) {          // FP8 prepared buffers: rows of 576 codes, both sides scaled alike
    const bool tok = p.q_scale_kind == CPPMEGA_MI355_SCALE_PER_TOKEN && p.kv_scale_kind == CPPMEGA_MI355_SCALE_PER_TOKEN &&
                     (((uintptr_t)p.q_scale | (uintptr_t)p.kv_scale) & 3) == 0;
    const bool e8 = p.q_scale_kind == CPPMEGA_MI355_SCALE_E8M0 && p.kv_scale_kind == CPPMEGA_MI355_SCALE_E8M0 &&
                    p.q_scale_block == 32 && p.kv_scale_block == 32 && ((uintptr_t)p.kv_scale & 1) == 0;
    return (tok || e8) && p.kv_dtype == CPPMEGA_MI355_E4M3 && p.d_qk == kDqk && p.d_kv == kDqk && p.d_v == kLat &&
           p.rope_dim == 0 && p.q_scale && p.kv_scale && p.topk >= 1 && (size_t)p.B * p.S != 0 &&
           (((uintptr_t)p.q | (uintptr_t)p.kv) & 15) == 0;
  }
  const bool f16 = p.q_dtype == CPPMEGA_MI355_F16;
  if ((p.q_dtype != CPPMEGA_MI355_BF16 && !f16) || p.q_scale_kind != CPPMEGA_MI355_SCALE_NONE) return false;
  if (p.d_qk != kDqk || p.d_v != kLat) return false;
  if (p.rope_dim != 0 && (p.rope_dim != kRope || p.rope_dtype != p.q_dtype)) return false;
  // float16 queries only with float16 rows: a dequantised e4m3 row can leave float16's range
  if (f16 && p.kv_dtype != CPPMEGA_MI355_F16) return false;
  if (p.kv_dtype == CPPMEGA_MI355_E4M3) {
    if (p.rope_dim != kRope || p.d_kv != kLat) return false;
    if (p.kv_scale_kind == CPPMEGA_MI355_SCALE_F32_BLOCK) {
      if (p.kv_scale_block < kLat / kMaxBlocks || kLat % p.kv_scale_block != 0) return false;
    } else if (p.kv_scale_kind != CPPMEGA_MI355_SCALE_PER_TOKEN && p.kv_scale_kind != CPPMEGA_MI355_SCALE_NONE) {
      return false;
    }
  } else if (p.kv_dtype == p.q_dtype) {
    if (p.kv_scale_kind != CPPMEGA_MI355_SCALE_NONE) return false;
    if (p.d_kv + p.rope_dim != kDqk) return false;
  } else {
    return false;
  }
  if (p.topk < 1 || (size_t)p.B * p.S == 0) return false;
  // pointers must allow 16-byte loads
  if (((uintptr_t)p.q | (uintptr_t)p.kv | (uintptr_t)p.rope) & 15) return false;
  return true;
}

// Chooses the key-split factor: enough workgroups to cover the 256 CUs, at least 64 keys per wavefront.
void sparse_mla_mfma_plan(MlaParams& p) {
  p.heads_per_wg = 0;
  p.tile_sharing = 0;
  if (sparse_mla_latent_supported(p)) {
    sparse_mla_latent_plan(p);
    return;
  }
  const int groups_per_kv = (p.heads_per_group + kHeads - 1) / kHeads;
  // 16-bit rows with several head groups per KV group: the wavefronts share one key stream
  // (with two head groups two wavefronts only fetch and it still wins: 4.2 ms against 4.7 ms at
  // 64 heads x 4096 queries x 2048 keys)
  p.tile_sharing = (p.kv_dtype != CPPMEGA_MI355_E4M3 || p.q_dtype == CPPMEGA_MI355_E4M3) && groups_per_kv >= 2;
  const int units = p.tile_sharing ? (groups_per_kv + kWaves - 1) / kWaves : groups_per_kv;
  const long long base = (long long)p.B * p.S * p.G * units;
  int splits = 1;
  while (base * splits < 256 && p.topk / (splits * 2) >= kWaves * 64 && splits < 16) splits *= 2;
  p.num_splits = splits;
  const int tiles = (p.topk + kTile - 1) / kTile;
  const int tiles_per_split = (tiles + splits - 1) / splits;
  p.keys_per_split = tiles_per_split * kTile;
}

size_t sparse_mla_mfma_workspace_bytes(const MlaParams& p) {
  if (p.heads_per_wg != 0) return sparse_mla_latent_workspace_bytes(p);
  if (p.num_splits <= 1) return 0;
  return (size_t)p.B * p.S * p.H * p.num_splits * (kLat + 2) * sizeof(float);
}

int sparse_mla_mfma_launch(const MlaParams& p, hipStream_t stream) {
  if (p.heads_per_wg != 0) return sparse_mla_latent_launch(p, stream);
  const int groups_per_kv = (p.heads_per_group + kHeads - 1) / kHeads;
  const int units = p.tile_sharing ? (groups_per_kv + kWaves - 1) / kWaves : groups_per_kv;
  const dim3 grid((unsigned)((size_t)p.B * p.S * p.G * units), (unsigned)p.num_splits), block(kWaves * 64);
  void (*kernel)(MlaParams) = nullptr;
  int smem = kRowsSmemBytes;
  if (p.kv_dtype == CPPMEGA_MI355_E4M3) {
    const bool e8 = p.q_scale_kind == CPPMEGA_MI355_SCALE_E8M0;
    if (p.q_dtype != CPPMEGA_MI355_E4M3) kernel = sparse_mla_mfma_kernel<true>;
    else if (p.tile_sharing) kernel = e8 ? sparse_mla_mfma_kernel<true, false, true, 2> : sparse_mla_mfma_kernel<true, false, true, 1>;
    else kernel = e8 ? sparse_mla_mfma_kernel<true, false, false, 2> : sparse_mla_mfma_kernel<true, false, false, 1>;
    smem = p.tile_sharing ? kRowsFp8SmemBytes : kSmemBytes;
  } else if (p.kv_dtype == CPPMEGA_MI355_F16) {
    kernel = p.tile_sharing ? sparse_mla_mfma_kernel<false, true, true> : sparse_mla_mfma_kernel<false, true, false>;
  } else {
    kernel = p.tile_sharing ? sparse_mla_mfma_kernel<false, false, true> : sparse_mla_mfma_kernel<false, false, false>;
  }
  CM_HIP_CHECK(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
  hipLaunchKernelGGL(kernel, grid, block, smem, stream, p);
  CM_HIP_CHECK(hipGetLastError());
  if (p.num_splits > 1) {
    const size_t qh = (size_t)p.B * p.S * p.H;
    hipLaunchKernelGGL(sparse_mla_combine_kernel, dim3((unsigned)((qh + 3) / 4)), dim3(256), 0, stream, p);
    CM_HIP_CHECK(hipGetLastError());
  }
  return 0;
}

}  // namespace cm
