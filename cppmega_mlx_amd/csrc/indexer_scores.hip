// Indexer scores -> top-k (gfx950).
//
// The tail of the reference's LightningIndexer.__call__ (cppmega_v4/nn/lightning_indexer.py:132-145,
// the same lines in cppmega_v4/nn/lightning_indexer_fp8.py:145-157):
//
//   scores[b,s,t] = sm_scale * sum_h weights[b,s,h] * sum_d q[b,s,h,d] * k[b,t,d]   (+ mask[b,s,t])
//   indices[b,s,:] = top-k of scores[b,s,:]
//
// No nonlinearity sits between the head sum and the key product, so the head sum is taken first:
// qw[b,s,:] = sum_h weights[b,s,h] * q[b,s,h,:] (fp32), and a score is one dot product of length D.
// That turns H*D multiply-adds per (query, key) into D and makes the key product a plain matrix
// product of a 16-query tile with the key rows, which runs on the matrix cores:
//
//   * indexer_qw_kernel forms qw once per query row in fp32 (q is read exactly once) and stores it
//     as two bf16 planes, hi and lo = bf16(qw - hi): hi + lo carries 16 significand bits;
//   * indexer_scores_kernel: a workgroup (4 wavefronts) owns 16 query rows of one batch and a
//     range of keys, with the 16 qw rows in LDS.  Each wavefront walks its keys 64 at a time.  The
//     keys are the MFMA's A rows, loaded straight from memory (bf16 rows as they are; fp32 rows
//     split into hi + lo as well), the queries its B columns: v_mfma_f32_16x16x32_bf16 products
//     k*hi + k*lo (+ k_lo*hi) into fp32 accumulators.  The A rows are numbered so that a lane ends
//     up with 16 consecutive keys of one query and writes them as four 16-byte stores;
//     score = acc * sm_scale (+ mask);
//   * scores go to a float32 buffer and the radix-select kernel of topk_select.hip picks the
//     indices.  Rows are scored and selected a chunk at a time (256 MiB of scores by default:
//     on this machine larger passes measured faster than cache-sized ones, 232 us against
//     295 us at 64 MiB for 8192 x 8192), which bounds the workspace; the full [B, Sq, Skv]
//     score matrix is only written when the caller asks for it.
//
// Sums are taken in an order that differs from an einsum's, so scores agree with a float64
// evaluation to rounding (about 2^-16 relative to sum |qw*k|), not bit for bit; with the scores
// given, the selection is exact (value descending, ties toward the lower index).

#include <string.h>

#include "common.h"

namespace cm {

int topk_select_launch(const cppmega_mi355_topk_args_t& a, hipStream_t stream);
int topk_workspace_bytes(const cppmega_mi355_topk_args_t& a, size_t* bytes);

namespace {

constexpr int kQRows = 16;          // query rows per workgroup (one MFMA tile)
constexpr int kMaxD = 256;          // widest head the LDS tile is sized for
constexpr int kPitch = kMaxD + 8;   // bf16 elements per LDS row (16 bytes of padding)
constexpr int kThreads = 256;
constexpr int kKeysPerIter = 4 * 64;   // 4 wavefronts x 4 tiles x 16 keys

struct IndexerParams {
  const void* q;
  const void* w;
  const void* k;
  const void* mask;
  float* scores;             // row (b - b_begin) * s_count + (s - s_begin), pitch Skv
  unsigned short* qw;        // [2][rows of the pass][Dp] bf16: hi plane, then lo plane
  int q_dtype, w_dtype, k_dtype, mask_dtype;
  int B, Sq, H, D, Skv;
  int b_begin, nb, s_begin, s_count;
  int keys_per_wg;           // multiple of kKeysPerIter
  int q_vec, k_vec, s_vec;   // 16-byte accesses allowed for q rows / k rows / score rows
  // Selection bounds of the pass's rows (row (b - b_begin) * s_count + (s - s_begin); null = none).
  // A workgroup scores only the keys some row of its query tile can select: under a causal bound
  // that is half the matrix.  Not used when the caller asked for the whole score matrix.
  const int* starts;
  const int* ends;
  float sm_scale;
};

__device__ __forceinline__ void split_bf16(float v, unsigned short& hi, unsigned short& lo) {
  hi = f32_to_bf16_bits(v);
  lo = f32_to_bf16_bits(v - bf16_bits_to_f32(hi));
}

// qw[row, :] = sum_h w[row, h] * q[row, h, :] in fp32, stored as bf16 hi + lo planes padded to Dp.
// One workgroup per query row: thread (c, hg) takes 8 channels and every hgroups-th head, so a
// row's H*D values arrive as independent 16-byte loads; the head groups meet in LDS.  q is read
// exactly once.
__global__ __launch_bounds__(kThreads) void indexer_qw_kernel(const IndexerParams p) {
  __shared__ float part[kThreads][9];
  const int D = p.D, H = p.H;
  const int Dp = (D + 31) & ~31;
  const int chunks = Dp / 8;                      // <= 32
  const int hgroups = kThreads / chunks;          // >= 8
  const int rows = p.nb * p.s_count;
  const int r = (int)blockIdx.x;
  const int tid = (int)threadIdx.x;
  const int c = tid % chunks, hg = tid / chunks;
  const size_t row = (size_t)(p.b_begin + r / p.s_count) * p.Sq + (size_t)(p.s_begin + r % p.s_count);
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (hg < hgroups) {
    if (p.q_vec) {
      if (8 * c < D) {
        const uint4* src = reinterpret_cast<const uint4*>((const unsigned short*)p.q + row * H * D + 8 * c);
#pragma unroll 8
        for (int h = hg; h < H; h += hgroups) {
          const float wh = load_as(p.w, row * H + h, p.w_dtype);
          const uint4 t = src[(size_t)h * (D / 8)];
          const unsigned u[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            acc[2 * i] = fmaf(wh, __uint_as_float(u[i] << 16), acc[2 * i]);
            acc[2 * i + 1] = fmaf(wh, __uint_as_float(u[i] & 0xffff0000u), acc[2 * i + 1]);
          }
        }
      }
    } else {
      for (int h = hg; h < H; h += hgroups) {
        const float wh = load_as(p.w, row * H + h, p.w_dtype);
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (8 * c + i < D) acc[i] = fmaf(wh, load_as(p.q, (row * H + h) * D + 8 * c + i, p.q_dtype), acc[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) part[tid][i] = acc[i];
  __syncthreads();
  if (tid >= chunks) return;
  for (int g = 1; g < hgroups; ++g) {             // fixed order: the result does not depend on timing
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += part[g * chunks + tid][i];
  }
  unsigned short hi[8], lo[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) split_bf16(acc[i], hi[i], lo[i]);
  const size_t at = (size_t)r * Dp + 8 * tid;
  *reinterpret_cast<uint4*>(p.qw + at) = make_uint4(hi[0] | ((unsigned)hi[1] << 16), hi[2] | ((unsigned)hi[3] << 16),
                                                    hi[4] | ((unsigned)hi[5] << 16), hi[6] | ((unsigned)hi[7] << 16));
  *reinterpret_cast<uint4*>(p.qw + (size_t)rows * Dp + at) =
      make_uint4(lo[0] | ((unsigned)lo[1] << 16), lo[2] | ((unsigned)lo[3] << 16), lo[4] | ((unsigned)lo[5] << 16),
                 lo[6] | ((unsigned)lo[7] << 16));
}

// The same head sum with one wavefront per query row, for bf16 rows whose padded width is 32, 64,
// 128 or 256 channels: a load instruction fetches 1 KiB of the row (64 / chunks heads, neighbouring
// lanes neighbouring 16 bytes), sixteen of them in flight per lane; the lanes that hold the same
// channels of different heads meet through lane exchanges in a fixed order.  No LDS, no barrier:
// a row is a 16 KiB stream at 64 heads of 128 channels, and a CU keeps 32 of them in flight.
// q is read once, so the loads are non-temporal: with ordinary loads the same kernel streams
// 128 MiB of query rows at 2.9 TB/s (the lines it allocates in the caches displace each other),
// with the hint at 5.1 TB/s.
constexpr int kQwWaves = 4;
__device__ __forceinline__ uint4 load_once(const uint4* src) {
  typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src));
  return make_uint4(t[0], t[1], t[2], t[3]);
}
// WDT: the dtype of the head weights, a template argument: behind a run-time dtype test every weight
// load sits in a basic block of its own and the sixteen loads of a round are waited for one after
// the other (11 us for the 32 rows of a decode step, against 3 us).
template <int WDT>
__global__ __launch_bounds__(kQwWaves * 64) void indexer_qw_wave_kernel(const IndexerParams p) {
  const int D = p.D, H = p.H;
  const int Dp = (D + 31) & ~31;
  const int chunks = Dp / 8;                      // 4, 8, 16 or 32 lanes per head
  const int hp = 64 / chunks;                     // heads per load instruction
  const int rows = p.nb * p.s_count;
  const int lane = (int)threadIdx.x & 63;
  const int r = (int)blockIdx.x * kQwWaves + ((int)threadIdx.x >> 6);
  if (r >= rows) return;
  const int c = lane & (chunks - 1), hs = lane / chunks;
  const size_t row = (size_t)(p.b_begin + r / p.s_count) * p.Sq + (size_t)(p.s_begin + r % p.s_count);
  const bool live = 8 * c < D;
  const uint4* src = reinterpret_cast<const uint4*>((const unsigned short*)p.q + row * H * D + 8 * (live ? c : 0));
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  auto add = [&](const uint4& t, float wh) {
    const unsigned u[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[2 * i] = fmaf(wh, __uint_as_float(u[i] << 16), acc[2 * i]);
      acc[2 * i + 1] = fmaf(wh, __uint_as_float(u[i] & 0xffff0000u), acc[2 * i + 1]);
    }
  };
  int h = hs;
  for (; h + 15 * hp < H; h += 16 * hp) {         // sixteen loads in flight
    uint4 t[16];
    float wh[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      t[j] = load_once(src + (size_t)(h + j * hp) * (D / 8));
      wh[j] = load_as(p.w, row * H + h + j * hp, WDT);
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) add(t[j], wh[j]);
  }
  for (; h < H; h += hp) add(load_once(src + (size_t)h * (D / 8)), load_as(p.w, row * H + h, WDT));
  for (int off = 32; off >= chunks; off >>= 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += __shfl_xor(acc[i], off, 64);
  }
  if (lane >= chunks) return;
  unsigned short hi[8], lo[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) split_bf16(live ? acc[i] : 0.0f, hi[i], lo[i]);
  const size_t at = (size_t)r * Dp + 8 * c;
  *reinterpret_cast<uint4*>(p.qw + at) = make_uint4(hi[0] | ((unsigned)hi[1] << 16), hi[2] | ((unsigned)hi[3] << 16),
                                                    hi[4] | ((unsigned)hi[5] << 16), hi[6] | ((unsigned)hi[7] << 16));
  *reinterpret_cast<uint4*>(p.qw + (size_t)rows * Dp + at) =
      make_uint4(lo[0] | ((unsigned)lo[1] << 16), lo[2] | ((unsigned)lo[3] << 16), lo[4] | ((unsigned)lo[5] << 16),
                 lo[6] | ((unsigned)lo[7] << 16));
}

// Keys are the MFMA's A rows and 16 queries its B columns: lane (n, kg) holds C rows
// 4 kg .. 4 kg + 3 of tile j, i.e. four consecutive keys key0 + 16 j + 4 kg + i of query n, and
// writes them as one 16-byte store; the four lanes of a query cover 64 contiguous bytes.
// A workgroup holds QT query tiles (16 QT rows): every key fragment it loads is used for all of them.
// STAGED (bf16 keys whose rows are exactly 32 KSTEPS channels, Skv a multiple of 4): the 64 keys of a
// wavefront step are one contiguous piece of memory and are fetched as such - neighbouring lanes,
// neighbouring 16 bytes; loads whose lanes each point into another row move a quarter of the bytes
// per clock - and pass through a private LDS tile (32 rows at a time, 16-byte slots XOR-swizzled by
// the row) on their way to operand order.  The finished 16 x 64 score tiles take the same way back:
// through the LDS tile into stores of whole 256-byte row segments, with the mask read the same way.
constexpr int kStageBytes = 32 * 2 * kMaxD / 2;    // 8 KB per wavefront: 32 key rows of 256 bytes, or a 16 x 64 float tile (+ padding)
constexpr int kCPitch = 68;                        // floats per row of the score tile in LDS (64 + 4: rows on distinct banks)
static_assert(16 * kCPitch * 4 <= kStageBytes, "the score tile reuses the key tile");

template <bool K_F32, int KSTEPS, int QT, bool STAGED = false>
__global__ __launch_bounds__(kThreads, 2) void indexer_scores_kernel(const IndexerParams p) {
  extern __shared__ __align__(16) unsigned short q_lds[];     // [2][16 QT][Dp + 8]: hi plane, lo plane; then the staging tiles
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bz = (int)blockIdx.z;
  const int b = p.b_begin + bz;
  const int s_off = kQRows * QT * (int)blockIdx.y;            // first query row of the workgroup within the pass
  const int rows_here = min(kQRows * QT, p.s_count - s_off);
  const int D = p.D;
  const int Dp = (D + 31) & ~31;
  const int pitch = Dp + 8;
  const int ksteps = KSTEPS > 0 ? KSTEPS : Dp / 32;
  const size_t out_row0 = (size_t)bz * p.s_count + (size_t)s_off;
  unsigned short* q_hi = q_lds;
  unsigned short* q_lo = q_lds + kQRows * QT * pitch;

  {  // the workgroup's qw rows -> LDS
    const int chunks = Dp / 8;
    const size_t plane = (size_t)p.nb * p.s_count * Dp;
    for (int e = tid; e < kQRows * QT * chunks; e += kThreads) {
      const int r = e / chunks, c = e % chunks;
      uint4 h4 = make_uint4(0u, 0u, 0u, 0u), l4 = h4;
      if (r < rows_here) {
        const size_t at = (out_row0 + r) * Dp + 8 * c;
        h4 = *reinterpret_cast<const uint4*>(p.qw + at);
        l4 = *reinterpret_cast<const uint4*>(p.qw + plane + at);
      }
      *reinterpret_cast<uint4*>(&q_hi[r * pitch + 8 * c]) = h4;
      *reinterpret_cast<uint4*>(&q_lo[r * pitch + 8 * c]) = l4;
    }
  }
  __syncthreads();

  const int n = lane & 15, kg = lane >> 4;
  int key_begin = (int)blockIdx.x * p.keys_per_wg;
  int key_end = min(p.Skv, key_begin + p.keys_per_wg);
  if (p.starts || p.ends) {                            // (rows_here <= 64: a lane per row, every wavefront the same)
    int lo = lane < rows_here && p.starts ? p.starts[out_row0 + lane] : (lane < rows_here ? 0 : p.Skv);
    int hi = lane < rows_here ? (p.ends ? p.ends[out_row0 + lane] : p.Skv) : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      lo = min(lo, __shfl_xor(lo, off, 64));
      hi = max(hi, __shfl_xor(hi, off, 64));
    }
    lo = max(lo, 0);
    if (lo > key_begin) key_begin += (lo - key_begin) / kKeysPerIter * kKeysPerIter;
    key_end = min(key_end, (hi + 63) & ~63);
  }
  // bf16 keys with 16-byte loads: the next 64 keys are requested before the current ones are used
  constexpr bool kPrefetch = !K_F32 && KSTEPS > 0;
  constexpr int kBuf = kPrefetch ? KSTEPS : 1;
  uint4 cur[kBuf][4], nxt[kBuf][4];
  auto fetch = [&](int key0, uint4 (&buf)[kBuf][4]) {
#pragma unroll
    for (int ks = 0; ks < kBuf; ++ks) {
      const int d0 = 32 * ks + 8 * kg;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = min(key0 + 16 * j + n, p.Skv - 1);   // clamped: keys past the end are never stored
        buf[ks][j] = make_uint4(0u, 0u, 0u, 0u);
        if (d0 < D) buf[ks][j] = *reinterpret_cast<const uint4*>((const unsigned short*)p.k + ((size_t)b * p.Skv + (size_t)key) * D + d0);
      }
    }
  };
  if constexpr (STAGED) {
    constexpr int PPR = 4 * KSTEPS;                      // 16-byte pieces per key row (4, 8 or 16)
    constexpr int RP = 16 / PPR;                         // rows per 256 bytes
    constexpr int NT = 4 * KSTEPS;                       // pieces per lane of a 64-key step
    unsigned char* stage = reinterpret_cast<unsigned char*>(q_lds + 2 * kQRows * QT * pitch) + wave * kStageBytes;
    float* ctile = reinterpret_cast<float*>(stage);
    typedef __attribute__((ext_vector_type(4))) unsigned u4;
    u4 kc[NT], kn[NT];
    auto fetch_rows = [&](int key0, u4 (&buf)[NT]) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int P = lane + 64 * t, row = P / PPR, c = P % PPR;
        const int key = min(key0 + row, p.Skv - 1);      // clamped: keys past the end are never stored
        const u4* src = reinterpret_cast<const u4*>((const unsigned short*)p.k + ((size_t)b * p.Skv + (size_t)key) * D + 8 * c);
        // one query tile per workgroup is the decode-time shape: every key row is read by one workgroup,
        // once (non-temporal: 132 -> 121 us at 32 x 65536 keys); with more tiles the workgroups of a
        // batch share the keys through the cache
        buf[t] = QT == 1 ? __builtin_nontemporal_load(src) : *src;
      }
    };
    int a_off[2][KSTEPS];                                // operand order inside a 32-row half: tile jj, step ks
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int row = 16 * jj + n, c = 4 * ks + kg;
        a_off[jj][ks] = (row * PPR + (c ^ ((row / RP) % PPR))) * 16;
      }
    // The query operands do not change over the keys: they are read from LDS once (64 registers at
    // two query tiles of 128 channels).  Two tiles and not four: the kernel then fits 256 registers,
    // two workgroups share a CU, and one's matrix products run under the other's fetches, staging
    // and stores - 56 us at 8192 x 8192 under a causal bound against 71 us for four tiles in 380
    // registers (one workgroup per CU) and 76 us for four tiles with the operands read in the loop.
    // (One query tile - the decode-time shape, bound by the key stream - keeps reading them from LDS.)
    constexpr bool kHoist = QT > 1;
    bf16x8 bq[kHoist ? QT : 1][kHoist ? KSTEPS : 1][2];
    if constexpr (kHoist) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const int d0 = 32 * ks + 8 * kg;
          bq[qt][ks][0] = *reinterpret_cast<const bf16x8*>(&q_hi[(16 * qt + n) * pitch + d0]);
          bq[qt][ks][1] = *reinterpret_cast<const bf16x8*>(&q_lo[(16 * qt + n) * pitch + d0]);
        }
    }
    if (key_begin + 64 * wave < key_end) fetch_rows(key_begin + 64 * wave, kc);
    for (int key0 = key_begin + 64 * wave; key0 < key_end; key0 += kKeysPerIter) {
      f32x4 acc[QT][4];
#pragma unroll
      for (int qt = 0; qt < QT; ++qt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[qt][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      if (key0 + kKeysPerIter < key_end) fetch_rows(key0 + kKeysPerIter, kn);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        // rows 32 half .. 32 half + 31 of the step: registers -> LDS in load order (slot swizzled by the row)
#pragma unroll
        for (int t = 0; t < NT / 2; ++t) {
          const int P = lane + 64 * t, row = P / PPR, c = P % PPR;      // position within the half
          *reinterpret_cast<u4*>(stage + (row * PPR + (c ^ ((row / RP) % PPR))) * 16) = kc[half * (NT / 2) + t];
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int j = 2 * half + jj;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) {
            const bf16x8 ka = *reinterpret_cast<const bf16x8*>(stage + a_off[jj][ks]);
#pragma unroll
            for (int qt = 0; qt < QT; ++qt) {
              bf16x8 b_hi, b_lo;
              if constexpr (kHoist) {
                b_hi = bq[qt][ks][0];
                b_lo = bq[qt][ks][1];
              } else {
                const int d0 = 32 * ks + 8 * kg;
                b_hi = *reinterpret_cast<const bf16x8*>(&q_hi[(16 * qt + n) * pitch + d0]);
                b_lo = *reinterpret_cast<const bf16x8*>(&q_lo[(16 * qt + n) * pitch + d0]);
              }
              acc[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, b_hi, acc[qt][j], 0, 0, 0);
              acc[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, b_lo, acc[qt][j], 0, 0, 0);
            }
          }
        }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) kc[t] = kn[t];
      // score tiles: lane (n, kg) holds query 16 qt + n, keys 16 j + 4 kg + i -> LDS [query][key] -> row segments
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          *reinterpret_cast<f32x4*>(ctile + n * kCPitch + 16 * j + 4 * kg) = acc[qt][j] * p.sm_scale;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int r = 16 * qt + 4 * u + (lane >> 4), col = 4 * (lane & 15);
          f32x4 v = *reinterpret_cast<const f32x4*>(ctile + (4 * u + (lane >> 4)) * kCPitch + col);
          const int key = key0 + col;
          if (r < rows_here && key < key_end) {          // (Skv is a multiple of 4: a group of four keys is in or out as a whole)
            if (p.mask) {
              const size_t mrow = ((size_t)b * p.Sq + (size_t)(p.s_begin + s_off + r)) * p.Skv + key;
#pragma unroll
              for (int i = 0; i < 4; ++i) v[i] += load_as(p.mask, mrow + i, p.mask_dtype);
            }
            *reinterpret_cast<f32x4*>(p.scores + (out_row0 + r) * (size_t)p.Skv + key) = v;
          }
        }
      }
    }
    return;
  }
  const bool prefetch = kPrefetch && p.k_vec;
  if (prefetch && key_begin + 64 * wave < key_end) fetch(key_begin + 64 * wave, cur);
  for (int key0 = key_begin + 64 * wave; key0 < key_end; key0 += kKeysPerIter) {
    f32x4 acc[QT][4];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[qt][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (prefetch) {
      if (key0 + kKeysPerIter < key_end) fetch(key0 + kKeysPerIter, nxt);
#pragma unroll
      for (int ks = 0; ks < kBuf; ++ks) {
        const int d0 = 32 * ks + 8 * kg;
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
          const bf16x8 b_hi = *reinterpret_cast<const bf16x8*>(&q_hi[(16 * qt + n) * pitch + d0]);
          const bf16x8 b_lo = *reinterpret_cast<const bf16x8*>(&q_lo[(16 * qt + n) * pitch + d0]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const bf16x8 ka = __builtin_bit_cast(bf16x8, cur[ks][j]);
            acc[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, b_hi, acc[qt][j], 0, 0, 0);
            acc[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, b_lo, acc[qt][j], 0, 0, 0);
          }
        }
      }
#pragma unroll
      for (int ks = 0; ks < kBuf; ++ks)
#pragma unroll
        for (int j = 0; j < 4; ++j) cur[ks][j] = nxt[ks][j];
    } else {
      for (int ks = 0; ks < ksteps; ++ks) {
        const int d0 = 32 * ks + 8 * kg;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int key = min(key0 + 16 * j + n, p.Skv - 1);
          const size_t base = ((size_t)b * p.Skv + (size_t)key) * D + d0;
          float v[8];
          if (!K_F32) {
            if (p.k_vec) {
              uint4 raw = make_uint4(0u, 0u, 0u, 0u);
              if (d0 < D) raw = *reinterpret_cast<const uint4*>((const unsigned short*)p.k + base);
              const unsigned u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
              for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(u[i] << 16); v[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u); }
            } else {
#pragma unroll
              for (int i = 0; i < 8; ++i) v[i] = (d0 + i < D) ? bf16_bits_to_f32(((const unsigned short*)p.k)[base + i]) : 0.0f;
            }
          } else if (p.k_vec) {
            float4 t0 = make_float4(0, 0, 0, 0), t1 = t0;
            if (d0 < D) {
              t0 = *reinterpret_cast<const float4*>((const float*)p.k + base);
              t1 = *reinterpret_cast<const float4*>((const float*)p.k + base + 4);
            }
            v[0] = t0.x; v[1] = t0.y; v[2] = t0.z; v[3] = t0.w; v[4] = t1.x; v[5] = t1.y; v[6] = t1.z; v[7] = t1.w;
          } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = (d0 + i < D) ? ((const float*)p.k)[base + i] : 0.0f;
          }
          unsigned short h8[8], l8[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) split_bf16(v[i], h8[i], l8[i]);      // (lo is zero for a bf16 key)
          const bf16x8 kh = __builtin_bit_cast(
              bf16x8, make_uint4(h8[0] | ((unsigned)h8[1] << 16), h8[2] | ((unsigned)h8[3] << 16),
                                 h8[4] | ((unsigned)h8[5] << 16), h8[6] | ((unsigned)h8[7] << 16)));
          const bf16x8 kl = __builtin_bit_cast(
              bf16x8, make_uint4(l8[0] | ((unsigned)l8[1] << 16), l8[2] | ((unsigned)l8[3] << 16),
                                 l8[4] | ((unsigned)l8[5] << 16), l8[6] | ((unsigned)l8[7] << 16)));
#pragma unroll
          for (int qt = 0; qt < QT; ++qt) {
            const bf16x8 b_hi = *reinterpret_cast<const bf16x8*>(&q_hi[(16 * qt + n) * pitch + d0]);
            const bf16x8 b_lo = *reinterpret_cast<const bf16x8*>(&q_lo[(16 * qt + n) * pitch + d0]);
            acc[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kh, b_hi, acc[qt][j], 0, 0, 0);
            acc[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kh, b_lo, acc[qt][j], 0, 0, 0);
            if (K_F32) acc[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kl, b_hi, acc[qt][j], 0, 0, 0);
          }
        }
      }
    }
    // lane (n, kg): query rows 16 qt + n, keys key0 + 16 j + 4 kg + i
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const int r = 16 * qt + n;
      if (r >= rows_here) continue;
      const size_t mask_row = ((size_t)b * p.Sq + (size_t)(p.s_begin + s_off + r)) * p.Skv;
      float* dst = p.scores + (out_row0 + r) * (size_t)p.Skv;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = key0 + 16 * j + 4 * kg;
        float s[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[i] = acc[qt][j][i] * p.sm_scale;
          if (p.mask && key + i < key_end) s[i] += load_as(p.mask, mask_row + key + i, p.mask_dtype);
        }
        if (p.s_vec && key + 3 < key_end) {
          *reinterpret_cast<float4*>(dst + key) = make_float4(s[0], s[1], s[2], s[3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (key + i < key_end) dst[key + i] = s[i];
        }
      }
    }
  }
}

struct Plan {
  int rows_per_pass;     // query rows of one batch per pass (when Sq is chunked), else Sq
  int batches_per_pass;  // batches per pass (when whole batches fit), else 1
  size_t score_bytes;    // bytes of the score chunk
  size_t qw_bytes;       // bytes of the head-summed queries of one pass (bf16 hi + lo planes)
  size_t topk_bytes;     // candidate buffers of the selector's two-stage path (wide rows)
};

constexpr size_t kChunkBytes = (size_t)256 << 20;

Plan make_plan(const cppmega_mi355_indexer_args_t& a) {
  Plan pl;
  const size_t row_bytes = (size_t)a.seq_kv * 4;
  if (a.scores_out) {                 // the caller keeps every score: one pass over everything
    pl.rows_per_pass = a.seq_q;
    pl.batches_per_pass = a.batch;
  } else {
    size_t cap = a.chunk_rows > 0 ? (size_t)a.chunk_rows : kChunkBytes / (row_bytes ? row_bytes : 1);
    if (cap < 1) cap = 1;
    if ((size_t)a.seq_q > cap) {
      pl.rows_per_pass = (int)(cap >= (size_t)kQRows ? cap / kQRows * kQRows : cap);
      pl.batches_per_pass = 1;
    } else {
      pl.rows_per_pass = a.seq_q;
      size_t nb = cap / (size_t)(a.seq_q > 0 ? a.seq_q : 1);
      pl.batches_per_pass = (int)(nb < 1 ? 1 : (nb > (size_t)a.batch ? (size_t)a.batch : nb));
    }
  }
  const size_t rows = (size_t)pl.rows_per_pass * (size_t)pl.batches_per_pass;
  pl.score_bytes = a.scores_out ? 0 : ((rows * row_bytes + 255) & ~(size_t)255);
  pl.qw_bytes = (rows * (size_t)((a.head_dim + 31) & ~31) * 2 * 2 + 255) & ~(size_t)255;
  cppmega_mi355_topk_args_t t;
  memset(&t, 0, sizeof(t));
  t.rows = (int)rows; t.width = a.seq_kv; t.row_stride = a.seq_kv; t.k = a.topk;
  pl.topk_bytes = 0;
  if (a.topk >= 1 && a.topk <= a.seq_kv) (void)topk_workspace_bytes(t, &pl.topk_bytes);
  return pl;
}

int validate(const cppmega_mi355_indexer_args_t& a, bool need_pointers) {
  if (a.batch < 0 || a.seq_q < 0 || a.heads < 1 || a.head_dim < 1 || a.seq_kv < 1)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "indexer: negative or empty dimension");
  if (a.head_dim > kMaxD) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "indexer: head_dim %d exceeds %d", a.head_dim, kMaxD);
  if (a.topk < 1 || a.topk > a.seq_kv) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk must be in [1, %d]; got %d", a.seq_kv, a.topk);
  const int fl[3] = {a.q_dtype, a.w_dtype, a.k_dtype};
  for (int i = 0; i < 3; ++i)
    if (fl[i] != CPPMEGA_MI355_F32 && fl[i] != CPPMEGA_MI355_BF16)
      return fail(CPPMEGA_MI355_ERR_DTYPE, "indexer: q, weights and k must be float32 or bfloat16");
  if (a.mask && a.mask_dtype != CPPMEGA_MI355_F32 && a.mask_dtype != CPPMEGA_MI355_BF16 && a.mask_dtype != CPPMEGA_MI355_F16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "indexer: mask must be float32, float16 or bfloat16");
  if (a.order != CPPMEGA_MI355_TOPK_ORDER_INDEX && a.order != CPPMEGA_MI355_TOPK_ORDER_VALUE)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "indexer: unknown order %d", a.order);
  if (a.seq_kv > (a.seq_kv % 4 == 0 ? 65536 : 32768))
    return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "indexer: seq_kv %d exceeds the selector's row limit (65536, or 32768 when not a multiple of 4)", a.seq_kv);
  if (need_pointers && (!a.q || !a.weights || !a.k || !a.indices))
    return fail(CPPMEGA_MI355_ERR_NULL, "indexer: q/weights/k/indices is NULL");
  return 0;
}

}  // namespace

int indexer_topk_workspace_bytes(const cppmega_mi355_indexer_args_t& a, size_t* bytes) {
  const int rc = validate(a, false);
  if (rc) return rc;
  const Plan pl = make_plan(a);
  *bytes = pl.score_bytes + pl.qw_bytes + pl.topk_bytes;
  return 0;
}

template <bool K_F32, int QT>
static int launch_scores(const IndexerParams& p, dim3 grid, hipStream_t stream) {
  const size_t q_bytes = (size_t)2 * kQRows * QT * (((p.D + 31) & ~31) + 8) * sizeof(unsigned short);   // (two query tiles are only used up to D = 128: 17 KB)
  const int ks = (p.D + 31) / 32;
  if constexpr (!K_F32) {
    if (p.k_vec && p.s_vec && p.D % 32 == 0 && (ks == 1 || ks == 2 || ks == 4)) {
      const size_t lds = q_bytes + (size_t)(kThreads / 64) * kStageBytes;
      const void* fn = ks == 1 ? (const void*)indexer_scores_kernel<false, 1, QT, true>
                     : ks == 2 ? (const void*)indexer_scores_kernel<false, 2, QT, true>
                               : (const void*)indexer_scores_kernel<false, 4, QT, true>;
      if (lds > 64 * 1024) CM_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      IndexerParams q = p;
      void* kargs[] = {(void*)&q};
      CM_HIP_CHECK(hipLaunchKernel(fn, grid, dim3(kThreads), kargs, lds, stream));
      return 0;
    }
  }
  switch (ks) {
    case 1: hipLaunchKernelGGL((indexer_scores_kernel<K_F32, 1, QT>), grid, dim3(kThreads), q_bytes, stream, p); break;
    case 2: hipLaunchKernelGGL((indexer_scores_kernel<K_F32, 2, QT>), grid, dim3(kThreads), q_bytes, stream, p); break;
    case 4: hipLaunchKernelGGL((indexer_scores_kernel<K_F32, 4, QT>), grid, dim3(kThreads), q_bytes, stream, p); break;
    default: hipLaunchKernelGGL((indexer_scores_kernel<K_F32, 0, QT>), grid, dim3(kThreads), q_bytes, stream, p); break;
  }
  return 0;
}

int indexer_topk_launch(const cppmega_mi355_indexer_args_t& a, hipStream_t stream) {
  int rc = validate(a, true);
  if (rc) return rc;
  if ((size_t)a.batch * a.seq_q == 0) return 0;
  const Plan pl = make_plan(a);
  const size_t need = pl.score_bytes + pl.qw_bytes + pl.topk_bytes;
  if (!a.workspace || a.workspace_bytes < need)
    return fail(CPPMEGA_MI355_ERR_WORKSPACE, "indexer: workspace of %zu bytes needed, %zu given", need,
                a.workspace ? a.workspace_bytes : (size_t)0);
  if (((uintptr_t)a.workspace | (uintptr_t)a.scores_out) & 15)
    return fail(CPPMEGA_MI355_ERR_ALIGNMENT, "indexer: workspace and scores_out must be 16-byte aligned");
  float* scores = a.scores_out ? a.scores_out : (float*)a.workspace;

  IndexerParams p;
  p.q = a.q; p.w = a.weights; p.k = a.k; p.mask = a.mask; p.scores = scores;
  p.starts = nullptr; p.ends = nullptr;
  p.qw = (unsigned short*)((char*)a.workspace + pl.score_bytes);
  p.q_dtype = a.q_dtype; p.w_dtype = a.w_dtype; p.k_dtype = a.k_dtype; p.mask_dtype = a.mask_dtype;
  p.B = a.batch; p.Sq = a.seq_q; p.H = a.heads; p.D = a.head_dim; p.Skv = a.seq_kv;
  p.sm_scale = a.sm_scale;
  p.q_vec = a.q_dtype == CPPMEGA_MI355_BF16 && a.head_dim % 8 == 0 && ((uintptr_t)a.q & 15) == 0;
  p.k_vec = a.head_dim % 8 == 0 && ((uintptr_t)a.k & 15) == 0;
  p.s_vec = a.seq_kv % 4 == 0;

  for (int b0 = 0; b0 < a.batch; b0 += pl.batches_per_pass) {
    const int nb = a.batch - b0 < pl.batches_per_pass ? a.batch - b0 : pl.batches_per_pass;
    for (int s_begin = 0; s_begin < a.seq_q; s_begin += pl.rows_per_pass) {
      const int s_count = a.seq_q - s_begin < pl.rows_per_pass ? a.seq_q - s_begin : pl.rows_per_pass;
      p.b_begin = b0; p.nb = nb; p.s_begin = s_begin; p.s_count = s_count;
      if (!a.scores_out) {
        const size_t first = (size_t)b0 * a.seq_q + (size_t)s_begin;
        p.starts = a.starts ? a.starts + first : nullptr;
        p.ends = a.ends ? a.ends + first : nullptr;
      }
      const int dp8 = ((a.head_dim + 31) & ~31) / 8;
      if (p.q_vec && (dp8 & (dp8 - 1)) == 0) {
        const dim3 qgrid((unsigned)((nb * s_count + kQwWaves - 1) / kQwWaves)), qblock(kQwWaves * 64);
        if (a.w_dtype == CPPMEGA_MI355_F32) hipLaunchKernelGGL(indexer_qw_wave_kernel<CPPMEGA_MI355_F32>, qgrid, qblock, 0, stream, p);
        else if (a.w_dtype == CPPMEGA_MI355_BF16) hipLaunchKernelGGL(indexer_qw_wave_kernel<CPPMEGA_MI355_BF16>, qgrid, qblock, 0, stream, p);
        else hipLaunchKernelGGL(indexer_qw_wave_kernel<CPPMEGA_MI355_F16>, qgrid, qblock, 0, stream, p);
      } else
        hipLaunchKernelGGL(indexer_qw_kernel, dim3((unsigned)(nb * s_count)), dim3(kThreads), 0, stream, p);
      const int qt = (s_count >= 4 * kQRows && a.head_dim <= 128) ? 2 : 1;     // query tiles per workgroup (prefill: two)
      const int tiles = (s_count + kQRows * qt - 1) / (kQRows * qt);
      const int max_splits = (a.seq_kv + kKeysPerIter - 1) / kKeysPerIter;
      int splits = (1024 + tiles * nb - 1) / (tiles * nb);
      splits = splits < 1 ? 1 : (splits > max_splits ? max_splits : splits);
      const int per = (a.seq_kv + splits - 1) / splits;
      p.keys_per_wg = (per + kKeysPerIter - 1) / kKeysPerIter * kKeysPerIter;
      const dim3 grid((unsigned)((a.seq_kv + p.keys_per_wg - 1) / p.keys_per_wg), (unsigned)tiles, (unsigned)nb);
      if (a.k_dtype == CPPMEGA_MI355_F32) rc = qt == 2 ? launch_scores<true, 2>(p, grid, stream) : launch_scores<true, 1>(p, grid, stream);
      else rc = qt == 2 ? launch_scores<false, 2>(p, grid, stream) : launch_scores<false, 1>(p, grid, stream);
      if (rc) return rc;
      CM_HIP_CHECK(hipGetLastError());

      const size_t row0 = (size_t)b0 * a.seq_q + (size_t)s_begin;    // first flattened query row of the pass
      cppmega_mi355_topk_args_t t;
      memset(&t, 0, sizeof(t));
      t.struct_size = (uint32_t)sizeof(t);
      t.score_dtype = CPPMEGA_MI355_F32;
      t.scores = scores;
      t.row_stride = a.seq_kv;
      t.rows = nb * s_count;
      t.width = a.seq_kv;
      t.k = a.topk;
      t.order = a.order;
      t.starts = a.starts ? a.starts + row0 : nullptr;
      t.ends = a.ends ? a.ends + row0 : nullptr;
      t.indices = a.indices + row0 * (size_t)a.topk;
      t.neg_inf_is_masked = a.mask ? 1 : 0;
      if (pl.topk_bytes) {
        t.workspace = (char*)a.workspace + pl.score_bytes + pl.qw_bytes;
        t.workspace_bytes = pl.topk_bytes;
      }
      rc = topk_select_launch(t, stream);
      if (rc) return rc;
    }
  }
  return 0;
}

}  // namespace cm
