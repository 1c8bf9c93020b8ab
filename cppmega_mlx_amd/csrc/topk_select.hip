// Radix-select top-k over indexer scores (gfx950).
//
// One workgroup owns one score row.  The row is read from HBM exactly once,
// with 16-byte loads, and stays in registers for the rest of the kernel; a
// 4096-bin histogram of the row lives in LDS.
//
// In topk_tile_kernel (rows of up to 32768 columns) every thread owns a
// contiguous run of columns: a thread's selected columns are then a bit mask,
// one block-wide prefix sum of the popcounts gives every thread its output
// offset, and the indices come out in ascending order.  Rows whose address and
// pitch allow 16-byte loads are fetched that way by the owning thread itself,
// the pieces of a run one load after the other (a wavefront's first load
// brings in the lines its next ones hit): the histogram can be cleared while
// the loads travel and no barrier precedes the first pass.  Other rows are
// loaded a column per lane and reach their owners through an LDS tile.  Wider
// rows (topk_wide_kernel, up to 65536 columns) keep the interleaved ownership
// of coalesced loads and compact with per-chunk ballots.
//
// Selection (k largest, ties toward the lower index):
//   pass 1  LDS-atomic histogram of bits[31:20] (sign, exponent, 3 mantissa
//           bits); a two-level scan over the bins, walking from the largest
//           value down, finds the bin where the running count reaches k
//   pass 2  the same over bits[19:8] of the elements that fell in that bin
//   pass 3  the same over bits[7:0]
// A pass ends the search early when the bin it found has to be taken whole;
// then "x >= lowest value of the bin" describes the selected set.  Only when
// the threshold value itself is duplicated beyond what is needed does the
// emission count equal elements and keep the first `rem` of them by index.
//
// Emission is a ballot/mbcnt compaction in ascending index order, staged in
// LDS and copied out with coalesced stores; the optional value-descending
// order sorts the selected (value, index) pairs in LDS first.
//
// Float compares give the ordering: -0.0 == +0.0, and NaN (which also stands
// for "outside [start,end)") never compares true, so it is never selected.
// After `x + 0.0f` every NaN is quiet, so NaNs fall into histogram bins no
// real number can reach (0x7f9..0x7ff, 0xff9..0xfff); the first scan counts
// those bins as empty instead of every element being tested.


#include <type_traits>

#include "common.h"

namespace cm {
namespace {

constexpr int kHistBins = 4096;

struct TopkParams {
  const void* scores;
  long long row_stride;
  const int* starts;
  const int* ends;
  int* out;
  int rows, width, k, order, neg_inf_masked;
  int sort_len;  // power of two >= k, used by the value-descending order
  // Rows too wide for one workgroup's fast path are selected in two stages (tile kernel only):
  // stage 1 launches one workgroup per (row, segment of seg_width columns) and writes the
  // segment's k best as candidates (value, column) in ascending column order; stage 2 selects
  // among a row's segs * k candidates and translates positions through index_map.
  int segs;             // > 1: stage 1; blockIdx.x = row * segs + segment, width = columns of the whole row
  int seg_width;
  float* cand_val;      // stage 1 out: [rows, segs, k] (NaN = no candidate)
  int* cand_idx;        // stage 1 out: [rows, segs, k] (-1 = no candidate)
  const int* index_map; // stage 2 in: [rows, width] column of each candidate position
};

struct Half {};   // tag types: 16-bit storage
struct BHalf {};
template <typename T> struct Storage { typedef unsigned short type; };
template <> struct Storage<float> { typedef float type; };

template <typename T> struct ScoreLoad;
template <> struct ScoreLoad<float> {
  static __device__ __forceinline__ void vec4(const float* p, float (&o)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
  }
  static __device__ __forceinline__ float one(const float* p) { return *p; }
};
template <> struct ScoreLoad<Half> {
  static __device__ __forceinline__ void vec4(const unsigned short* p, float (&o)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    o[0] = f16_bits_to_f32((unsigned short)(t.x & 0xffffu));
    o[1] = f16_bits_to_f32((unsigned short)(t.x >> 16));
    o[2] = f16_bits_to_f32((unsigned short)(t.y & 0xffffu));
    o[3] = f16_bits_to_f32((unsigned short)(t.y >> 16));
  }
  static __device__ __forceinline__ float one(const unsigned short* p) { return f16_bits_to_f32(*p); }
};
template <> struct ScoreLoad<BHalf> {
  static __device__ __forceinline__ void vec4(const unsigned short* p, float (&o)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    o[0] = __uint_as_float(t.x << 16);
    o[1] = __uint_as_float(t.x & 0xffff0000u);
    o[2] = __uint_as_float(t.y << 16);
    o[3] = __uint_as_float(t.y & 0xffff0000u);
  }
  static __device__ __forceinline__ float one(const unsigned short* p) { return bf16_bits_to_f32(*p); }
};

// Walk order of the bins, largest value first:
//   kSigned      bin = bits[31:20]: non-negative bins 2047..0, then negative bins 2048..4095
//   kDescending  larger digit = larger value  (non-negative prefix)
//   kAscending   larger digit = smaller value (negative prefix)
enum { kSigned = 0, kDescending = 1, kAscending = 2 };

// LDS layout (unsigned words) after the histogram
constexpr int kWaveTot = kHistBins;        // [16] per-wave totals of a scan
constexpr int kHit = kHistBins + 16;       // [4]  bin, above, cnt

struct BinHit {
  unsigned bin, above, cnt, total;
};

// Inclusive prefix sum over the first N (a power of two, at most 16) lanes of every row of 16.
template <int N>
__device__ __forceinline__ unsigned row_inclusive_sum_dpp(unsigned v) {
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);                  // row_shr:1
  if constexpr (N > 2) v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);   // row_shr:2
  if constexpr (N > 4) v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);   // row_shr:4
  if constexpr (N > 8) v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);   // row_shr:8
  return v;
}

// Given every wavefront's total in smem[at .. at + WAVES), returns the sum over the wavefronts
// before this one and the sum over all of them: lanes 0 .. WAVES-1 scan the totals, two lane reads
// pick the results (a handful of instructions where a loop over the wavefronts costs two each).
template <int WAVES>
__device__ __forceinline__ void waves_before_and_total(const unsigned* smem, int at, int lane, int wave, unsigned& before, unsigned& total) {
  static_assert(WAVES >= 2 && WAVES <= 16 && (WAVES & (WAVES - 1)) == 0, "wavefronts per workgroup");
  const unsigned incl = row_inclusive_sum_dpp<WAVES>(smem[at + (lane & (WAVES - 1))]);
  total = (unsigned)__builtin_amdgcn_readlane((int)incl, WAVES - 1);
  const unsigned upto = (unsigned)__builtin_amdgcn_readlane((int)incl, wave > 0 ? wave - 1 : 0);
  before = wave > 0 ? upto : 0u;
}

// Finds the bin at which the running count, walking from the largest value
// down, first reaches `need`.  All THREADS threads call it.  The walk visits the
// kHistBins bins in a mode-dependent order; the thread at walk position t takes
// the run of kHistBins / THREADS consecutive bins that the walk reaches t-th,
// front to back or back to front as the walk goes: one scan over the threads'
// run sums finds the thread, which then walks its own run.
// `skip_nan_bins` (first pass only): the bins 0x7f9..0x7ff and 0xff9..0xfff, which no number but only
// NaN patterns reach, count as empty.
template <int NB, int THREADS>
__device__ BinHit find_bin(unsigned* smem, unsigned need, int mode, bool skip_nan_bins = false) {
  static_assert(NB == kHistBins, "the scan walks the whole histogram");
  constexpr int BPT = NB / THREADS;               // 16, 8 or 4 bins per thread
  constexpr int WAVES = THREADS / 64;
  static_assert(BPT >= 4 && BPT % 4 == 0 && BPT * THREADS == NB, "bins per thread");
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // kSigned: bins 2047..0 (the non-negative values, largest first), then 2048..4095
  const bool desc = mode == kDescending || (mode == kSigned && tid < THREADS / 2);
  const int run = mode == kAscending ? tid : mode == kDescending ? THREADS - 1 - tid : (desc ? THREADS / 2 - 1 - tid : tid);
  unsigned c[BPT];
  unsigned sum = 0;
#pragma unroll
  for (int i = 0; i < BPT / 4; ++i) {
    const uint4 q = reinterpret_cast<const uint4*>(smem)[run * (BPT / 4) + i];
    c[4 * i] = q.x; c[4 * i + 1] = q.y; c[4 * i + 2] = q.z; c[4 * i + 3] = q.w;
    sum += q.x + q.y + q.z + q.w;
  }
  if (skip_nan_bins && ((run * BPT + BPT - 1) & 0x7ff) >= 0x7f9) {      // (two threads, or four)
    sum = 0;
#pragma unroll
    for (int i = 0; i < BPT; ++i) {
      if (((run * BPT + i) & 0x7ff) >= 0x7f9) c[i] = 0;
      sum += c[i];
    }
  }
  const unsigned incl = wave_inclusive_sum_dpp(sum);
  if (lane == 63) smem[kWaveTot + wave] = incl;
  __syncthreads();
  unsigned before, total;
  waves_before_and_total<WAVES>(smem, kWaveTot, lane, wave, before, total);
  before += incl - sum;
  if (before < need && need <= before + sum) {      // exactly one thread when need <= total
    // The walk direction is the same for a whole wavefront (a mode, or the half of the workgroup
    // in the signed pass): a scalar branch picks one of two walks with constant register indices,
    // and one write follows the walk (with the direction as a per-lane value every step was an
    // eight-way register select: ~150 instructions that the rest of the row waits for).
    unsigned hit_i = 0, hit_walked = before, hit_n = 0, walked = before;
    auto walk = [&](auto dir) {
      constexpr bool D = decltype(dir)::value;
#pragma unroll
      for (int i = 0; i < BPT; ++i) {
        const unsigned n = c[D ? BPT - 1 - i : i];
        const bool here = walked < need && need <= walked + n;
        hit_i = here ? (unsigned)(D ? BPT - 1 - i : i) : hit_i;
        hit_walked = here ? walked : hit_walked;
        hit_n = here ? n : hit_n;
        walked += n;
      }
    };
    if (__builtin_amdgcn_readfirstlane((int)desc)) walk(std::true_type{});
    else walk(std::false_type{});
    smem[kHit + 0] = (unsigned)(run * BPT) + hit_i;
    smem[kHit + 1] = hit_walked;
    smem[kHit + 2] = hit_n;
  }
  __syncthreads();
  BinHit hit;
  hit.bin = smem[kHit + 0];
  hit.above = smem[kHit + 1];
  hit.cnt = smem[kHit + 2];
  hit.total = total;
  return hit;
}

template <int THREADS>
__device__ __forceinline__ void zero_hist(unsigned* hist, int nbins) {
  uint4* dst = reinterpret_cast<uint4*>(hist);
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (int i = (int)threadIdx.x; i < nbins / 4; i += THREADS) dst[i] = z;
}

// Monotone key of a float: larger value <=> larger key.
__device__ __forceinline__ unsigned order_key(float x) {
  const unsigned u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// ---------------------------------------------------------------------------
// Rows of up to 8192 columns: 256 threads, thread t owns columns [t*E, (t+1)*E).
// ---------------------------------------------------------------------------
constexpr int kTileThreads = 256;
constexpr int kTileScratch = kHistBins + 64;            // words: histogram + scan scratch
// The row tile is not padded (8192 columns are 32 KiB: four such workgroups fit a CU, and the
// allocation of a padded tile let only three in).  A thread's run of E columns is E/4 pieces of 16
// bytes; piece i of thread t sits at position (i + rot(t)) mod E/4 of the run, with rot chosen so
// that the sixteen lanes of one LDS cycle read sixteen different 16-byte bank groups.
template <int E>
__device__ __forceinline__ int tile_piece_slot(int t, int i) {
  constexpr int PP = E / 4;                               // pieces per thread: 1, 2, 4 or 8
  if constexpr (PP == 1) return t;
  constexpr int SH = PP == 2 ? 3 : PP == 4 ? 2 : 1;       // log2(16 / PP)
  return PP * t + ((i + (t >> SH)) & (PP - 1));
}
// both histograms fit the tile's allocation of the widest shape with 64 words to spare
__host__ __device__ constexpr bool tile_two_hists(int E, int threads) { return threads * E >= 2 * kHistBins; }

// MODE 0: a row per workgroup.  MODE 1: stage 1 of a wide row (a segment per workgroup, candidates
// out).  MODE 2: stage 2 (a row of candidates per workgroup, positions translated through index_map).
// DIRECT: a thread fetches its own run of columns from memory, 16 bytes at a time, the pieces of
// a run one load after the other (the lines a wavefront touches with its first load serve its
// next ones from the cache): no trip through an LDS tile and no barriers before the first pass.
template <typename ScoreT, int E, int VEC, int THREADS = kTileThreads, int MODE = 0, bool DIRECT = false>
__global__ __launch_bounds__(THREADS, E > 16 ? 4 : 8) void topk_tile_kernel(const TopkParams p) {
  static_assert(!DIRECT || VEC == 4, "direct loads are 16-byte loads");
  constexpr int ITEMS = E / VEC;                        // loads per thread
  constexpr int CHUNK = THREADS * VEC;                  // columns covered by one load per thread
  extern __shared__ __align__(16) unsigned smem[];
  float* tile = reinterpret_cast<float*>(smem);
  unsigned* hist = smem;
  typedef typename Storage<ScoreT>::type St;

  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr bool stage1 = MODE == 1;
  const int row = stage1 ? (int)blockIdx.x / p.segs : (int)blockIdx.x;
  const int base = stage1 ? ((int)blockIdx.x % p.segs) * p.seg_width : 0;   // first column of this workgroup's share
  const int T = stage1 ? min(p.seg_width, p.width - base) : p.width;
  int start = (p.starts ? p.starts[row] : 0) - base;
  int end = (p.ends ? p.ends[row] : p.width) - base;
  start = min(max(start, 0), T);
  end = min(max(end, 0), T);
  const St* src = reinterpret_cast<const St*>(p.scores) + (long long)row * p.row_stride + base;
  int* out_row = p.out + (long long)row * p.k;
  const float kNaN = __uint_as_float(0x7fc00000u);
  const float kNegInf = __uint_as_float(0xff800000u);
  const unsigned k = (unsigned)p.k;

  float v[E];
  constexpr int kHist2 = tile_two_hists(E, THREADS) ? kHistBins + 64 : 0;
  if constexpr (DIRECT) {
    // (no tile in LDS on this path: the histograms are cleared before the row's bounds have arrived)
    zero_hist<THREADS>(hist, kHist2 ? kHist2 + kHistBins : kHistBins);
    const int c0 = tid * E;
    const bool any = c0 < end && c0 + E > start;          // (a run with nothing selectable is not read)
#pragma unroll
    for (int i = 0; i < E / 4; ++i) {
      float t4[4] = {kNaN, kNaN, kNaN, kNaN};
      if (any && c0 + 4 * i < T) ScoreLoad<ScoreT>::vec4(src + c0 + 4 * i, t4);
      v[4 * i] = t4[0]; v[4 * i + 1] = t4[1]; v[4 * i + 2] = t4[2]; v[4 * i + 3] = t4[3];
    }
  } else {
  // ---- HBM -> LDS, coalesced; chunks with nothing selectable are not read ----------
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int chunk_lo = j * CHUNK;
    const int col = chunk_lo + tid * VEC;
    if (chunk_lo >= end || chunk_lo + CHUNK <= start || col >= T) continue;
    float* dst = tile + 4 * tile_piece_slot<E>(col / E, (col % E) >> 2) + (col & 3);
    if constexpr (VEC == 4) {
      float t4[4];
      ScoreLoad<ScoreT>::vec4(src + col, t4);
      *reinterpret_cast<float4*>(dst) = make_float4(t4[0], t4[1], t4[2], t4[3]);
    } else {
      *dst = ScoreLoad<ScoreT>::one(src + col);
    }
  }
  __syncthreads();
  // ---- LDS -> registers: my contiguous run ------------------------------------------
#pragma unroll
  for (int i = 0; i < E / 4; ++i) {
    const float4 t4 = *reinterpret_cast<const float4*>(tile + 4 * tile_piece_slot<E>(tid, i));
    v[4 * i] = t4.x; v[4 * i + 1] = t4.y; v[4 * i + 2] = t4.z; v[4 * i + 3] = t4.w;
  }
  __syncthreads();
  }
  // two cleared histograms: pass 1 uses the first, pass 2 the second (no clear + barrier in between)
  if constexpr (!DIRECT) zero_hist<THREADS>(hist, kHist2 ? kHist2 + kHistBins : kHistBins);
  __syncthreads();

  // ---- canonicalise (-0 -> +0, NaN -> quiet NaN, masked -> NaN) + pass 1 -------------
  // A row with no more selectable columns than k needs no threshold: everything that is a number is
  // taken (the rows of a causal prefill whose prefix is shorter than k).
  const int col0 = tid * E;
  const bool take_all = end - start <= (int)k;      // (uniform)
  if (take_all) {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      float x = v[i] + 0.0f;
      const int idx = col0 + i;
      x = (idx >= start && idx < end) ? x : kNaN;
      if (p.neg_inf_masked) x = (x == kNegInf) ? kNaN : x;
      v[i] = x;
    }
  } else if (col0 >= start && col0 + E <= end && !p.neg_inf_masked) {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      const float x = v[i] + 0.0f;
      v[i] = x;
      atomicAdd(&hist[__float_as_uint(x) >> 20], 1u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      float x = v[i] + 0.0f;
      const int idx = col0 + i;
      x = (idx >= start && idx < end) ? x : kNaN;
      if (p.neg_inf_masked) x = (x == kNegInf) ? kNaN : x;
      v[i] = x;
      if (x == x) atomicAdd(&hist[__float_as_uint(x) >> 20], 1u);
    }
  }
  float thr = kNegInf;
  unsigned rem = 0;
  bool tie = false;
  BinHit h1;
  h1.bin = 0; h1.above = 0; h1.cnt = 0; h1.total = 0;
  if (!take_all) {
    __syncthreads();
    h1 = find_bin<kHistBins, THREADS>(smem, k, kSigned, true);
  }
  if (h1.total <= k) {
    thr = kNegInf;   // every selectable element is taken
  } else {
    unsigned lo_bits;
    const bool neg = (h1.bin & 0x800u) != 0;
    rem = k - h1.above;
    if (rem == h1.cnt) {
      lo_bits = (h1.bin << 20) | (neg ? 0x000fffffu : 0u);
    } else {
      // ---- pass 2: bits[19:8] of the elements in bin h1 -----------------------------
      unsigned* hist2 = smem + kHist2;
      if (!kHist2) {
        zero_hist<THREADS>(hist, kHistBins);
        __syncthreads();
      }
      const unsigned p1 = h1.bin;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const unsigned u = __float_as_uint(v[i]);
        if ((u >> 20) == p1) atomicAdd(&hist2[(u >> 8) & 0xfffu], 1u);
      }
      __syncthreads();
      const BinHit h2 = find_bin<kHistBins, THREADS>(hist2, rem, neg ? kAscending : kDescending);
      rem -= h2.above;
      const unsigned p2 = (p1 << 12) | h2.bin;     // bits[31:8]
      if (rem == h2.cnt) {
        lo_bits = (p2 << 8) | (neg ? 0xffu : 0u);
      } else {
        // ---- pass 3: bits[7:0] (256 of the cleared slots are used) -------------------------
        constexpr int NB3 = kHistBins;                      // (the scan walks the whole histogram)
        zero_hist<THREADS>(hist, NB3);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const unsigned u = __float_as_uint(v[i]);
          if ((u >> 8) == p2) atomicAdd(&hist[u & 0xffu], 1u);
        }
        __syncthreads();
        const BinHit h3 = find_bin<NB3, THREADS>(smem, rem, neg ? kAscending : kDescending);
        rem -= h3.above;
        lo_bits = (p2 << 8) | h3.bin;
        tie = rem != h3.cnt;
      }
    }
    if (lo_bits > 0xff800000u) lo_bits = 0xff800000u;   // below -inf there are only NaN patterns
    thr = __uint_as_float(lo_bits);
  }

  // ---- emission: bit masks, one block-wide prefix sum, ascending indices --------------
  // (the common case - index order, no duplicated threshold - only counts here and compares again
  // when it writes: a compare and an add-with-carry per element instead of building a mask and
  // taking it apart)
  const bool sorted = p.order == CPPMEGA_MI355_TOPK_ORDER_VALUE;
  const bool plain = !sorted && !tie;
  unsigned gmask = 0, emask = 0, cg = 0, ce = 0;
  if (plain) {
#pragma unroll
    for (int i = 0; i < E; ++i) cg += (v[i] >= thr) ? 1u : 0u;
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      const float x = v[i];
      gmask |= ((tie ? (x > thr) : (x >= thr)) ? 1u : 0u) << i;
      if (tie) emask |= ((x == thr) ? 1u : 0u) << i;
    }
    cg = (unsigned)__popc(gmask);
    ce = (unsigned)__popc(emask);
  }
  const unsigned packed = cg | (ce << 16);               // both counts fit in 16 bits (<= 8192)
  const unsigned incl = wave_inclusive_sum_dpp(packed);
  if (lane == 63) smem[kWaveTot + wave] = incl;
  __syncthreads();
  unsigned before, totals;
  waves_before_and_total<THREADS / 64>(smem, kWaveTot, lane, wave, before, totals);
  before += incl - packed;
  unsigned run_g = before & 0xffffu, run_e = before >> 16;
  const unsigned n_sel = (totals & 0xffffu) + min(totals >> 16, rem);
  int* stage = reinterpret_cast<int*>(smem + kTileScratch);
  unsigned long long* pairs = reinterpret_cast<unsigned long long*>(smem + kTileScratch);
  if (plain) {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      const bool g = v[i] >= thr;
      if (g) stage[run_g] = col0 + i;
      run_g += g ? 1u : 0u;
    }
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      const bool g = (gmask >> i) & 1u, e = (emask >> i) & 1u;
      const bool sel = g || (e && run_e < rem);
      const unsigned pos = run_g + min(run_e, rem);
      if (sel) {
        const unsigned idx = (unsigned)(col0 + i);
        if (sorted) pairs[pos] = ((unsigned long long)order_key(v[i]) << 32) | (0xffffffffu - idx);
        else stage[pos] = (int)idx;
      }
      run_g += g ? 1u : 0u;
      run_e += e ? 1u : 0u;
    }
  }
  if (!sorted) {
    __syncthreads();
    if (stage1) {                                        // candidates: (value, column of the whole row), ascending column
      const long long at = (long long)blockIdx.x * p.k;
      for (unsigned i = tid; i < k; i += THREADS) {
        const bool have = i < n_sel;
        const int c = have ? stage[i] : 0;
        p.cand_idx[at + i] = have ? base + c : -1;
        p.cand_val[at + i] = have ? ScoreLoad<ScoreT>::one(src + c) + 0.0f : kNaN;
      }
      return;
    }
    const int* map = MODE == 2 ? p.index_map + (long long)row * p.width : nullptr;
    // (written once, not read again here: non-temporal; four slots per thread and store where the
    // row allows it - the stage starts on a 16-byte boundary)
    if (MODE != 2 && (k & 3u) == 0 && (((size_t)out_row) & 15) == 0) {
      typedef int i32x4_t __attribute__((ext_vector_type(4)));
      for (unsigned i = 4 * tid; i < k; i += 4 * THREADS) {
        i32x4_t q = *reinterpret_cast<const i32x4_t*>(stage + i);
#pragma unroll
        for (int c = 0; c < 4; ++c) q[c] = (i + c < n_sel) ? q[c] : -1;
        __builtin_nontemporal_store(q, reinterpret_cast<i32x4_t*>(out_row + i));
      }
      return;
    }
    for (unsigned i = tid; i < k; i += THREADS)
      __builtin_nontemporal_store((i < n_sel) ? (MODE == 2 ? map[stage[i]] : stage[i]) : -1, out_row + i);
    return;
  }
  const int* map = MODE == 2 ? p.index_map + (long long)row * p.width : nullptr;
  const unsigned P = (unsigned)p.sort_len;
  for (unsigned i = n_sel + tid; i < P; i += THREADS) pairs[i] = 0ull;   // sorts last
  __syncthreads();
  // bitonic sort, descending: larger value first, then lower index
  for (unsigned size = 2; size <= P; size <<= 1) {
    for (unsigned stride = size >> 1; stride > 0; stride >>= 1) {
      for (unsigned t = tid; t < P / 2; t += THREADS) {
        const unsigned i = 2 * t - (t & (stride - 1));
        const unsigned jx = i + stride;
        const bool desc = (i & size) == 0;
        const unsigned long long a = pairs[i], b = pairs[jx];
        if ((a < b) == desc) { pairs[i] = b; pairs[jx] = a; }
      }
      __syncthreads();
    }
  }
  for (unsigned i = tid; i < k; i += THREADS) {
    const int pos = (int)(0xffffffffu - (unsigned)(pairs[i] & 0xffffffffull));
    out_row[i] = (i < n_sel) ? (MODE == 2 ? map[pos] : pos) : -1;
  }
}

// ---------------------------------------------------------------------------
// Wider rows (up to 65536 columns): 1024 threads, interleaved ownership as loaded
// (column = (j*THREADS + tid)*VEC + c).  Bins come from the monotone key of the
// value, so every walk is "larger digit first".
// ---------------------------------------------------------------------------
constexpr int kWideThreads = 1024;
constexpr int kWideWaves = kWideThreads / 64;
constexpr int kWideEmit = kHistBins + 64;               // [ITEMS*16*2] per (chunk, wave) counts
constexpr int kWideScratch = kHistBins + 64 + 2 * 32 * kWideWaves;

template <typename ScoreT, int ITEMS, int VEC>
__global__ __launch_bounds__(kWideThreads) void topk_wide_kernel(const TopkParams p) {
  constexpr int THREADS = kWideThreads, WAVES = kWideWaves;
  constexpr int CHUNK = THREADS * VEC;
  extern __shared__ __align__(16) unsigned smem[];
  unsigned* hist = smem;
  typedef typename Storage<ScoreT>::type St;

  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row = (int)blockIdx.x;
  const int T = p.width;
  int start = p.starts ? p.starts[row] : 0;
  int end = p.ends ? p.ends[row] : T;
  start = min(max(start, 0), T);
  end = min(max(end, 0), T);
  const St* src = reinterpret_cast<const St*>(p.scores) + (long long)row * p.row_stride;
  int* out_row = p.out + (long long)row * p.k;
  const float kNaN = __uint_as_float(0x7fc00000u);
  const float kNegInf = __uint_as_float(0xff800000u);
  const unsigned k = (unsigned)p.k;

  float v[ITEMS][VEC];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int chunk_lo = j * CHUNK;
    const int base = chunk_lo + tid * VEC;
    if (chunk_lo >= end || chunk_lo + CHUNK <= start || base >= T) {
#pragma unroll
      for (int c = 0; c < VEC; ++c) v[j][c] = kNaN;
    } else if constexpr (VEC == 4) {
      ScoreLoad<ScoreT>::vec4(src + base, v[j]);
    } else {
      v[j][0] = ScoreLoad<ScoreT>::one(src + base);
    }
  }
  zero_hist<THREADS>(hist, kHistBins);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      float x = v[j][c] + 0.0f;
      const int idx = j * CHUNK + tid * VEC + c;
      x = (idx >= start && idx < end) ? x : kNaN;
      if (p.neg_inf_masked) x = (x == kNegInf) ? kNaN : x;
      v[j][c] = x;
      if (x == x) atomicAdd(&hist[order_key(x) >> 20], 1u);
    }
  }
  __syncthreads();

  BinHit h1 = find_bin<kHistBins, THREADS>(smem, k, kDescending);
  float thr;
  unsigned rem = 0;
  bool tie = false;
  if (h1.total <= k) {
    thr = kNegInf;
  } else {
    unsigned lo_key;
    rem = k - h1.above;
    if (rem == h1.cnt) {
      lo_key = h1.bin << 20;
    } else {
      zero_hist<THREADS>(hist, kHistBins);
      __syncthreads();
      const unsigned p1 = h1.bin;
#pragma unroll
      for (int j = 0; j < ITEMS; ++j)
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
          const float x = v[j][c];
          const unsigned key = order_key(x);
          if (x == x && (key >> 20) == p1) atomicAdd(&hist[(key >> 8) & 0xfffu], 1u);
        }
      __syncthreads();
      const BinHit h2 = find_bin<kHistBins, THREADS>(smem, rem, kDescending);
      rem -= h2.above;
      const unsigned p2 = (p1 << 12) | h2.bin;
      if (rem == h2.cnt) {
        lo_key = p2 << 8;
      } else {
        zero_hist<THREADS>(hist, kHistBins);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < ITEMS; ++j)
#pragma unroll
          for (int c = 0; c < VEC; ++c) {
            const float x = v[j][c];
            const unsigned key = order_key(x);
            if (x == x && (key >> 8) == p2) atomicAdd(&hist[key & 0xffu], 1u);
          }
        __syncthreads();
        const BinHit h3 = find_bin<kHistBins, THREADS>(smem, rem, kDescending);
        rem -= h3.above;
        lo_key = (p2 << 8) | h3.bin;
        tie = rem != h3.cnt;
      }
    }
    if (lo_key < 0x007fffffu) lo_key = 0x007fffffu;       // the key of -inf; below it only NaN patterns
    thr = __uint_as_float((lo_key & 0x80000000u) ? (lo_key ^ 0x80000000u) : ~lo_key);
  }

  // ---- emission: per-chunk ballots ------------------------------------------------------
  unsigned long long gflags = 0, eflags = 0;   // bit j*VEC+c
  unsigned short pre_g[ITEMS], pre_e[ITEMS];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    unsigned pg = 0, pe = 0, tg = 0, te = 0;
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      const float x = v[j][c];
      const bool g = tie ? (x > thr) : (x >= thr);
      const unsigned long long mg = __ballot(g);
      pg += mbcnt(mg);
      tg += (unsigned)__popcll(mg);
      gflags |= (g ? 1ull : 0ull) << (j * VEC + c);
      if (tie) {
        const bool e = (x == thr);
        const unsigned long long me = __ballot(e);
        pe += mbcnt(me);
        te += (unsigned)__popcll(me);
        eflags |= (e ? 1ull : 0ull) << (j * VEC + c);
      }
    }
    pre_g[j] = (unsigned short)pg;
    pre_e[j] = (unsigned short)pe;
    if (lane == 0) {
      smem[kWideEmit + (j * WAVES + wave) * 2 + 0] = tg;
      smem[kWideEmit + (j * WAVES + wave) * 2 + 1] = te;
    }
  }
  __syncthreads();
  const bool sorted = p.order == CPPMEGA_MI355_TOPK_ORDER_VALUE;
  int* stage = reinterpret_cast<int*>(smem + kWideScratch);
  unsigned long long* pairs = reinterpret_cast<unsigned long long*>(smem + kWideScratch);
  unsigned base_g = 0, base_e = 0;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    unsigned run_g = base_g, run_e = base_e;
    for (int w = 0; w < WAVES; ++w) {
      const unsigned tg = smem[kWideEmit + (j * WAVES + w) * 2 + 0];
      const unsigned te = smem[kWideEmit + (j * WAVES + w) * 2 + 1];
      if (w < wave) { run_g += tg; run_e += te; }
      base_g += tg;
      base_e += te;
    }
    run_g += pre_g[j];
    run_e += pre_e[j];
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      const bool g = (gflags >> (j * VEC + c)) & 1ull;
      const bool e = (eflags >> (j * VEC + c)) & 1ull;
      const bool sel = g || (e && run_e < rem);
      const unsigned pos = run_g + min(run_e, rem);
      if (sel) {
        const unsigned idx = (unsigned)(j * CHUNK + tid * VEC + c);
        if (sorted) pairs[pos] = ((unsigned long long)order_key(v[j][c]) << 32) | (0xffffffffu - idx);
        else stage[pos] = (int)idx;
      }
      run_g += g ? 1u : 0u;
      run_e += e ? 1u : 0u;
    }
  }
  const unsigned n_sel = base_g + min(base_e, rem);
  if (!sorted) {
    __syncthreads();
    for (unsigned i = tid; i < k; i += THREADS) out_row[i] = (i < n_sel) ? stage[i] : -1;
    return;
  }
  const unsigned P = (unsigned)p.sort_len;
  for (unsigned i = n_sel + tid; i < P; i += THREADS) pairs[i] = 0ull;
  __syncthreads();
  for (unsigned size = 2; size <= P; size <<= 1) {
    for (unsigned stride = size >> 1; stride > 0; stride >>= 1) {
      for (unsigned t = tid; t < P / 2; t += THREADS) {
        const unsigned i = 2 * t - (t & (stride - 1));
        const unsigned jx = i + stride;
        const bool desc = (i & size) == 0;
        const unsigned long long a = pairs[i], b = pairs[jx];
        if ((a < b) == desc) { pairs[i] = b; pairs[jx] = a; }
      }
      __syncthreads();
    }
  }
  for (unsigned i = tid; i < k; i += THREADS)
    out_row[i] = (i < n_sel) ? (int)(0xffffffffu - (unsigned)(pairs[i] & 0xffffffffull)) : -1;
}

template <typename K>
int launch_kernel(K kernel, const TopkParams& p, int threads, size_t smem, hipStream_t stream) {
  if (smem > 64 * 1024 &&
      hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
    return -2;
  hipLaunchKernelGGL(kernel, dim3((unsigned)(p.rows * (p.segs > 1 ? p.segs : 1))), dim3((unsigned)threads), smem, stream, p);
  return 0;
}

template <typename ScoreT, int MODE = 0>
int launch_for_type(const TopkParams& p, bool vec4, hipStream_t stream, size_t* smem_out) {
  const int T = p.segs > 1 ? p.seg_width : p.width;      // columns one workgroup looks at
  const bool sorted = p.order == CPPMEGA_MI355_TOPK_ORDER_VALUE;
  const size_t out_words = sorted ? (size_t)p.sort_len * 2 : (size_t)p.k;
  if (T <= 32768) {
    auto tile_smem = [&](int E, int threads) {
      const size_t tile_words = (size_t)threads * E;
      // (with two histograms the second one's scan scratch, 64 words, lies behind it)
      const size_t need = (size_t)kTileScratch + (tile_two_hists(E, threads) && out_words < (size_t)kHistBins + 64 ? (size_t)kHistBins + 64 : out_words);
      return (need > tile_words ? need : tile_words) * 4;
    };
#define CM_TOPK_TILE(E, THR)                                                              \
  do {                                                                                    \
    const size_t smem = tile_smem(E, THR);                                                \
    *smem_out = smem;                                                                     \
    if (smem > 160 * 1024) return -3;                                                     \
    return vec4 ? launch_kernel(topk_tile_kernel<ScoreT, E, 4, THR, MODE, true>, p, THR, smem, stream) \
                : launch_kernel(topk_tile_kernel<ScoreT, E, 1, THR, MODE, false>, p, THR, smem, stream); \
  } while (0)
    if constexpr (MODE == 1) {                            // a segment is always kSegWidth columns wide
      CM_TOPK_TILE(16, 512);
    }
    if (T <= 1024) CM_TOPK_TILE(4, kTileThreads);
    if (T <= 2048) CM_TOPK_TILE(8, kTileThreads);
    if (T <= 4096) CM_TOPK_TILE(16, kTileThreads);
    // the widest rows: 512 threads x 16 columns (twice the wavefronts per row shorten every phase
    // of the row's pipeline, and the narrower runs need fewer registers)
    if (T <= 8192) CM_TOPK_TILE(16, 512);
    // up to 32768 columns: the same kernel on 1024 threads (half the time of the keyed-bin kernel below)
    if (T <= 16384) CM_TOPK_TILE(16, 1024);
    CM_TOPK_TILE(32, 1024);
#undef CM_TOPK_TILE
  }
  const size_t smem = ((size_t)kWideScratch + out_words) * 4;
  *smem_out = smem;
  if (smem > 160 * 1024) return -3;
  if (vec4) {
    if (T <= 32768) return launch_kernel(topk_wide_kernel<ScoreT, 8, 4>, p, kWideThreads, smem, stream);
    if (T <= 65536) return launch_kernel(topk_wide_kernel<ScoreT, 16, 4>, p, kWideThreads, smem, stream);
  } else {
    if (T <= 32768) return launch_kernel(topk_wide_kernel<ScoreT, 32, 1>, p, kWideThreads, smem, stream);
  }
  return -1;
}

}  // namespace

// Rows wider than 16384 columns are cut into segments of 8192 (the fastest single-workgroup
// shape) when the caller supplies a workspace; k must fit a segment and segs * k one stage-2 row.
constexpr int kSegWidth = 8192;
static int topk_segments(const cppmega_mi355_topk_args_t& a) {
  if (a.width <= 16384 || a.k > kSegWidth || a.width % 4 != 0 || a.row_stride % 4 != 0) return 1;
  const int segs = (a.width + kSegWidth - 1) / kSegWidth;
  if ((long long)segs * a.k > 32768 || ((long long)segs * a.k) % 4 != 0) return 1;
  return segs;
}
static size_t topk_workspace_for(const cppmega_mi355_topk_args_t& a, int segs) {
  const size_t cands = (size_t)a.rows * segs * a.k;
  return ((cands * 4 + 255) & ~(size_t)255) + cands * 4;
}

int topk_workspace_bytes(const cppmega_mi355_topk_args_t& a, size_t* bytes) {
  if (a.rows < 0 || a.width < 1 || a.k < 1 || a.k > a.width) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk: rows=%d width=%d k=%d", a.rows, a.width, a.k);
  const int segs = topk_segments(a);
  *bytes = segs > 1 ? topk_workspace_for(a, segs) : 0;
  return 0;
}

int topk_select_launch(const cppmega_mi355_topk_args_t& a, hipStream_t stream) {
  if (!a.scores || !a.indices) return fail(CPPMEGA_MI355_ERR_NULL, "topk: scores/indices is NULL");
  if (a.rows < 0 || a.width < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk: rows=%d width=%d", a.rows, a.width);
  if (a.k < 1 || a.k > a.width)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "topk must be in [1, %d]; got %d", a.width, a.k);
  if (a.row_stride < a.width) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk: row_stride %lld < width %d", (long long)a.row_stride, a.width);
  if (a.order != CPPMEGA_MI355_TOPK_ORDER_INDEX && a.order != CPPMEGA_MI355_TOPK_ORDER_VALUE)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "topk: unknown order %d", a.order);
  if (a.score_dtype != CPPMEGA_MI355_F32 && a.score_dtype != CPPMEGA_MI355_F16 && a.score_dtype != CPPMEGA_MI355_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "topk: scores must be float32, float16 or bfloat16");
  const int esz = dtype_size(a.score_dtype);
  const bool vec4 = (a.width % 4 == 0) && (a.row_stride % 4 == 0) && (((uintptr_t)a.scores) % (size_t)(4 * esz) == 0);
  if (a.width > (vec4 ? 65536 : 32768))
    return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "topk: width %d exceeds what one workgroup keeps in registers (%d)",
                a.width, vec4 ? 65536 : 32768);
  if (a.rows == 0) return 0;

  TopkParams p;
  p.scores = a.scores; p.row_stride = a.row_stride; p.starts = a.starts; p.ends = a.ends; p.out = a.indices;
  p.rows = a.rows; p.width = a.width; p.k = a.k; p.order = a.order; p.neg_inf_masked = a.neg_inf_is_masked ? 1 : 0;
  int sort_len = 2;
  while (sort_len < a.k) sort_len <<= 1;
  p.sort_len = sort_len;
  p.segs = 1; p.seg_width = 0; p.cand_val = nullptr; p.cand_idx = nullptr; p.index_map = nullptr;

  int rc;
  size_t smem = 0;
  const int segs = topk_segments(a);
  if (segs > 1 && a.workspace) {
    const size_t need = topk_workspace_for(a, segs);
    if (a.workspace_bytes < need)
      return fail(CPPMEGA_MI355_ERR_WORKSPACE, "topk: workspace of %zu bytes needed, %zu given", need, (size_t)a.workspace_bytes);
    if ((uintptr_t)a.workspace & 15) return fail(CPPMEGA_MI355_ERR_ALIGNMENT, "topk: workspace must be 16-byte aligned");
    const size_t cands = (size_t)a.rows * segs * a.k;
    // stage 1: every (row, segment) keeps its k best, ascending column (so a candidate's position
    // orders like its column and stage 2 breaks ties toward the lower column)
    TopkParams s1 = p;
    s1.segs = segs; s1.seg_width = kSegWidth; s1.order = CPPMEGA_MI355_TOPK_ORDER_INDEX;
    s1.cand_val = (float*)a.workspace;
    s1.cand_idx = (int*)((char*)a.workspace + ((cands * 4 + 255) & ~(size_t)255));
    if (a.score_dtype == CPPMEGA_MI355_F32) rc = launch_for_type<float, 1>(s1, vec4, stream, &smem);
    else if (a.score_dtype == CPPMEGA_MI355_F16) rc = launch_for_type<Half, 1>(s1, vec4, stream, &smem);
    else rc = launch_for_type<BHalf, 1>(s1, vec4, stream, &smem);
    if (rc == 0) {
      // stage 2: the bounds and the -inf rule have been applied; what is left is a plain selection
      TopkParams s2 = p;
      s2.scores = s1.cand_val; s2.row_stride = (long long)segs * a.k; s2.width = segs * a.k;
      s2.starts = nullptr; s2.ends = nullptr; s2.neg_inf_masked = 0; s2.index_map = s1.cand_idx;
      rc = launch_for_type<float, 2>(s2, true, stream, &smem);
    }
  } else if (a.score_dtype == CPPMEGA_MI355_F32) rc = launch_for_type<float>(p, vec4, stream, &smem);
  else if (a.score_dtype == CPPMEGA_MI355_F16) rc = launch_for_type<Half>(p, vec4, stream, &smem);
  else rc = launch_for_type<BHalf>(p, vec4, stream, &smem);
  if (rc == -3)
    return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "topk: k=%d with this order needs %zu bytes of LDS (limit 160 KiB)", a.k, smem);
  if (rc != 0) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "topk: no kernel for width %d (rc %d)", a.width, rc);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
