// Wavefront radix-select top-k over indexer scores (gfx950).
//
// One 64-lane wavefront owns one score row.  The row is read from HBM exactly
// once, with 16-byte loads, and stays in registers (up to 128 values per lane)
// for the rest of the kernel.  A 4096-bin histogram in LDS, private to the
// wavefront, is filled by LDS atomics and scanned by the same wavefront, so the
// kernel needs no cross-wavefront barrier.
//
// Selection (k largest, ties toward the lower index):
//   pass 1  histogram of bits[31:20] (sign, exponent, 3 mantissa bits) over the
//           selectable positions; a two-level scan, walking the bins from the
//           largest value down, finds the bin where the running count reaches k
//   pass 2  the same over bits[19:8] of the elements that fell in that bin
//   pass 3  the same over bits[7:0]
// A pass ends the search early when the bin it found has to be taken whole;
// then "x >= lowest value of the bin" describes the selected set.  Only when
// the threshold value itself is duplicated beyond what is needed does the
// emission count equal elements and keep the first `rem` of them by index.
//
// Emission is a ballot/mbcnt compaction in ascending index order; the optional
// value-descending order sorts the selected (value, index) pairs in LDS.
//
// Float compares give the ordering: -0.0 == +0.0, and NaN (which also stands
// for "outside [start,end)") never compares true, so it is never selected.

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
};

template <typename T>
struct ScoreLoad;
template <>
struct ScoreLoad<float> {
  static __device__ __forceinline__ void vec4(const float* p, float (&o)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
  }
  static __device__ __forceinline__ float one(const float* p) { return *p; }
};
struct Half {};   // tag types: 16-bit storage
struct BHalf {};
template <>
struct ScoreLoad<Half> {
  static __device__ __forceinline__ void vec4(const unsigned short* p, float (&o)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    o[0] = f16_bits_to_f32((unsigned short)(t.x & 0xffffu));
    o[1] = f16_bits_to_f32((unsigned short)(t.x >> 16));
    o[2] = f16_bits_to_f32((unsigned short)(t.y & 0xffffu));
    o[3] = f16_bits_to_f32((unsigned short)(t.y >> 16));
  }
  static __device__ __forceinline__ float one(const unsigned short* p) { return f16_bits_to_f32(*p); }
};
template <>
struct ScoreLoad<BHalf> {
  static __device__ __forceinline__ void vec4(const unsigned short* p, float (&o)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    o[0] = __uint_as_float(t.x << 16);
    o[1] = __uint_as_float(t.x & 0xffff0000u);
    o[2] = __uint_as_float(t.y << 16);
    o[3] = __uint_as_float(t.y & 0xffff0000u);
  }
  static __device__ __forceinline__ float one(const unsigned short* p) { return bf16_bits_to_f32(*p); }
};
template <typename T> struct Storage { typedef unsigned short type; };
template <> struct Storage<float> { typedef float type; };

struct BinHit {
  unsigned bin;    // raw bin index in the histogram
  unsigned above;  // elements in bins that rank before it
  unsigned cnt;    // elements in it
  unsigned total;  // elements in all bins
};

// Walk order of the bins, largest value first:
//   kSigned      bin = bits[31:20]: non-negative bins 2047..0, then negative bins 2048..4095
//   kDescending  larger digit = larger value  (non-negative prefix)
//   kAscending   larger digit = smaller value (negative prefix)
enum { kSigned = 0, kDescending = 1, kAscending = 2 };

template <int NB>
__device__ __forceinline__ void lane_block(int lane, int mode, int& blk, bool& rev) {
  // NB/64 consecutive walk positions per lane map to one aligned block in memory.
  if (mode == kSigned) {
    if (lane < 32) { blk = 31 - lane; rev = true; } else { blk = lane; rev = false; }
  } else if (mode == kDescending) {
    blk = 63 - lane; rev = true;
  } else {
    blk = lane; rev = false;
  }
}

// Finds the bin at which the running count, walking from the largest value
// down, first reaches `need` (1 <= need <= total is the caller's business; if
// need > total the hit is meaningless and only `total` may be used).
template <int NB>
__device__ BinHit find_bin(const unsigned* hist, unsigned need, int mode) {
  constexpr int L = NB / 64;
  static_assert(L >= 1 && L <= 64 && (L % 4 == 0), "bins per lane");
  const int lane = lane_id();
  int blk; bool rev;
  lane_block<NB>(lane, mode, blk, rev);
  unsigned sum = 0;
  const uint4* src = reinterpret_cast<const uint4*>(hist + blk * L);
#pragma unroll
  for (int i = 0; i < L / 4; ++i) {
    const uint4 t = src[i];
    sum += t.x + t.y + t.z + t.w;
  }
  const unsigned incl = wave_inclusive_sum(sum);
  BinHit hit;
  hit.total = __shfl(incl, 63, 64);
  const unsigned long long m1 = __ballot(incl >= need);
  const int lx = m1 ? __builtin_ctzll(m1) : 63;
  const unsigned above_lane = __shfl(incl - sum, lx, 64);
  int blkx; bool revx;
  lane_block<NB>(lx, mode, blkx, revx);
  const int slot = revx ? (L - 1 - lane) : lane;
  const unsigned c = (lane < L) ? hist[blkx * L + slot] : 0u;
  const unsigned incl2 = wave_inclusive_sum(c);
  const unsigned long long m2 = __ballot(lane < L && above_lane + incl2 >= need);
  const int ix = m2 ? __builtin_ctzll(m2) : 0;
  hit.bin = (unsigned)(blkx * L + (revx ? (L - 1 - ix) : ix));
  hit.above = above_lane + __shfl(incl2 - c, ix, 64);
  hit.cnt = __shfl(c, ix, 64);
  return hit;
}

__device__ __forceinline__ void zero_hist(unsigned* hist, int lane) {
  uint4* dst = reinterpret_cast<uint4*>(hist);
  const uint4 z = make_uint4(0, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < kHistBins / 4 / 64; ++i) dst[i * 64 + lane] = z;
}

// Monotone key of a float: larger value <=> larger key.
__device__ __forceinline__ unsigned order_key(float x) {
  const unsigned u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Compaction of the selected elements, ascending by index.
//   TIE == false: selected <=> x >= thr
//   TIE == true : selected <=> x > thr, or x == thr and fewer than `rem`
//                 equal elements precede it
// SORTED == false: out_row[pos] = index.   SORTED == true: pairs[pos] = key.
template <int ITEMS, int VEC, bool TIE, bool SORTED>
__device__ __forceinline__ unsigned emit(const float (&v)[ITEMS][VEC], float thr, unsigned rem,
                                         int* out_row, unsigned long long* pairs) {
  const int lane = lane_id();
  unsigned base_g = 0, base_e = 0;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    bool g[VEC], e[VEC];
    unsigned pre_g = 0, pre_e = 0, tot_g = 0, tot_e = 0;
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      const float x = v[j][c];
      g[c] = TIE ? (x > thr) : (x >= thr);
      const unsigned long long mg = __ballot(g[c]);
      pre_g += mbcnt(mg);
      tot_g += (unsigned)__popcll(mg);
      if (TIE) {
        e[c] = (x == thr);
        const unsigned long long me = __ballot(e[c]);
        pre_e += mbcnt(me);
        tot_e += (unsigned)__popcll(me);
      } else {
        e[c] = false;
      }
    }
    if (tot_g + tot_e) {
      unsigned run_g = base_g + pre_g, run_e = base_e + pre_e;
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        const bool sel = g[c] || (TIE && e[c] && run_e < rem);
        const unsigned pos = run_g + (TIE ? min(run_e, rem) : 0u);
        if (sel) {
          const unsigned idx = (unsigned)((j * 64 + lane) * VEC + c);
          if (SORTED) {
            pairs[pos] = ((unsigned long long)order_key(v[j][c]) << 32) | (0xffffffffu - idx);
          } else {
            out_row[pos] = (int)idx;
          }
        }
        run_g += g[c] ? 1u : 0u;
        if (TIE) run_e += e[c] ? 1u : 0u;
      }
    }
    base_g += tot_g;
    base_e += tot_e;
  }
  return base_g + (TIE ? min(base_e, rem) : 0u);
}

template <typename ScoreT, int ITEMS, int VEC>
__global__ __launch_bounds__(64) void topk_wave_kernel(const TopkParams p) {
  extern __shared__ __align__(16) unsigned smem[];
  unsigned* hist = smem;
  typedef typename Storage<ScoreT>::type St;

  const int lane = lane_id();
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

  // ---- the row: HBM -> registers, once -----------------------------------
  float v[ITEMS][VEC];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int chunk_lo = j * 64 * VEC;
    const int base = chunk_lo + lane * VEC;
    if (chunk_lo >= end || chunk_lo + 64 * VEC <= start) {   // uniform: nothing selectable here
#pragma unroll
      for (int c = 0; c < VEC; ++c) v[j][c] = kNaN;
    } else if constexpr (VEC == 4) {
      if (base < T) {
        ScoreLoad<ScoreT>::vec4(src + base, v[j]);
      } else {
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[j][c] = kNaN;
      }
    } else {
      v[j][0] = (base < T) ? ScoreLoad<ScoreT>::one(src + base) : kNaN;
    }
  }
  zero_hist(hist, lane);

  // ---- canonicalise: -0 -> +0, signalling NaN -> quiet NaN, mask -> NaN -----
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int chunk_lo = j * 64 * VEC;
    const bool inside = chunk_lo >= start && chunk_lo + 64 * VEC <= end;   // uniform
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      float x = v[j][c] + 0.0f;
      if (!inside) {
        const int idx = chunk_lo + lane * VEC + c;
        x = (idx >= start && idx < end) ? x : kNaN;
      }
      if (p.neg_inf_masked) x = (x == kNegInf) ? kNaN : x;
      v[j][c] = x;
    }
  }
  __syncthreads();

  // ---- pass 1: bits[31:20] ---------------------------------------------------
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      const float x = v[j][c];
      if (x == x) atomicAdd(&hist[__float_as_uint(x) >> 20], 1u);
    }
  }
  __syncthreads();

  const unsigned k = (unsigned)p.k;
  BinHit h1 = find_bin<kHistBins>(hist, k, kSigned);
  float thr;
  unsigned rem = 0;
  bool tie = false;
  if (h1.total <= k) {
    thr = kNegInf;   // every selectable element is taken
  } else {
    unsigned lo_bits;
    const bool neg = (h1.bin & 0x800u) != 0;
    rem = k - h1.above;
    if (rem == h1.cnt) {
      lo_bits = (h1.bin << 20) | (neg ? 0x000fffffu : 0u);
    } else {
      // ---- pass 2: bits[19:8] of the elements in bin h1 --------------------
      __syncthreads();
      zero_hist(hist, lane);
      __syncthreads();
      const unsigned p1 = h1.bin;
#pragma unroll
      for (int j = 0; j < ITEMS; ++j) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
          const unsigned u = __float_as_uint(v[j][c]);
          if ((u >> 20) == p1) atomicAdd(&hist[(u >> 8) & 0xfffu], 1u);
        }
      }
      __syncthreads();
      const BinHit h2 = find_bin<kHistBins>(hist, rem, neg ? kAscending : kDescending);
      rem -= h2.above;
      const unsigned p2 = (p1 << 12) | h2.bin;     // bits[31:8]
      if (rem == h2.cnt) {
        lo_bits = (p2 << 8) | (neg ? 0xffu : 0u);
      } else {
        // ---- pass 3: bits[7:0] ------------------------------------------------
        __syncthreads();
        if (lane < 64) reinterpret_cast<uint4*>(hist)[lane] = make_uint4(0, 0, 0, 0);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
#pragma unroll
          for (int c = 0; c < VEC; ++c) {
            const unsigned u = __float_as_uint(v[j][c]);
            if ((u >> 8) == p2) atomicAdd(&hist[u & 0xffu], 1u);
          }
        }
        __syncthreads();
        const BinHit h3 = find_bin<256>(hist, rem, neg ? kAscending : kDescending);
        rem -= h3.above;
        lo_bits = (p2 << 8) | h3.bin;
        tie = rem != h3.cnt;
      }
    }
    // bins above 0xff800000 hold only NaN patterns: the lowest real value is -inf
    if (lo_bits > 0xff800000u) lo_bits = 0xff800000u;
    thr = __uint_as_float(lo_bits);
  }
  __syncthreads();   // the histogram memory is reused by the sorted emission

  // ---- emission ---------------------------------------------------------------
  unsigned n_sel;
  unsigned long long* pairs = reinterpret_cast<unsigned long long*>(smem);
  if (p.order == CPPMEGA_MI355_TOPK_ORDER_INDEX) {
    n_sel = tie ? emit<ITEMS, VEC, true, false>(v, thr, rem, out_row, pairs)
                : emit<ITEMS, VEC, false, false>(v, thr, rem, out_row, pairs);
    for (unsigned i = n_sel + lane; i < k; i += 64) out_row[i] = -1;
    return;
  }

  n_sel = tie ? emit<ITEMS, VEC, true, true>(v, thr, rem, out_row, pairs)
              : emit<ITEMS, VEC, false, true>(v, thr, rem, out_row, pairs);
  const unsigned P = (unsigned)p.sort_len;
  for (unsigned i = n_sel + lane; i < P; i += 64) pairs[i] = 0ull;   // sorts last
  __syncthreads();
  // bitonic sort, descending: larger value first, then lower index
  for (unsigned size = 2; size <= P; size <<= 1) {
    for (unsigned stride = size >> 1; stride > 0; stride >>= 1) {
      for (unsigned t = lane; t < P / 2; t += 64) {
        const unsigned i = 2 * t - (t & (stride - 1));
        const unsigned jx = i + stride;
        const bool desc = (i & size) == 0;
        const unsigned long long a = pairs[i], b = pairs[jx];
        if ((a < b) == desc) { pairs[i] = b; pairs[jx] = a; }
      }
      __syncthreads();
    }
  }
  for (unsigned i = lane; i < k; i += 64)
    out_row[i] = (i < n_sel) ? (int)(0xffffffffu - (unsigned)(pairs[i] & 0xffffffffull)) : -1;
}

template <typename ScoreT>
int launch_for_type(const TopkParams& p, bool vec4, size_t smem, hipStream_t stream) {
  const dim3 grid((unsigned)p.rows), block(64);
  const int T = p.width;
#define CM_TOPK_LAUNCH(ITEMS, VEC)                                                        \
  do {                                                                                    \
    hipLaunchKernelGGL((topk_wave_kernel<ScoreT, ITEMS, VEC>), grid, block, smem, stream, p); \
    return 0;                                                                             \
  } while (0)
  if (vec4) {
    if (T <= 512) CM_TOPK_LAUNCH(2, 4);
    if (T <= 2048) CM_TOPK_LAUNCH(8, 4);
    if (T <= 8192) CM_TOPK_LAUNCH(32, 4);
  } else {
    if (T <= 512) CM_TOPK_LAUNCH(8, 1);
    if (T <= 2048) CM_TOPK_LAUNCH(32, 1);
    if (T <= 8192) CM_TOPK_LAUNCH(128, 1);
  }
#undef CM_TOPK_LAUNCH
  return -1;
}

}  // namespace

int topk_select_launch(const cppmega_mi355_topk_args_t& a, hipStream_t stream) {
  if (!a.scores || !a.indices) return fail(CPPMEGA_MI355_ERR_NULL, "topk: scores/indices is NULL");
  if (a.rows < 0 || a.width < 1) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk: rows=%d width=%d", a.rows, a.width);
  if (a.k < 1 || a.k > a.width)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "topk must be in [1, %d]; got %d", a.width, a.k);
  if (a.row_stride < a.width) return fail(CPPMEGA_MI355_ERR_SHAPE, "topk: row_stride %lld < width %d", (long long)a.row_stride, a.width);
  if (a.order != CPPMEGA_MI355_TOPK_ORDER_INDEX && a.order != CPPMEGA_MI355_TOPK_ORDER_VALUE)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "topk: unknown order %d", a.order);
  if (a.width > 8192)
    return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "topk: width %d exceeds the 8192 a wavefront keeps in registers", a.width);
  if (a.rows == 0) return 0;

  const int esz = dtype_size(a.score_dtype);
  if (a.score_dtype != CPPMEGA_MI355_F32 && a.score_dtype != CPPMEGA_MI355_F16 && a.score_dtype != CPPMEGA_MI355_BF16)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "topk: scores must be float32, float16 or bfloat16");
  const bool vec4 = (a.width % 4 == 0) && (a.row_stride % 4 == 0) && (((uintptr_t)a.scores) % (size_t)(4 * esz) == 0);

  TopkParams p;
  p.scores = a.scores; p.row_stride = a.row_stride; p.starts = a.starts; p.ends = a.ends; p.out = a.indices;
  p.rows = a.rows; p.width = a.width; p.k = a.k; p.order = a.order; p.neg_inf_masked = a.neg_inf_is_masked ? 1 : 0;
  int sort_len = 2;
  while (sort_len < a.k) sort_len <<= 1;
  p.sort_len = sort_len;
  size_t smem = (size_t)kHistBins * 4;
  if (a.order == CPPMEGA_MI355_TOPK_ORDER_VALUE && (size_t)sort_len * 8 > smem) smem = (size_t)sort_len * 8;

  int rc;
  if (a.score_dtype == CPPMEGA_MI355_F32) rc = launch_for_type<float>(p, vec4, smem, stream);
  else if (a.score_dtype == CPPMEGA_MI355_F16) rc = launch_for_type<Half>(p, vec4, smem, stream);
  else rc = launch_for_type<BHalf>(p, vec4, smem, stream);
  if (rc != 0) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "topk: no kernel for width %d", a.width);
  CM_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // namespace cm
