/*
 * cppmega_mi355.h -- C ABI of the MI355X (gfx950) sparse-attention hot path.
 *
 * One shared library, libcppmega_mi355.so, exports the entry points below.
 * They are what a binding of the reference's kernel boundary would call in
 * place of the TileLang/TVM-FFI artefacts it compiles today.  Conventions are
 * taken from the reference's only native C ABI,
 * cppmega_mlx/nn/_tilelang/native_bridge/tilelang_mlx_tvm_ffi_bridge.h:18-39:
 *
 *   - every call takes a pointer to a plain struct plus sizeof(struct); the
 *     struct starts with `struct_size` so old callers keep working when fields
 *     are appended;
 *   - the return value is an int status, 0 = ok (1 = null argument,
 *     2 = struct too small, as in tilelang_mlx_tvm_ffi_bridge.cpp:33-69);
 *   - outputs are caller-owned ("owner-output", reference AGENTS.md:3-20):
 *     the library never allocates, copies or casts a tensor.  The only device
 *     memory beyond inputs and outputs is an optional caller-provided
 *     workspace whose size the matching *_workspace_bytes() call reports;
 *   - all pointers are device pointers unless stated; tensors are dense and
 *     row-major with the shapes given per field; work is enqueued on `stream`
 *     (a hipStream_t, passed as void*; NULL = the default stream) and the call
 *     returns without synchronising.
 */
#ifndef CPPMEGA_MI355_H_
#define CPPMEGA_MI355_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CPPMEGA_MI355_ABI_VERSION 1

/* ---- status codes -------------------------------------------------------- */
enum {
  CPPMEGA_MI355_OK = 0,
  CPPMEGA_MI355_ERR_NULL = 1,          /* a required pointer is NULL            */
  CPPMEGA_MI355_ERR_STRUCT_SIZE = 2,   /* args_size smaller than this ABI needs  */
  CPPMEGA_MI355_ERR_SHAPE = 3,         /* shape / value contract -> ValueError   */
  CPPMEGA_MI355_ERR_DTYPE = 4,         /* unsupported dtype combo -> TypeError   */
  CPPMEGA_MI355_ERR_UNSUPPORTED = 5,   /* valid request, no kernel for it        */
  CPPMEGA_MI355_ERR_WORKSPACE = 6,     /* workspace missing or too small         */
  CPPMEGA_MI355_ERR_LAUNCH = 7,        /* HIP reported a launch/runtime error    */
  CPPMEGA_MI355_ERR_ALIGNMENT = 8      /* pointer or stride misaligned           */
};

/* ---- element types ------------------------------------------------------- */
enum {
  CPPMEGA_MI355_F32 = 0,
  CPPMEGA_MI355_F16 = 1,
  CPPMEGA_MI355_BF16 = 2,
  CPPMEGA_MI355_E4M3 = 3,   /* OCP e4m3fn bytes (uint8 storage)                */
  CPPMEGA_MI355_I32 = 4,
  CPPMEGA_MI355_I64 = 5
};

/* ---- how a quantised operand is scaled ----------------------------------- */
enum {
  CPPMEGA_MI355_SCALE_NONE = 0,       /* float carrier, no scale                */
  CPPMEGA_MI355_SCALE_PER_TOKEN = 1,  /* float32, one per row     [..rows]      */
  CPPMEGA_MI355_SCALE_E8M0 = 2,       /* uint8 E8M0, one per `block` elements   */
  CPPMEGA_MI355_SCALE_F32_BLOCK = 3   /* float32,    one per `block` elements   */
};

/* Probe: replaces cppmega_tilelang_mlx_tvm_ffi_bridge_probe
 * (native_bridge/tilelang_mlx_tvm_ffi_bridge.h:18-39).  Host memory. */
typedef struct cppmega_mi355_status {
  uint32_t struct_size;
  int32_t abi_version;
  int32_t device_count;       /* HIP devices visible, 0 when none            */
  int32_t gfx950_devices;     /* how many of them report gcnArchName gfx950  */
  char built_for[32];         /* offload arch the kernels were compiled for  */
  char message[160];
} cppmega_mi355_status_t;

int cppmega_mi355_status(cppmega_mi355_status_t* out, size_t out_size);

/* Static text for a status code (host memory, never NULL). */
const char* cppmega_mi355_error_string(int code);

/* After a non-zero return: detail of the last failure on the calling thread. */
const char* cppmega_mi355_last_error(void);

/* ---- top-k selector --------------------------------------------------------
 * Replaces the kernel compiled by _path_c_tvm_ffi_kernel_for and called as
 * kernel(ends, indices, scores, starts)
 * (cppmega_mlx/nn/_tilelang/topk_selector.py:522-629, 655-674, 771), and the
 * masked rows that path sends to topk_selector_reference (:227-330, 728-733).
 *
 * Per row: the k largest of scores[row, clip(start) .. clip(end)), ties
 * toward the lower index; slots past the number of selectable positions hold
 * -1.  NaN scores are never selected.
 */
enum { CPPMEGA_MI355_TOPK_ORDER_INDEX = 0, CPPMEGA_MI355_TOPK_ORDER_VALUE = 1 };

typedef struct cppmega_mi355_topk_args {
  uint32_t struct_size;
  int32_t score_dtype;        /* F32, F16 or BF16                              */
  const void* scores;         /* [rows, width], row pitch = row_stride elems   */
  int64_t row_stride;
  int32_t rows;
  int32_t width;
  int32_t k;                  /* 1 <= k <= width                               */
  int32_t order;              /* ORDER_INDEX: ascending index; ORDER_VALUE:
                                 value descending, lower index first           */
  const int32_t* starts;      /* [rows] or NULL (= 0)                          */
  const int32_t* ends;        /* [rows] or NULL (= width)                      */
  int32_t* indices;           /* out [rows, k], dense                          */
  int32_t neg_inf_is_masked;  /* non-zero: an in-range -inf is unselectable    */
  int32_t reserved;

  /* Appended after the first ABI (a caller whose struct_size ends at `reserved`
   * gets NULL / 0). */
  void* workspace;            /* optional, uninitialised: with *_workspace_bytes of it,
                               * rows wider than 16384 columns are selected in two
                               * stages (k best of every 8192-column segment, then k of
                               * those), one workgroup per segment instead of one per
                               * row; same result                               */
  size_t workspace_bytes;
} cppmega_mi355_topk_args_t;

#define CPPMEGA_MI355_TOPK_ARGS_V1_SIZE (offsetof(cppmega_mi355_topk_args_t, workspace))

int cppmega_mi355_topk_select(const cppmega_mi355_topk_args_t* args, size_t args_size, void* stream);

/* Bytes of workspace that let cppmega_mi355_topk_select take the two-stage path for this
 * shape (0 when it has none: narrow rows, k above 8192 or 32768 / segments). */
int cppmega_mi355_topk_workspace_bytes(const cppmega_mi355_topk_args_t* args, size_t args_size, size_t* bytes);

/* ---- indexer scores -> top-k -------------------------------------------------
 * The score and selection tail of the reference's LightningIndexer.__call__
 * (cppmega_v4/nn/lightning_indexer.py:132-145; the FP8 variant has the same
 * lines, cppmega_v4/nn/lightning_indexer_fp8.py:145-157):
 *   scores[b,s,t]  = sm_scale * sum_h weights[b,s,h] * sum_d q[b,s,h,d] * k[b,t,d]
 *                    (+ mask[b,s,t])
 *   indices[b,s,:] = the topk largest of scores[b,s,:]
 *   q        [B, Sq, H, D]   float32 or bfloat16 (D <= 256)
 *   weights  [B, Sq, H]      float32 or bfloat16 (the caller has applied H^-1/2)
 *   k        [B, Skv, D]     float32 or bfloat16
 *   mask     [B, Sq, Skv]    additive, float32/float16/bfloat16, or NULL
 *   starts, ends  [B*Sq] int32 or NULL: selectable window per query row, as in
 *            cppmega_mi355_topk_select (a causal bound costs no mask read)
 *   indices  [B, Sq, topk] int32.  Selection rule of cppmega_mi355_topk_select:
 *            value descending, ties toward the lower index; a slot beyond the
 *            selectable entries of a row holds -1 (with a mask, an entry whose
 *            score is -inf is not selectable; the reference's argpartition picks
 *            arbitrary masked positions there).
 * The [B,Sq,Skv] score matrix is not kept: rows are scored and selected a chunk at
 * a time through `workspace` (*_workspace_bytes; 256 MiB of scores per pass by
 * default, `chunk_rows` overrides the rows per pass; the head-summed queries of a
 * pass live there too).  When `scores_out` is set every score is written there
 * instead (float32 [B,Sq,Skv], 16-byte aligned) in one pass and the selection
 * reads exactly those values; the workspace then only holds the summed queries. */
typedef struct cppmega_mi355_indexer_args {
  uint32_t struct_size;
  int32_t q_dtype;
  const void* q;
  const void* weights;
  const void* k;
  const void* mask;
  int32_t w_dtype;
  int32_t k_dtype;
  int32_t mask_dtype;
  int32_t order;              /* CPPMEGA_MI355_TOPK_ORDER_*                    */
  const int32_t* starts;
  const int32_t* ends;
  int32_t batch, seq_q, heads, head_dim, seq_kv, topk;
  float sm_scale;
  int32_t chunk_rows;         /* 0 = the library's choice                      */
  int32_t* indices;
  float* scores_out;
  void* workspace;
  size_t workspace_bytes;
} cppmega_mi355_indexer_args_t;

int cppmega_mi355_indexer_topk_workspace_bytes(const cppmega_mi355_indexer_args_t* args, size_t args_size,
                                               size_t* bytes);
int cppmega_mi355_indexer_topk(const cppmega_mi355_indexer_args_t* args, size_t args_size, void* stream);

/* ---- sparse MLA forward ----------------------------------------------------
 * One entry point for the three prepared-buffer kernels of the reference and
 * the float-carrier one:
 *   blockscaled_sparse_mla_apply_kernel  (q_fp8,q_scale,kv_fp8,kv_scale,indices,
 *       sm_scale_buf,out,lse)  sparse_mla_blockscaled_path_c.py:1054-1164
 *   fp8_sparse_mla_apply_kernel (.., sinks, has_sinks, out, lse)
 *       sparse_mla_fp8_path_c.py:1821-1956
 *   sparse_mla_fwd_direct (indices,kv,lse,out,q,sm_scale_buf)
 *       sparse_mla_path_c.py:2291-2382
 * and for the pure-MLX fallback they are checked against
 * (cppmega_mlx/nn/sparse_mla.py:125-210).
 *
 *   q        [B, S, H, d_qk]
 *   kv       [B, Skv, G, d_kv]      d_kv = d_qk - rope_dim
 *   kv_rope  [B, Skv, G, rope_dim]  optional tail of every key row (QK only)
 *   indices  [B, S, G, topk]        entry < 0 or >= Skv is skipped
 *   out      [B, S, H, d_v]         d_v <= d_kv: V = first d_v channels of kv
 *   lse      [B, S, H] float32, natural log, includes sm_scale; 0 for a row
 *            with nothing to attend to.  May be NULL.
 *   sinks    [H] float32 or NULL: one extra logit per head that joins the
 *            max and the denominator and carries no value row.
 * Scales: *_scale_kind says how q / kv bytes are scaled; per-token scales are
 * [B,S,H] / [B,Skv,G]; block scales are [.., d/block].
 */
enum {
  CPPMEGA_MI355_MLA_KERNEL_AUTO = 0,
  CPPMEGA_MI355_MLA_KERNEL_SCALAR = 1,   /* one wavefront per (b,s,h), fp32 VALU */
  CPPMEGA_MI355_MLA_KERNEL_MFMA = 2      /* head-batched MFMA, split-KV: d_qk 576, d_v 512; latent cache, 16-bit rows, or FP8 rows with per-token / E8M0 scales */
};

typedef struct cppmega_mi355_sparse_mla_args {
  uint32_t struct_size;
  int32_t kernel;             /* CPPMEGA_MI355_MLA_KERNEL_*                    */

  const void* q;
  const void* q_scale;        /* NULL when q_scale_kind == SCALE_NONE          */
  int32_t q_dtype;            /* F32/F16/BF16/E4M3                             */
  int32_t q_scale_kind;
  int32_t q_scale_block;      /* elements per scale for the block kinds        */

  int32_t kv_dtype;
  const void* kv;
  const void* kv_scale;
  int32_t kv_scale_kind;
  int32_t kv_scale_block;

  const void* kv_rope;        /* NULL when rope_dim == 0                       */
  int32_t rope_dtype;         /* F32/F16/BF16                                  */
  int32_t rope_dim;

  const void* indices;
  int32_t index_dtype;        /* I32 or I64                                    */

  int32_t batch, seq_q, heads, kv_groups, seq_kv, topk;
  int32_t d_qk;               /* width of a q row                              */
  int32_t d_v;
  float sm_scale;

  const float* sinks;
  void* out;
  float* lse;
  int32_t out_dtype;          /* F32/F16/BF16                                  */
  int32_t reserved;

  void* workspace;            /* split-KV partials; see *_workspace_bytes      */
  size_t workspace_bytes;

  /* Fields below were added after the first ABI; a caller whose struct_size
   * ends at workspace_bytes gets zeros for them. */
  const float* sm_scale_dev;  /* device float32[1] or NULL.  When set the kernels
                               * read the softmax scale from it on the stream
                               * (the reference's `sm_scale_buf` parameter) and
                               * `sm_scale` above is ignored.                   */
  const int32_t* has_sinks_dev; /* device int32[1] or NULL.  When set and the
                               * value is 0, `sinks` is ignored (the `has_sinks`
                               * buffer of sparse_mla_fp8_path_c.py:1821-1835).  */
  int32_t seq_kv_pitch;       /* key rows between two batches of kv / kv_scale /
                               * kv_rope; 0 = seq_kv.  Lets a cache buffer of
                               * capacity `pitch` be attended over its first
                               * seq_kv rows (entries >= seq_kv are skipped).   */
  int32_t reserved2;
} cppmega_mi355_sparse_mla_args_t;

/* struct_size of the first ABI of the struct above (through workspace_bytes). */
#define CPPMEGA_MI355_SPARSE_MLA_ARGS_V1_SIZE (offsetof(cppmega_mi355_sparse_mla_args_t, sm_scale_dev))

/* Bytes of workspace cppmega_mi355_sparse_mla_fwd needs for these shapes with
 * the kernel it would pick (0 when none).  Only the shape / dtype / kernel
 * fields are read.  Returns a status code; the size goes to *bytes. */
int cppmega_mi355_sparse_mla_workspace_bytes(const cppmega_mi355_sparse_mla_args_t* args,
                                             size_t args_size, size_t* bytes);

int cppmega_mi355_sparse_mla_fwd(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size,
                                 void* stream);

/* cppmega_mi355_sparse_mla_fwd for callers that cannot allocate device memory or
 * carry a workspace around (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments, kernels and results as cppmega_mi355_sparse_mla_fwd, but the
 * split-KV partials go to a fixed array of CPPMEGA_MI355_NOALLOC_SCRATCH_BYTES that
 * is part of the library image on every GPU the library runs on; `workspace` and
 * `workspace_bytes` of args are ignored, and the call allocates nothing.  A request
 * whose *_workspace_bytes exceeds the array fails with CPPMEGA_MI355_ERR_WORKSPACE
 * before anything is launched.  All calls on one GPU share that GPU's array, whose
 * contents are undefined between calls (nothing in it has to start at zero): two
 * calls that overlap in time on one GPU, on different streams, race; calls on one
 * stream, or otherwise ordered, do not. */
#define CPPMEGA_MI355_NOALLOC_SCRATCH_BYTES (20u << 20)
int cppmega_mi355_sparse_mla_fwd_noalloc(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size,
                                         void* stream);

/* Which kernel AUTO resolves to for these shapes (CPPMEGA_MI355_MLA_KERNEL_*),
 * or a negative status code. */
int cppmega_mi355_sparse_mla_select_kernel(const cppmega_mi355_sparse_mla_args_t* args,
                                           size_t args_size);

/* Scores only: scores[b, s, h, j] = sm_scale * q . key(indices[b, s, g, j]), float32
 * [B, S, H, topk]; a skipped slot holds -3.4028234663852886e38 (the most negative
 * finite float32).  Replaces the QK-only kernels the reference keeps as test seams:
 * fp8_sparse_mla_indexed_qk_reduce_path_c
 * (cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:1611-1690, sentinel :80).
 * `out`, `lse`, `sinks`, `d_v` (any valid value) and `workspace` of args are ignored. */
int cppmega_mi355_sparse_mla_scores(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size,
                                    float* scores, void* stream);

/* ---- sparse MLA backward ---------------------------------------------------------
 * Replaces sparse_mla_bwd_direct, called as kernel(d_out, indices, kv, q, sm_scale_buf,
 * out=(dkv, dq)) (cppmega_mlx/nn/_tilelang/sparse_mla_path_c.py:2644-2816, 3314-3421),
 * its per-token FP8 form fp8_sparse_mla_bwd_kernel(q_fp8, q_scale, kv_fp8, kv_scale,
 * d_out, indices, sm_scale_buf, dq_dequant, dkv_dequant)
 * (sparse_mla_fp8_path_c.py:1966-2214, 3007-3080), and the dkv clearing kernels in
 * front of them (sparse_mla_path_c.py:3163-3230, sparse_mla_fp8_path_c.py:2217-2272):
 *   dq  [B, S, H, d_qk]      gradient of q, float32 / float16 / bfloat16
 *   dkv [B, Skv, G, d_qk]    gradient of the KV rows, float32, accumulated with atomic
 *                            adds; cleared first when clear_dkv is non-zero
 * for out = softmax(sm_scale * q . K_sel^T) . K_sel[:, :d_v] and the cotangent d_out
 * [B, S, H, d_v].  q, kv: float32 / float16 / bfloat16, or e4m3 bytes with per-token
 * float32 scales q_scale [B,S,H] / kv_scale [B,Skv,G] (gradients are then with respect
 * to the dequantised values); d_out a float carrier; everything dense; an index < 0 or
 * >= Skv is skipped; a row with nothing to attend to contributes zero gradients. */
typedef struct cppmega_mi355_sparse_mla_bwd_args {
  uint32_t struct_size;
  int32_t q_dtype;
  const void* q;
  const void* kv;
  const void* d_out;
  const void* indices;
  int32_t kv_dtype, d_out_dtype, dq_dtype, index_dtype;
  int32_t batch, seq_q, heads, kv_groups, seq_kv, topk, d_qk, d_v;
  float sm_scale;
  int32_t clear_dkv;
  const float* sm_scale_dev;  /* device float32[1] read in place of sm_scale, or NULL */
  void* dq;
  float* dkv;
  const float* q_scale;       /* e4m3 q only */
  const float* kv_scale;      /* e4m3 kv only */
} cppmega_mi355_sparse_mla_bwd_args_t;

int cppmega_mi355_sparse_mla_bwd(const cppmega_mi355_sparse_mla_bwd_args_t* args, size_t args_size, void* stream);

/* ---- DSA indexer KL loss, per position ---------------------------------------------
 * Replaces the two kernels behind dsa_splitk_indexer_loss_tilelang
 * (cppmega_mlx/nn/_tilelang/dsa_splitk_indexer_loss.py: dsa_stage1 :398-656, dsa_stage2
 * :855-1165, called at :1514-1570):
 *   loss[b, sq] = sum_{j <= sq} p[j] * (log(p[j] + 1e-10) - log(q[j] + 1e-10))
 *   p = head average of the causal attention softmax of softmax_scale * query . key
 *       (+ index_mask), q = softmax over all keys of index_scores (+ index_mask)
 *   query [ASq, AB, AH, AD], key [Sk, AB, AH, AD]: float32 / float16 / bfloat16
 *   index_scores, index_mask [AB, ASq, Sk] float32 (index_mask NULL = no additive mask)
 *   topk_indices [AB, ASq, topk] int32 / int64 or NULL: the sparse loss.  A key that is not
 *       in its row's list counts as masked with -inf, which is what the reference's
 *       scatter(-inf, topk_indices, 0) mask (:1443-1445) adds, without the [AB, ASq, Sk]
 *       tensor; entries outside [0, Sk) select nothing; topk must be >= 1.
 *   loss [AB, ASq] float32.  The caller takes mean(loss) * loss_coeff. */
typedef struct cppmega_mi355_dsa_loss_args {
  uint32_t struct_size;
  int32_t in_dtype;
  const void* query;
  const void* key;
  const float* index_scores;
  const float* index_mask;
  float* loss;
  int32_t seq_q, batch, heads, head_dim, seq_k;
  float softmax_scale;
  const void* topk_indices;
  int32_t topk;
  int32_t index_dtype;
} cppmega_mi355_dsa_loss_args_t;

int cppmega_mi355_dsa_indexer_loss(const cppmega_mi355_dsa_loss_args_t* args, size_t args_size, void* stream);

/* ---- FP8 vecmat / skinny GEMM ----------------------------------------------
 * Replaces fp8_vecmat_reduce_direct, called as kernel(A, A_scale, B, B_scale, C)
 * (cppmega_mlx/nn/_tilelang/fp8_vecmat_path_c.py:737-821, 1039-1046) and the
 * inline kernel of fused_fp8_gemm (cppmega_v4/_tilelang/fused_fp8_gemm.py:83-142).
 *
 *   out[m, n] = sum_k dec(w[n, k]) * w_scale(n, k) * x(m, k)     fp32 accumulate
 *   w        [N, K] e4m3 bytes ("already transposed" weight)
 *   x        [M, K]: E4M3 bytes with one float32 scale_x (x(m,k) =
 *            dec(x)*scale_x[0]), or F32/F16/BF16 with scale_x == NULL
 *   out      [M, N] F32/F16/BF16
 */
enum {
  CPPMEGA_MI355_WSCALE_SCALAR = 0,     /* float32 [1]                           */
  CPPMEGA_MI355_WSCALE_PER_ROW = 1,    /* float32 [N]                           */
  CPPMEGA_MI355_WSCALE_ROW_BLOCK = 2,  /* float32 [N, ceil(K/128)]              */
  CPPMEGA_MI355_WSCALE_GRID_128 = 3    /* float32 [ceil(N/128), ceil(K/128)]    */
};

typedef struct cppmega_mi355_vecmat_args {
  uint32_t struct_size;
  int32_t x_dtype;
  const void* x;
  const float* scale_x;
  const uint8_t* w;
  const float* scale_w;
  int32_t scale_w_kind;
  int32_t m, n, k;
  int32_t out_dtype;
  int32_t reserved;
  void* out;
  void* workspace;            /* split-K partials (M >= 5); may be NULL when
                                 *_workspace_bytes reports 0                   */
  size_t workspace_bytes;
} cppmega_mi355_vecmat_args_t;

int cppmega_mi355_fp8_vecmat_workspace_bytes(const cppmega_mi355_vecmat_args_t* args,
                                             size_t args_size, size_t* bytes);

int cppmega_mi355_fp8_vecmat(const cppmega_mi355_vecmat_args_t* args, size_t args_size, void* stream);

/* ---- per-head projections of the absorbed MLA decode ----------------------------
 * Y[m, g, n] = sum_k X[m, g, k] * W[g, n, k]: one skinny matrix product per group g.
 * Replaces the two einsums that bracket the attention call in the reference's
 * absorbed_mla_decode (cppmega_v4/nn/mla_absorb.py:116-134):
 *   "bthk,hkv->bthv"  q_abs = q . W_UK^T[h]:   m = b*t rows, g = h, k = D_k, n = D_kv,
 *                     W[h][v][k] = w_uk[h][v][k] (the layout absorb_weights :39-77 is given)
 *   "bthv,hvm->btm"   out = sum_h v_abs . (W_UV W_O)[h]: one group, k = H*D_kv,
 *                     W[0][m][h*D_kv + v] = w_uv_w_o[h][v][m]
 * and serves the per-head un-absorb o[b,t,h,:] . W_UV[h] (g = h, k = D_kv, n = D_v).
 *   x   [M, G, K] float32 or bfloat16; row pitch x_row_pitch, group pitch x_group_pitch
 *       (elements), k contiguous
 *   w   [G, N, K] float32 or bfloat16, dense: the contraction index is contiguous
 *   y   [M, G, N] float32 / float16 / bfloat16 with its own row and group pitch, so a
 *       result can land inside wider rows (q_abs inside [.., D_kv + rope] query rows)
 * fp32 accumulation; float32 operands enter the matrix cores as bf16 hi + lo pairs
 * (16 significand bits). */
typedef struct cppmega_mi355_head_gemm_args {
  uint32_t struct_size;
  int32_t x_dtype;
  const void* x;
  const void* w;
  void* y;
  int32_t w_dtype;
  int32_t y_dtype;
  int32_t m, groups, n, k;
  int64_t x_row_pitch, x_group_pitch;
  int64_t y_row_pitch, y_group_pitch;
} cppmega_mi355_head_gemm_args_t;

int cppmega_mi355_head_gemm(const cppmega_mi355_head_gemm_args_t* args, size_t args_size, void* stream);

/* dequant_block_fp8 (cppmega_v4/nn/_external/_mlx_lm_fp8_dequant_vendored.py:24-46), the
 * tensor step of sanitize_fp8_weights (:50-71): out[r, c] = dec(weight[r, c]) *
 * scale_inv[r / 128, c / 128], weight e4m3 bytes [rows, cols], scale_inv float32
 * [ceil(rows/128), ceil(cols/128)], out [rows, cols] bfloat16 (float16 / float32 also
 * accepted).  The bytes 0x7F / 0xFF decode to NaN. */
typedef struct cppmega_mi355_dequant_block_args {
  uint32_t struct_size;
  int32_t out_dtype;
  const void* weight;
  const float* scale_inv;
  void* out;
  int32_t rows, cols;
} cppmega_mi355_dequant_block_args_t;

int cppmega_mi355_dequant_block_fp8(const cppmega_mi355_dequant_block_args_t* args, size_t args_size, void* stream);

/* ---- FP8 producers ------------------------------------------------------------
 * The quantisers that write the prepared buffers of the attention entry points, and the
 * matching dequantiser:
 *   PER_TOKEN   fp8_per_token_quant(x, fp8, scale)
 *               (cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:2667-2753):
 *               scale[row] = max(amax(row) * (1/448), 1e-12), code = rne(clamp(x / scale, +-448))
 *   PER_TENSOR  _to_fp8_with_per_tensor_scale (sparse_mla_fp8.py:123-145): one amax over
 *               the tensor, the scale replicated per row
 *   MXFP8       _quantize_mxfp8 (sparse_mla_blockscaled.py:60-76): one E8M0 byte per 32
 *               channels, byte = clamp(127 + rint(log2(amax/448)), 1, 254): the exponent
 *               rounds to nearest (the rule that reproduces the reference's seeded receipt
 *               bench/tilelang_ports/sparse_mla_blockscaled.json parity.blockscaled_vs_bf16),
 *               codes saturate at +-448
 *   DEQUANT_*   _from_fp8_with_scale (sparse_mla_fp8.py:148-157) / _dequantize_mxfp8
 *               (sparse_mla_blockscaled.py:79-87): recovered = dec(codes) * scale
 *   QUANT_UNIT / DEQUANT_UNIT   half_to_fp8 / fp8_to_half
 *               (cppmega_mlx/nn/_tilelang/fp8_msl_kernels.py:65-81): the bare conversions,
 *               code = rne(clamp(x, +-448)) (NaN -> the NaN code of its sign) and
 *               recovered = dec(codes); no scale is read or written
 * x is [rows, k] float32/float16/bfloat16, dense.  Any of codes / scale / recovered may be
 * NULL in a quantise call (at least one is not); `recovered` receives dec(code) * scale in
 * x's dtype.  PER_TENSOR needs `scratch`, 4 bytes of device memory. */
enum {
  CPPMEGA_MI355_QUANT_PER_TOKEN = 0,
  CPPMEGA_MI355_QUANT_PER_TENSOR = 1,
  CPPMEGA_MI355_QUANT_MXFP8 = 2,
  CPPMEGA_MI355_DEQUANT_PER_TOKEN = 3,   /* codes + float32 scale[rows] -> recovered */
  CPPMEGA_MI355_DEQUANT_MXFP8 = 4,       /* codes + uint8 scale[rows, k/32] -> recovered */
  CPPMEGA_MI355_QUANT_UNIT = 5,          /* x -> codes, scale 1                           */
  CPPMEGA_MI355_DEQUANT_UNIT = 6         /* codes -> recovered, scale 1                   */
};

typedef struct cppmega_mi355_quantize_args {
  uint32_t struct_size;
  int32_t x_dtype;            /* F32/F16/BF16: dtype of x and of recovered          */
  const void* x;              /* [rows, k]; unused by the DEQUANT modes             */
  int64_t rows;
  int32_t k;
  int32_t mode;               /* CPPMEGA_MI355_QUANT_* / DEQUANT_*                   */
  uint8_t* codes;             /* [rows, k] e4m3 bytes (output; input of DEQUANT)    */
  void* scale;                /* float32 [rows] or uint8 [rows, k/32]               */
  void* recovered;            /* [rows, k] in x_dtype                               */
  void* scratch;              /* 4 bytes, PER_TENSOR only                           */
} cppmega_mi355_quantize_args_t;

int cppmega_mi355_fp8_quantize(const cppmega_mi355_quantize_args_t* args, size_t args_size, void* stream);

/* ---- KV-cache append: FP8 producer fused with the write into the cache ------------------
 * Replaces the append path in front of the sparse-attention kernels:
 *   ContiguousKVCache.update_and_fetch_sparse_fp8 (cppmega_mlx/inference/engine.py:76-98,
 *   validation :436-466) -- prepared e4m3 bytes + one float32 scale per row are appended
 *   along the sequence axis -- and, in front of it, the producer fp8_per_token_quant
 *   (cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:2667-2753).
 * The cache is preallocated, [B, capacity, G, ...]; `new_tokens` rows per (batch, group) are
 * written at positions `position` .. (or positions[b] ..).  Two source forms:
 *   src_dtype E4M3      src is e4m3 bytes [B, S_new, G, D], src_scale their float32 scales
 *                       [B, S_new, G, D/scale_block or 1]: bytes and scales are copied
 *                       (the reference's semantics);
 *   src_dtype F32/F16/BF16   src is quantised on the way: scale_block 0 = one scale per
 *                       row, max(amax * (1/448), 1e-12) (the reference's producer);
 *                       scale_block 128 = one float32 scale per 128 channels by the same
 *                       formula, or with pow2_scales != 0 the smallest power of two s with
 *                       448 * s >= amax (1.0 for an all-zero block): the latent cache format
 *                       the decode kernel gathers.
 * rope (optional, [B, S_new, G, R] float32/float16/bfloat16) is stored as bfloat16.
 * D % 128 == 0, D <= 2048, R <= 256.  With `positions` NULL the range position ..
 * position + S_new - 1 is checked against the capacity on the host (ERR_SHAPE); per-batch
 * positions live on the device, so rows that would fall outside [0, capacity) are skipped
 * by the kernel instead. */
typedef struct cppmega_mi355_cache_append_args {
  uint32_t struct_size;
  int32_t src_dtype;          /* E4M3 (prepared) or F32/F16/BF16 (quantise)          */
  const void* src;            /* [B, S_new, G, D]                                    */
  const float* src_scale;     /* prepared form only                                  */
  const void* rope;           /* [B, S_new, G, R] or NULL                            */
  int32_t rope_dtype;
  int32_t scale_block;        /* 0: one scale per row; 128: one per 128 channels     */
  uint8_t* kv_cache;          /* [B, capacity, G, D] e4m3 bytes                      */
  float* scale_cache;         /* [B, capacity, G, 1 or D/128]                        */
  void* rope_cache;           /* [B, capacity, G, R] bfloat16, or NULL               */
  const int32_t* positions;   /* [B] first position per batch entry, or NULL         */
  int32_t position;           /* first position for every batch entry (positions NULL) */
  int32_t batch, new_tokens, groups, dim, rope_dim, capacity;
  int32_t pow2_scales;
  int32_t reserved;
} cppmega_mi355_cache_append_args_t;

int cppmega_mi355_kv_cache_append(const cppmega_mi355_cache_append_args_t* args, size_t args_size, void* stream);

/* ---- sparse index producers -------------------------------------------------------------
 * causal_sparse_indices (cppmega_mlx/nn/attention.py:251-284):
 *   indices[b, s, g, j] = query_offset + s - j if that lies in [0, key_length), else -1.
 * sparse_indices_from_attention_mask (attention.py:287-360): per (b, s, g) the newest
 *   n = min(topk, key_length) valid keys of the mask row in ascending order, right-aligned,
 *   -1 in front when fewer are valid.  A key is valid where a boolean mask is non-zero or a
 *   float mask is finite.  The mask is addressed as mask[b*stride_b + g*stride_g +
 *   s*stride_s + k] (strides in elements; 0 broadcasts). */
typedef struct cppmega_mi355_causal_indices_args {
  uint32_t struct_size;
  int32_t index_dtype;        /* I32 or I64                                          */
  void* indices;              /* [B, S, G, topk]                                     */
  int32_t batch, seq, groups, topk;
  int64_t query_offset;
  int64_t key_length;
} cppmega_mi355_causal_indices_args_t;

int cppmega_mi355_causal_sparse_indices(const cppmega_mi355_causal_indices_args_t* args, size_t args_size, void* stream);

enum { CPPMEGA_MI355_MASK_BOOL = 0 /* one byte per key */, CPPMEGA_MI355_MASK_F32 = 1, CPPMEGA_MI355_MASK_F16 = 2, CPPMEGA_MI355_MASK_BF16 = 3 };

typedef struct cppmega_mi355_mask_indices_args {
  uint32_t struct_size;
  int32_t mask_dtype;         /* CPPMEGA_MI355_MASK_*                                */
  const void* mask;
  int64_t stride_b, stride_g, stride_s;
  int32_t batch, seq, groups, topk, key_length;
  int32_t reserved;
  int32_t* indices;           /* [B, S, G, min(topk, key_length)] int32              */
} cppmega_mi355_mask_indices_args_t;

int cppmega_mi355_mask_sparse_indices(const cppmega_mi355_mask_indices_args_t* args, size_t args_size, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CPPMEGA_MI355_H_ */
