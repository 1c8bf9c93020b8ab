// extern "C" boundary of libcppmega_mi355.so: argument checking and dispatch.
// No device memory is allocated here or anywhere below.

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "sparse_mla_common.h"

namespace cm {

static thread_local char g_last_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int topk_select_launch(const cppmega_mi355_topk_args_t& a, hipStream_t stream);
int topk_workspace_bytes(const cppmega_mi355_topk_args_t& a, size_t* bytes);
int fp8_vecmat_launch(const cppmega_mi355_vecmat_args_t& a, hipStream_t stream);
int fp8_vecmat_workspace_bytes(const cppmega_mi355_vecmat_args_t& a, size_t* bytes);
int fp8_quantize_launch(const cppmega_mi355_quantize_args_t& a, hipStream_t stream);
int kv_cache_append_launch(const cppmega_mi355_cache_append_args_t& a, hipStream_t stream);
int causal_indices_launch(const cppmega_mi355_causal_indices_args_t& a, hipStream_t stream);
int mask_indices_launch(const cppmega_mi355_mask_indices_args_t& a, hipStream_t stream);
int sparse_mla_bwd_launch(const cppmega_mi355_sparse_mla_bwd_args_t& a, hipStream_t stream);
int dsa_indexer_loss_launch(const cppmega_mi355_dsa_loss_args_t& a, hipStream_t stream);
int head_gemm_launch(const cppmega_mi355_head_gemm_args_t& a, hipStream_t stream);
int dequant_block_fp8_launch(const cppmega_mi355_dequant_block_args_t& a, hipStream_t stream);
int indexer_topk_launch(const cppmega_mi355_indexer_args_t& a, hipStream_t stream);
int indexer_topk_workspace_bytes(const cppmega_mi355_indexer_args_t& a, size_t* bytes);

static bool is_float_carrier(int dt) {
  return dt == CPPMEGA_MI355_F32 || dt == CPPMEGA_MI355_F16 || dt == CPPMEGA_MI355_BF16;
}

// Validates the request and fills the kernel parameter block.
static int build_mla_params(const cppmega_mi355_sparse_mla_args_t& a, MlaParams& p, bool need_pointers, bool need_out = true) {
  if (a.batch < 0 || a.seq_q < 0 || a.heads < 1 || a.kv_groups < 1 || a.seq_kv < 0 || a.topk < 0)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "sparse_mla: negative or empty dimension");
  if (a.heads % a.kv_groups != 0)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "heads %d not divisible by kv_group %d", a.heads, a.kv_groups);
  if (a.rope_dim < 0 || a.rope_dim >= a.d_qk)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "sparse_mla: rope_dim %d must be in [0, d_qk=%d)", a.rope_dim, a.d_qk);
  const int d_kv = a.d_qk - a.rope_dim;
  if (a.d_v <= 0 || a.d_v > d_kv)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "d_v must be in (0, %d], got %d", d_kv, a.d_v);
  if (!is_float_carrier(a.q_dtype) && a.q_dtype != CPPMEGA_MI355_E4M3)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla: q dtype %d", a.q_dtype);
  if (!is_float_carrier(a.kv_dtype) && a.kv_dtype != CPPMEGA_MI355_E4M3)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla: kv dtype %d", a.kv_dtype);
  if (!is_float_carrier(a.out_dtype)) return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla: out dtype %d", a.out_dtype);
  if (a.index_dtype != CPPMEGA_MI355_I32 && a.index_dtype != CPPMEGA_MI355_I64)
    return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla: indices must be int32 or int64");
  if (a.rope_dim > 0 && !is_float_carrier(a.rope_dtype))
    return fail(CPPMEGA_MI355_ERR_DTYPE, "sparse_mla: rope dtype %d", a.rope_dtype);
  const int kinds[2] = {a.q_scale_kind, a.kv_scale_kind};
  const int blocks[2] = {a.q_scale_block, a.kv_scale_block};
  const int widths[2] = {a.d_qk, d_kv};
  for (int i = 0; i < 2; ++i) {
    if (kinds[i] < CPPMEGA_MI355_SCALE_NONE || kinds[i] > CPPMEGA_MI355_SCALE_F32_BLOCK)
      return fail(CPPMEGA_MI355_ERR_SHAPE, "sparse_mla: unknown scale kind %d", kinds[i]);
    if (kinds[i] == CPPMEGA_MI355_SCALE_E8M0 || kinds[i] == CPPMEGA_MI355_SCALE_F32_BLOCK) {
      if (blocks[i] < 1 || widths[i] % blocks[i] != 0)
        return fail(CPPMEGA_MI355_ERR_SHAPE, "sparse_mla: width %d not divisible by scale block %d", widths[i], blocks[i]);
    }
  }
  if (need_pointers) {
    if (!a.q || !a.kv || !a.indices || (need_out && !a.out)) return fail(CPPMEGA_MI355_ERR_NULL, "sparse_mla: q/kv/indices/out is NULL");
    if (a.q_scale_kind != CPPMEGA_MI355_SCALE_NONE && !a.q_scale) return fail(CPPMEGA_MI355_ERR_NULL, "sparse_mla: q_scale is NULL");
    if (a.kv_scale_kind != CPPMEGA_MI355_SCALE_NONE && !a.kv_scale) return fail(CPPMEGA_MI355_ERR_NULL, "sparse_mla: kv_scale is NULL");
    if (a.rope_dim > 0 && !a.kv_rope) return fail(CPPMEGA_MI355_ERR_NULL, "sparse_mla: kv_rope is NULL");
  }
  p.q = a.q; p.q_scale = a.q_scale; p.kv = a.kv; p.kv_scale = a.kv_scale; p.rope = a.kv_rope;
  p.indices = a.indices; p.sinks = a.sinks; p.out = a.out; p.lse = a.lse; p.workspace = a.workspace; p.scores = nullptr;
  p.q_dtype = a.q_dtype; p.q_scale_kind = a.q_scale_kind; p.q_scale_block = a.q_scale_block > 0 ? a.q_scale_block : a.d_qk;
  p.kv_dtype = a.kv_dtype; p.kv_scale_kind = a.kv_scale_kind; p.kv_scale_block = a.kv_scale_block > 0 ? a.kv_scale_block : d_kv;
  p.rope_dtype = a.rope_dtype; p.rope_dim = a.rope_dim; p.index_dtype = a.index_dtype; p.out_dtype = a.out_dtype;
  p.B = a.batch; p.S = a.seq_q; p.H = a.heads; p.G = a.kv_groups; p.Skv = a.seq_kv; p.topk = a.topk;
  p.d_qk = a.d_qk; p.d_kv = d_kv; p.d_v = a.d_v; p.heads_per_group = a.heads / a.kv_groups;
  p.num_splits = 1; p.keys_per_split = a.topk; p.heads_per_wg = 0; p.tile_sharing = 0; p.sm_scale = a.sm_scale;
  p.sm_scale_dev = a.sm_scale_dev; p.has_sinks_dev = a.has_sinks_dev;
  if (a.seq_kv_pitch != 0 && a.seq_kv_pitch < a.seq_kv)
    return fail(CPPMEGA_MI355_ERR_SHAPE, "sparse_mla: seq_kv_pitch %d is below seq_kv %d", a.seq_kv_pitch, a.seq_kv);
  p.Skv_pitch = a.seq_kv_pitch != 0 ? a.seq_kv_pitch : a.seq_kv;
  return 0;
}

// Copies the caller's sparse-MLA struct into the current layout; a caller built against the first
// ABI (struct_size ends at workspace_bytes) gets zeros for the fields appended since.
static int widen_mla_args(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size, cppmega_mi355_sparse_mla_args_t& a) {
  if (!args) return fail(CPPMEGA_MI355_ERR_NULL, "args is NULL");
  const size_t have = args_size < (size_t)args->struct_size ? args_size : (size_t)args->struct_size;
  if (have < CPPMEGA_MI355_SPARSE_MLA_ARGS_V1_SIZE)
    return fail(CPPMEGA_MI355_ERR_STRUCT_SIZE, "args struct is %zu/%u bytes, need %zu", args_size, args->struct_size,
                (size_t)CPPMEGA_MI355_SPARSE_MLA_ARGS_V1_SIZE);
  memset(&a, 0, sizeof(a));
  memcpy(&a, args, have < sizeof(a) ? have : sizeof(a));
  return 0;
}

static int pick_mla_kernel(const cppmega_mi355_sparse_mla_args_t& a, const MlaParams& p) {
  if (a.kernel == CPPMEGA_MI355_MLA_KERNEL_SCALAR) return CPPMEGA_MI355_MLA_KERNEL_SCALAR;
  const bool ok = sparse_mla_mfma_supported(p);
  if (a.kernel == CPPMEGA_MI355_MLA_KERNEL_MFMA)
    return ok ? CPPMEGA_MI355_MLA_KERNEL_MFMA
              : -fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla: the MFMA kernel does not cover this shape/dtype");
  if (a.kernel != CPPMEGA_MI355_MLA_KERNEL_AUTO) return -fail(CPPMEGA_MI355_ERR_SHAPE, "sparse_mla: unknown kernel %d", a.kernel);
  return ok ? CPPMEGA_MI355_MLA_KERNEL_MFMA : CPPMEGA_MI355_MLA_KERNEL_SCALAR;
}

// ---- scratch of the entry point that allocates nothing ------------------------------------
// The array is part of the code object, so every GPU that loads the library holds its own copy at
// its own address until the process ends.  In host code the name `scratch` is only a handle for
// hipGetSymbolAddress; the address the kernels get is the one looked up per device below.
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[CPPMEGA_MI355_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];          // device address of `scratch`, per device; NULL = not looked up yet
static std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch` (looked up once per device).
static int scratch_of_current_device(void** out) {
  int dev = -1;
  CM_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "device ordinal %d is outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    CM_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr || ((uintptr_t)ptr & 255)) return fail(CPPMEGA_MI355_ERR_LAUNCH, "static scratch resolved to %p", ptr);
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

}  // namespace cm

using namespace cm;

#define CM_CHECK_ARGS(args, args_size, T)                                              \
  do {                                                                                 \
    if (!(args)) return fail(CPPMEGA_MI355_ERR_NULL, "args is NULL");                  \
    if ((args_size) < sizeof(T) || (args)->struct_size < sizeof(T))                    \
      return fail(CPPMEGA_MI355_ERR_STRUCT_SIZE, "args struct is %zu/%u bytes, need %zu", \
                  (size_t)(args_size), (args)->struct_size, sizeof(T));                \
  } while (0)

extern "C" {

const char* cppmega_mi355_error_string(int code) {
  switch (code) {
    case CPPMEGA_MI355_OK: return "ok";
    case CPPMEGA_MI355_ERR_NULL: return "a required pointer is NULL";
    case CPPMEGA_MI355_ERR_STRUCT_SIZE: return "argument struct too small for this ABI";
    case CPPMEGA_MI355_ERR_SHAPE: return "shape or value outside the contract";
    case CPPMEGA_MI355_ERR_DTYPE: return "unsupported dtype";
    case CPPMEGA_MI355_ERR_UNSUPPORTED: return "no kernel covers this request";
    case CPPMEGA_MI355_ERR_WORKSPACE: return "workspace missing or too small";
    case CPPMEGA_MI355_ERR_LAUNCH: return "HIP launch or runtime error";
    case CPPMEGA_MI355_ERR_ALIGNMENT: return "pointer or stride misaligned";
    default: return "unknown status code";
  }
}

const char* cppmega_mi355_last_error(void) { return g_last_error; }

int cppmega_mi355_status(cppmega_mi355_status_t* out, size_t out_size) {
  if (!out) return CPPMEGA_MI355_ERR_NULL;
  if (out_size < sizeof(cppmega_mi355_status_t)) return CPPMEGA_MI355_ERR_STRUCT_SIZE;
  memset(out, 0, sizeof(*out));
  out->struct_size = (uint32_t)sizeof(*out);
  out->abi_version = CPPMEGA_MI355_ABI_VERSION;
  snprintf(out->built_for, sizeof(out->built_for), "gfx950");
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  out->device_count = n;
  for (int i = 0; i < n; ++i) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, i) == hipSuccess && strncmp(prop.gcnArchName, "gfx950", 6) == 0)
      out->gfx950_devices += 1;
  }
  if (n == 0) snprintf(out->message, sizeof(out->message), "no HIP device visible");
  else if (out->gfx950_devices == 0) snprintf(out->message, sizeof(out->message), "no gfx950 device among %d HIP devices", n);
  else snprintf(out->message, sizeof(out->message), "ready: %d gfx950 device(s)", out->gfx950_devices);
  return CPPMEGA_MI355_OK;
}

// Copies the caller's top-k struct into the current layout (zeros for fields appended after the first ABI).
static int widen_topk_args(const cppmega_mi355_topk_args_t* args, size_t args_size, cppmega_mi355_topk_args_t& a) {
  if (!args) return fail(CPPMEGA_MI355_ERR_NULL, "args is NULL");
  const size_t have = args_size < (size_t)args->struct_size ? args_size : (size_t)args->struct_size;
  if (have < CPPMEGA_MI355_TOPK_ARGS_V1_SIZE)
    return fail(CPPMEGA_MI355_ERR_STRUCT_SIZE, "args struct is %zu/%u bytes, need %zu", args_size, args->struct_size,
                (size_t)CPPMEGA_MI355_TOPK_ARGS_V1_SIZE);
  memset(&a, 0, sizeof(a));
  memcpy(&a, args, have < sizeof(a) ? have : sizeof(a));
  return 0;
}

int cppmega_mi355_topk_select(const cppmega_mi355_topk_args_t* args, size_t args_size, void* stream) {
  cppmega_mi355_topk_args_t a;
  const int rc = widen_topk_args(args, args_size, a);
  if (rc) return rc;
  return topk_select_launch(a, (hipStream_t)stream);
}

int cppmega_mi355_topk_workspace_bytes(const cppmega_mi355_topk_args_t* args, size_t args_size, size_t* bytes) {
  cppmega_mi355_topk_args_t a;
  const int rc = widen_topk_args(args, args_size, a);
  if (rc) return rc;
  if (!bytes) return fail(CPPMEGA_MI355_ERR_NULL, "bytes is NULL");
  return topk_workspace_bytes(a, bytes);
}

int cppmega_mi355_indexer_topk_workspace_bytes(const cppmega_mi355_indexer_args_t* args, size_t args_size, size_t* bytes) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_indexer_args_t);
  if (!bytes) return fail(CPPMEGA_MI355_ERR_NULL, "bytes is NULL");
  return indexer_topk_workspace_bytes(*args, bytes);
}

int cppmega_mi355_indexer_topk(const cppmega_mi355_indexer_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_indexer_args_t);
  return indexer_topk_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_sparse_mla_select_kernel(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size) {
  cppmega_mi355_sparse_mla_args_t a;
  int rc = widen_mla_args(args, args_size, a);
  if (rc) return -rc;
  MlaParams p;
  rc = build_mla_params(a, p, false);
  if (rc) return -rc;
  return pick_mla_kernel(a, p);
}

int cppmega_mi355_sparse_mla_workspace_bytes(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size,
                                             size_t* bytes) {
  cppmega_mi355_sparse_mla_args_t a;
  int rc = widen_mla_args(args, args_size, a);
  if (rc) return rc;
  if (!bytes) return fail(CPPMEGA_MI355_ERR_NULL, "bytes is NULL");
  MlaParams p;
  rc = build_mla_params(a, p, false);
  if (rc) return rc;
  const int kern = pick_mla_kernel(a, p);
  if (kern < 0) return -kern;
  *bytes = 0;
  if (kern == CPPMEGA_MI355_MLA_KERNEL_MFMA) {
    sparse_mla_mfma_plan(p);
    *bytes = sparse_mla_mfma_workspace_bytes(p);
  }
  return 0;
}

int cppmega_mi355_sparse_mla_fwd(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size, void* stream) {
  cppmega_mi355_sparse_mla_args_t a;
  int rc = widen_mla_args(args, args_size, a);
  if (rc) return rc;
  MlaParams p;
  rc = build_mla_params(a, p, true);
  if (rc) return rc;
  const int kern = pick_mla_kernel(a, p);
  if (kern < 0) return -kern;
  if (kern == CPPMEGA_MI355_MLA_KERNEL_MFMA) {
    sparse_mla_mfma_plan(p);
    const size_t need = sparse_mla_mfma_workspace_bytes(p);
    if (need > 0 && (!a.workspace || a.workspace_bytes < need))
      return fail(CPPMEGA_MI355_ERR_WORKSPACE, "sparse_mla: workspace of %zu bytes needed, %zu given", need,
                  a.workspace ? a.workspace_bytes : (size_t)0);
    return sparse_mla_mfma_launch(p, (hipStream_t)stream);
  }
  return sparse_mla_scalar_launch(p, (hipStream_t)stream);
}

int cppmega_mi355_sparse_mla_fwd_noalloc(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size, void* stream) {
  cppmega_mi355_sparse_mla_args_t a;
  int rc = widen_mla_args(args, args_size, a);
  if (rc) return rc;
  MlaParams p;
  rc = build_mla_params(a, p, true);
  if (rc) return rc;
  const int kern = pick_mla_kernel(a, p);
  if (kern < 0) return -kern;
  if (kern != CPPMEGA_MI355_MLA_KERNEL_MFMA) return sparse_mla_scalar_launch(p, (hipStream_t)stream);
  sparse_mla_mfma_plan(p);
  const size_t need = sparse_mla_mfma_workspace_bytes(p);
  if (need > (size_t)CPPMEGA_MI355_NOALLOC_SCRATCH_BYTES)
    return fail(CPPMEGA_MI355_ERR_WORKSPACE,
                "sparse_mla_fwd_noalloc: these shapes need %zu bytes of scratch, the static array holds %zu; "
                "use cppmega_mi355_sparse_mla_fwd with a caller workspace", need, (size_t)CPPMEGA_MI355_NOALLOC_SCRATCH_BYTES);
  p.workspace = nullptr;
  if (need > 0) {
    void* ptr = nullptr;
    rc = scratch_of_current_device(&ptr);
    if (rc) return rc;
    p.workspace = ptr;
  }
  return sparse_mla_mfma_launch(p, (hipStream_t)stream);
}

int cppmega_mi355_sparse_mla_scores(const cppmega_mi355_sparse_mla_args_t* args, size_t args_size, float* scores,
                                    void* stream) {
  cppmega_mi355_sparse_mla_args_t a;
  int rc = widen_mla_args(args, args_size, a);
  if (rc) return rc;
  if (!scores) return fail(CPPMEGA_MI355_ERR_NULL, "sparse_mla_scores: scores is NULL");
  MlaParams p;
  rc = build_mla_params(a, p, true, false);
  if (rc) return rc;
  p.scores = scores;
  return sparse_mla_scores_launch(p, (hipStream_t)stream);
}

int cppmega_mi355_sparse_mla_bwd(const cppmega_mi355_sparse_mla_bwd_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_sparse_mla_bwd_args_t);
  return sparse_mla_bwd_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_dsa_indexer_loss(const cppmega_mi355_dsa_loss_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_dsa_loss_args_t);
  return dsa_indexer_loss_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_head_gemm(const cppmega_mi355_head_gemm_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_head_gemm_args_t);
  return head_gemm_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_dequant_block_fp8(const cppmega_mi355_dequant_block_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_dequant_block_args_t);
  return dequant_block_fp8_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_fp8_quantize(const cppmega_mi355_quantize_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_quantize_args_t);
  return fp8_quantize_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_kv_cache_append(const cppmega_mi355_cache_append_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_cache_append_args_t);
  return kv_cache_append_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_causal_sparse_indices(const cppmega_mi355_causal_indices_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_causal_indices_args_t);
  return causal_indices_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_mask_sparse_indices(const cppmega_mi355_mask_indices_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_mask_indices_args_t);
  return mask_indices_launch(*args, (hipStream_t)stream);
}

int cppmega_mi355_fp8_vecmat_workspace_bytes(const cppmega_mi355_vecmat_args_t* args, size_t args_size,
                                             size_t* bytes) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_vecmat_args_t);
  return fp8_vecmat_workspace_bytes(*args, bytes);
}

int cppmega_mi355_fp8_vecmat(const cppmega_mi355_vecmat_args_t* args, size_t args_size, void* stream) {
  CM_CHECK_ARGS(args, args_size, cppmega_mi355_vecmat_args_t);
  return fp8_vecmat_launch(*args, (hipStream_t)stream);
}

}  // extern "C"
