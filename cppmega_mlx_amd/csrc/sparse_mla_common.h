// Parameter block shared by the sparse-MLA kernels.
#pragma once

#include "common.h"

namespace cm {

struct MlaParams {
  const void* q;
  const void* q_scale;
  const void* kv;
  const void* kv_scale;
  const void* rope;
  const void* indices;
  const float* sinks;
  void* out;
  float* lse;
  void* workspace;
  float* scores;        // score-only entry point: [B, S, H, topk] fp32
  int q_dtype, q_scale_kind, q_scale_block;
  int kv_dtype, kv_scale_kind, kv_scale_block;
  int rope_dtype, rope_dim;
  int index_dtype, out_dtype;
  int B, S, H, G, Skv, topk;
  int d_qk, d_kv, d_v;
  int heads_per_group;
  int num_splits;       // split-KV factor of the MFMA kernel
  int keys_per_split;
  int heads_per_wg;     // 0: 32-head tile kernel; 64: shared-tile latent kernel (sparse_mla_latent.hip)
  int tile_sharing;     // tile kernel on 16-bit rows: the 4 wavefronts take 4 head groups over one key stream
  float sm_scale;
  const float* sm_scale_dev;     // device copy of the softmax scale; read in place of sm_scale when set
  const int* has_sinks_dev;      // device flag; sinks are ignored when it is set and holds 0
  int Skv_pitch;                 // key rows between two batches of the cache buffers (>= Skv)
};

// softmax scale and sink switch as the kernels read them (uniform loads)
__device__ __forceinline__ float mla_sm_scale(const MlaParams& p) { return p.sm_scale_dev ? *p.sm_scale_dev : p.sm_scale; }
__device__ __forceinline__ bool mla_has_sinks(const MlaParams& p) {
  return p.sinks != nullptr && (p.has_sinks_dev == nullptr || *p.has_sinks_dev != 0);
}

__device__ __forceinline__ long long load_index(const MlaParams& p, size_t i) {
  return p.index_dtype == CPPMEGA_MI355_I64 ? ((const long long*)p.indices)[i]
                                            : (long long)((const int*)p.indices)[i];
}

// scale of element block `blk` of row `row` (row = flattened leading index)
__device__ __forceinline__ float row_scale(const void* scale, int kind, size_t row, int nblk, int blk) {
  switch (kind) {
    case CPPMEGA_MI355_SCALE_PER_TOKEN: return ((const float*)scale)[row];
    case CPPMEGA_MI355_SCALE_E8M0: return e8m0_to_f32(((const unsigned char*)scale)[row * nblk + blk]);
    case CPPMEGA_MI355_SCALE_F32_BLOCK: return ((const float*)scale)[row * nblk + blk];
    default: return 1.0f;
  }
}

int sparse_mla_scalar_launch(const MlaParams& p, hipStream_t stream);
int sparse_mla_scores_launch(const MlaParams& p, hipStream_t stream);
int sparse_mla_mfma_launch(const MlaParams& p, hipStream_t stream);
bool sparse_mla_mfma_supported(const MlaParams& p);
size_t sparse_mla_mfma_workspace_bytes(const MlaParams& p);
void sparse_mla_mfma_plan(MlaParams& p);

// shared-tile kernel for FP8 latent caches (sparse_mla_latent.hip); dispatched by the *_mfma_* functions
bool sparse_mla_latent_supported(const MlaParams& p);
void sparse_mla_latent_plan(MlaParams& p);
int sparse_mla_latent_launch(const MlaParams& p, hipStream_t stream);   // includes its combine step
size_t sparse_mla_latent_workspace_bytes(const MlaParams& p);

}  // namespace cm
