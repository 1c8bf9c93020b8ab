// Head-batched MFMA sparse-MLA kernel (placeholder until the kernel lands).
#include "sparse_mla_common.h"
namespace cm {
bool sparse_mla_mfma_supported(const MlaParams&) { return false; }
size_t sparse_mla_mfma_workspace_bytes(const MlaParams&) { return 0; }
void sparse_mla_mfma_plan(MlaParams&) {}
int sparse_mla_mfma_launch(const MlaParams&, hipStream_t) {
  return fail(CPPMEGA_MI355_ERR_UNSUPPORTED, "sparse_mla: MFMA kernel not built");
}
}  // namespace cm
