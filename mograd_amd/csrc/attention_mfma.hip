// Flash attention on the matrix cores (placeholder until the MFMA kernels land).
#include "attention_generic.h"
#include "mg_internal.h"

namespace mg {

bool attn_mfma_supported(int, int64_t, const void* const*, int) { return false; }

int attn_fwd_mfma(const void*, const void*, const void*, const void*, void*, float*, AttnDims, float, bool, bool, int,
                  hipStream_t) {
  return fail(MG_ERR_UNSUPPORTED, "flash_attn_fwd: MFMA path not built");
}

int attn_bwd_mfma(const void*, const void*, const void*, const void*, const void*, const void*, const float*, void*,
                  void*, void*, AttnDims, float, bool, bool, int, hipStream_t) {
  return fail(MG_ERR_UNSUPPORTED, "flash_attn_bwd: MFMA path not built");
}

}  // namespace mg
