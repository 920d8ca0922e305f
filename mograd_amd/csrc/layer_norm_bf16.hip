// LayerNorm kernels for bf16 storage.
#include "layer_norm_impl.h"
MG_DEFINE_LAYER_NORM(mg::bf16_t, bf16)
