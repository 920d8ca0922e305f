// LayerNorm kernels for f16 storage.
#include "layer_norm_impl.h"
MG_DEFINE_LAYER_NORM(mg::f16_t, f16)
