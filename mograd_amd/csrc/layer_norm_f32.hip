// LayerNorm kernels for f32 storage.
#include "layer_norm_impl.h"
MG_DEFINE_LAYER_NORM(float, f32)
