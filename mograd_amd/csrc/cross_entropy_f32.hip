// Softmax cross-entropy kernels for f32 storage.
#include "cross_entropy_impl.h"
MG_DEFINE_CROSS_ENTROPY(float, f32)
