// Softmax cross-entropy kernels for f16 storage.
#include "cross_entropy_impl.h"
MG_DEFINE_CROSS_ENTROPY(mg::f16_t, f16)
