// Softmax cross-entropy kernels for bf16 storage.
#include "cross_entropy_impl.h"
MG_DEFINE_CROSS_ENTROPY(mg::bf16_t, bf16)
