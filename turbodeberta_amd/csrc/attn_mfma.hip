// Matrix-core (MFMA) disentangled-attention forward for bf16, head_dim 64.  (placeholder)
#include "tdb_internal.h"

bool tdb_mfma_supported(const TdbKernelParams&, int) { return false; }
hipError_t tdb_launch_mfma(const TdbKernelParams&, int, hipStream_t) { return hipErrorNotSupported; }
