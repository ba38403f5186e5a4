// Capability manifest: one bit per fully implemented operation
// (reference: ferrule_cutlass_provider_manifest, abi/cutlass_provider.h:14-35, 390;
// Ferrule compiles its plan against this mask and fails closed,
// crates/ferrule-backend/src/cuda/provider.rs:31-77).
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"

namespace ferrule_hip {
thread_local int32_t g_last_hip_error = 0;
}

extern "C" int32_t ferrule_hip_last_error_code(void) { return ferrule_hip::g_last_hip_error; }

#ifndef FERRULE_HIP_SOURCE_DIGEST
#define FERRULE_HIP_SOURCE_DIGEST "unknown"
#endif
extern "C" const char *ferrule_hip_source_digest(void) { return FERRULE_HIP_SOURCE_DIGEST; }

extern "C" FerruleHipProviderManifest ferrule_hip_provider_manifest(void) {
  FerruleHipProviderManifest manifest;
  manifest.kernel_mask = FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_QUANT_GEMV) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_MOE_DECODE) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_DENSE_FFN_DECODE) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_FP8_QUERY_A_KV) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_FP8_PROJECTION) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_FP8_BLOCK_GEMM) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_GROUPED_FP4_MOE) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_SHARED_FFN) |
                         FERRULE_HIP_KERNEL_BIT(FERRULE_HIP_KERNEL_HYPER_CONNECTION_PRODUCER);
  return manifest;
}
