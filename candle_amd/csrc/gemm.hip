// Prefill GEMM on int8 MFMA (placeholder until the tile kernel lands).
#include "qhip_internal.h"

bool cq_gemm_supported(const cq_weight *, int64_t, int) { return false; }
hipError_t cq_launch_gemm(const cq_weight *, cq_act_view, int, int64_t, float *, hipStream_t) {
    return hipErrorNotSupported;
}
