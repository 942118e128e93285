// gemm_oil4_mfma.hip -- prefill GEMM over uniform OIL4 tensors (placeholder until the MFMA kernel lands).
#include "common.h"

namespace oilhip {
int launch_gemm_oil4_bf16(const oilhip_weights&, const uint16_t*, float*, int, hipStream_t) {
    return fail(OILHIP_E_ARG, "bf16 prefill GEMM kernel is not built into this library yet");
}
}  // namespace oilhip
