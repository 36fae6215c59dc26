// INT4 engine: f16 MFMA kernel for m > 8 (placeholder dispatcher until the
// kernel lands: reports "unsupported" so the reference-order kernel runs).
#include "w4.h"

namespace rumus {

bool w4_gemm_supported(const W4Args&) { return false; }

int w4_launch_gemm(const W4Args&, hipStream_t) {
    return set_error(RUMUS_HIP_EINVAL, "w4 gemm: kernel not available");
}

}  // namespace rumus
