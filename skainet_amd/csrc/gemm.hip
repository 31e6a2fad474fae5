// Prefill dequant-GEMM entry (placeholder body until the MFMA kernel lands in this file).
#include "common.h"

namespace skh {
int launch_gemv(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y);
int launch_gemm(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y) {
    return launch_gemv(enc, w, x, m, k, n, y);
}
}  // namespace skh
