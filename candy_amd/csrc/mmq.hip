// Batched (m >= 16) quantized matmul.
#include "blocks.h"
#include "internal.h"

namespace candy {

int launch_mmq(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales, int64_t m,
               float *y) {
    // Until the MFMA tile kernel takes over, large m runs the small-batch kernel in slices
    // (same arithmetic, re-reads the weights once per slice).
    return launch_matvec(dev, w, qs, scales, m, y);
}

}  // namespace candy
