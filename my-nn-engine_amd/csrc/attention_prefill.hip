// Causal prefill attention on the matrix cores (replaces the reference's attention_tc,
// attention.cuh:45-314).  Until that kernel is in, every Sq > 1 call takes the per-row
// flash-decode path of attention_decode.hip.
#include "attention.h"

namespace mynn {
bool attention_prefill_supported(const AttnParams &, int, int, int) { return false; }
int attention_prefill_launch(const AttnParams &, int, int, hipStream_t) {
    return fail(MYNN_ERR_UNSUPPORTED, "attention: matrix-core prefill kernel not built");
}
}  // namespace mynn
