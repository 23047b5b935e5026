// gqa_prefill.hip -- placeholder until the MFMA causal prefill kernel lands.
#include "common.hpp"
namespace cwick {
int launch_gqa_prefill(const uint16_t *, const uint16_t *, int64_t, int64_t, int, int,
                       const uint16_t *, int, float, float *, hipStream_t) {
    set_error("gqa_prefill: not built yet");
    return 0;
}
}  // namespace cwick
