// placeholder until the loop kernel lands
#include "qm_host.h"
extern "C" int32_t qm_predictor_attention_loop(
    const uint16_t*, const uint16_t*, const uint16_t*, const uint16_t*, const uint16_t*, const uint16_t*,
    const uint16_t*, uint16_t*, uint16_t*, uint16_t*, int32_t, int32_t, int32_t, int32_t, float, void*) {
    return QM_ERR_ARGUMENT; }
