// placeholder until the MFMA kernel lands
#include "qm_host.h"
extern "C" int32_t qm_prefill_attention_causal(
    const uint16_t*, const uint16_t*, const uint16_t*, uint16_t*, const qm_kv_cache*, const int32_t*,
    int32_t, int32_t, int32_t, int32_t, int32_t, float, uint32_t*, void*) { return QM_ERR_ARGUMENT; }
