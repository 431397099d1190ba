// MFMA prefill / chunked-prefill attention (placeholder until the tiled kernel lands): reports
// "not supported", so sequences with more than 16 rows per KV head run on the fp32 kernel.
#include "rpa_common.h"

namespace rpa {
bool prefill_supported(const AttnParams&) { return false; }
int launch_attn_prefill(hipStream_t, const AttnParams&) { return (int)hipErrorNotSupported; }
}  // namespace rpa
