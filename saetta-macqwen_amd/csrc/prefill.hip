// placeholder until the flash kernel lands
#include "common.hpp"
using namespace saetta;
extern "C" int saetta_attn_prefill(saetta_stream_t, const uint16_t *, const uint16_t *, const uint16_t *,
                                   const float *, float *, saetta_flash_params) {
    return fail(SAETTA_E_DEVICE, "attn_prefill: not built yet");
}
extern "C" int saetta_attn_prefill_quant(saetta_stream_t, int, const uint16_t *, saetta_quant_rows,
                                         saetta_quant_rows, const float *, float *, saetta_flash_params) {
    return fail(SAETTA_E_DEVICE, "attn_prefill_quant: not built yet");
}
