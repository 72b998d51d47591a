// placeholder until the W4A8 path lands
#include "common.h"
extern "C" {
int dpep_mx_quant(const void*, int, int, void*, uint8_t*, void*) { return dpep::fail(DPEP_ERUNTIME, "mx_quant: not built yet"); }
size_t dpep_megamoe_workspace_bytes(int, int, int, int, int) { return 0; }
int dpep_megamoe_prepare_weights(const uint8_t*, const uint8_t*, int, int, int, uint8_t*, uint8_t*, void*) { return dpep::fail(DPEP_ERUNTIME, "megamoe: not built yet"); }
int dpep_megamoe_forward(void*, const void*, const uint8_t*, const int32_t*, const float*, const uint8_t*, const uint8_t*, const uint8_t*, const uint8_t*, int, int, int, int, int, int, int, void*, int32_t*, void*) { return dpep::fail(DPEP_ERUNTIME, "megamoe: not built yet"); }
}
