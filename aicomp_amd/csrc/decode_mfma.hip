#include "common.h"
namespace aicomp {
bool decode_mfma_supported(const DecodeArgs&) { return false; }
int launch_decode_mfma(const DecodeArgs&) { set_error("not built"); return AICOMP_KV_EUNSUPPORTED; }
}
