#include "common.h"
namespace aicomp {
bool prefill_mfma_supported(const DecodeArgs&, int) { return false; }
int launch_prefill_mfma(const DecodeArgs&, int) { set_error("not built"); return AICOMP_KV_EUNSUPPORTED; }
}
