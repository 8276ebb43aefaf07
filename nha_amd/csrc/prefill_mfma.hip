// placeholder until the MFMA kernels land
#include "common.h"
namespace nha {
bool prefill_mfma_supported(const NhaPrefillArgs*) { return false; }
size_t prefill_mfma_scratch_bytes(const NhaPrefillArgs*) { return 0; }
int prefill_mfma_impl(const NhaPrefillArgs*) { set_error("mfma prefill not built"); return NHA_ERR_UNSUPPORTED; }
}
