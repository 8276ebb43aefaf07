// placeholder translation unit, filled in below
#include "mfma_common.h"
namespace nha {
bool prefill_ring_supported(const mf::MP&, int) { return false; }
int prefill_ring_launch(const mf::MP&, int, hipStream_t) { return NHA_ERR_UNSUPPORTED; }
}  // namespace nha
