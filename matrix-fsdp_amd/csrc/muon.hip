// Placeholder entry points while the Newton-Schulz kernels are being written.
#include "mfsdp_common.h"
using namespace mfsdp;
extern "C" int64_t mfsdp_muon_workspace_bytes(int64_t, int64_t) { return 0; }
extern "C" int mfsdp_newton_schulz(const void*, int, int64_t, int64_t, float, float, float, int, float, void*, void*, int64_t, void*) {
  return fail(MFSDP_ERR_UNSUPPORTED, "newton_schulz not built");
}
extern "C" int mfsdp_muon_step(void*, const void*, void*, int, int64_t, int64_t, float, float, float, int, float, float, float, int,
                               float, float, void*, int64_t, void*) {
  return fail(MFSDP_ERR_UNSUPPORTED, "muon_step not built");
}
