// bf16 MFMA kernels (placeholder until the tuned kernels land: reports "not supported"
// so that every launch takes the generic kernels).
#include "tk_device.h"

namespace tk {
bool pass_mfma_supported(const PassArgs&) { return false; }
int launch_pass_mfma(const PassArgs&, const SegView&, const SegLayout&, hipStream_t) { return TK_ERR_UNSUPPORTED; }
bool wgrad_mfma_supported(const WgradArgs&) { return false; }
int launch_wgrad_mfma(const WgradArgs&, const SegView&, const SegLayout&, hipStream_t) { return TK_ERR_UNSUPPORTED; }
}  // namespace tk
