// placeholder: MFMA weight-gradient kernels
#include "fgms_internal.h"
namespace fgms {
bool mfma_wgrad_supported(const WgradArgs &) { return false; }
int launch_mfma_wgrad(const WgradArgs &) { return FGMS_E_INVALID; }
}
