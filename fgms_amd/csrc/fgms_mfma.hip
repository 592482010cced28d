// placeholder: MFMA kernels
#include "fgms_internal.h"
namespace fgms {
bool mfma_gms_supported(const GmsArgs &) { return false; }
int launch_mfma_gms(const GmsArgs &) { return FGMS_E_INVALID; }
bool mfma_wgrad_supported(const WgradArgs &) { return false; }
int launch_mfma_wgrad(const WgradArgs &) { return FGMS_E_INVALID; }
bool planned_gms_supported(const GmsArgs &, const Plan *) { return false; }
int launch_planned_gms(const GmsArgs &, const Plan *) { return FGMS_E_INVALID; }
}
