#include "cp4_internal.h"
namespace cp4 {
bool fwd_mfma_supported(const FwdArgs&) { return false; }
hipError_t fwd_mfma_launch(const FwdArgs&, hipStream_t) { return hipErrorNotSupported; }
}
