// placeholder until the MFMA prefill kernel lands
#include "pa_common.h"
namespace pa {
bool prefill_supported(const PrefillParams&) { return false; }
hipError_t launch_prefill(const PrefillParams&, hipStream_t) { return hipErrorNotSupported; }
}  // namespace pa
