#include "common.h"
#include "launchers.h"
namespace xdit {
hipError_t launch_attn_fwd_fp8(const AttnParams&, int, hipStream_t) { return hipErrorNotSupported; }
}
