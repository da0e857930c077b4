#include "common.h"
#include "launchers.h"
namespace xdit {
hipError_t launch_attn_fwd_f32(const AttnParams&, int, int, hipStream_t) { return hipErrorNotSupported; }
}
