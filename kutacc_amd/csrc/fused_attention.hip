#include <hip/hip_runtime.h>
#include "device_util.h"
#include "launch_internal.h"
namespace kutacc_launch {
bool fused_attention_supports(const kutacc_hip_attention_args_t &) { return false; }
int gating_attention_fused(const kutacc_hip_attention_args_t &, hipStream_t) { return KUTACC_HIP_EUNSUPPORTED; }
}
