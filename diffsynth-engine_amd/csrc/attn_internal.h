// Launchers shared between the attention translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/dsx.h"

namespace dsx {
// Attention without fused RMSNorm/RoPE (parameters already validated by dsx_attn_fwd).
int launch_attn_plain(const dsx_attn_params& p, hipStream_t stream);
}  // namespace dsx
