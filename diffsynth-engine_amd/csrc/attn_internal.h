// Launchers shared between the attention translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/dsx.h"

namespace dsx {
// Attention without fused RMSNorm/RoPE (parameters already validated by dsx_attn_fwd).  `scratch` is
// optional device memory (16-byte aligned) for splitting the key range of the last round of workgroups.
int launch_attn_plain(const dsx_attn_params& p, void* scratch, int64_t scratch_bytes, hipStream_t stream);
// Scratch bytes with which launch_attn_plain would split (0 when it would not).
int64_t attn_plain_workspace_bytes(const dsx_attn_params& p);
}  // namespace dsx
