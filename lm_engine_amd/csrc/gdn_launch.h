// Internal launch entry points shared between the C-ABI translation unit and the kernels.
#pragma once

#include <hip/hip_runtime.h>

#include "gdn_hip.h"

namespace gdn {

// Arguments are validated by the caller (gdn_api.hip); these only pick an instantiation and launch.
int launch_recurrent(const gdn_args& a, hipStream_t stream);
// `events`, when not null, holds GDN_CHUNK_KERNELS + 1 events recorded around the kernels.
int launch_chunk_fwd(const gdn_args& a, hipStream_t stream, hipEvent_t* events = nullptr);
uint64_t chunk_workspace_bytes(const gdn_args& a);
bool chunk_shape_supported(const gdn_args& a);

}  // namespace gdn
