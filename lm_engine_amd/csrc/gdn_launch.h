// Internal launch entry points shared between the C-ABI translation unit and the kernels.
#pragma once

#include <hip/hip_runtime.h>

#include "gdn_hip.h"

namespace gdn {

// compute units of the current device (looked up once per device)
inline int compute_units() {
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// Arguments are validated by the caller (gdn_api.hip); these only pick an instantiation and launch.
int launch_recurrent(const gdn_args& a, hipStream_t stream);
// `events`, when not null, holds GDN_CHUNK_KERNELS + 1 events recorded around the kernels.
// `saves`, when not null, selects the state-saving scan (see gdn_chunk_fwd_saving).
int launch_chunk_fwd(const gdn_args& a, hipStream_t stream, hipEvent_t* events = nullptr, const gdn_chunk_saves* saves = nullptr);
uint64_t chunk_workspace_bytes(const gdn_args& a);
uint64_t chunk_record_bytes(const gdn_args& a);  // the records alone, [H][chunk slots]
uint64_t chunk_header_bytes(const gdn_args& a);  // what precedes the records: chunk offsets, error latch, ready flags
uint64_t chunk_error_latch_offset(const gdn_args& a);  // byte offset of the error latch (an int32) in the workspace
bool chunk_shape_supported(const gdn_args& a);
bool chunk_saving_scan_is_staged(const gdn_args& a, const gdn_chunk_saves& saves);  // bf16 saves / no output available
bool chunk_runs_as_one_launch(const gdn_args& a);  // gdn_chunk_fwd would run prepare and scan as one launch (shape fields, flags, cu_seqlens)
int launch_chunk_bwd_local(const gdn_chunk_local_args& a, hipStream_t stream);  // gdn_chunk_bwd.hip
bool chunk_bwd_local_supported(const gdn_chunk_local_args& a);
int launch_chunk_bwd_prepare(const gdn_chunk_bwd_prepare_args& a, hipStream_t stream);
bool chunk_bwd_prepare_supported(const gdn_chunk_bwd_prepare_args& a);
uint64_t chunk_bwd_record_bytes(const gdn_chunk_bwd_prepare_args& a);
int launch_conv_bwd(const gdn_conv_bwd_args& a, hipStream_t stream);  // gdn_conv1d_bwd.hip
#ifdef GDN_CYCLE_BUDGET
uint64_t* cycle_buffer();  // gdn_chunk.hip, measurement build only: the device buffer sampled waves report their cycles into
#endif

}  // namespace gdn
