// placeholder until the chunked forward lands
#include "gdn_common.h"
#include "gdn_launch.h"
namespace gdn {
bool chunk_shape_supported(const gdn_args&) { return false; }
uint64_t chunk_workspace_bytes(const gdn_args&) { return 0; }
int launch_chunk_fwd(const gdn_args&, hipStream_t) { return GDN_ERR_UNSUPPORTED; }
}  // namespace gdn
