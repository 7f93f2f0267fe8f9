// Temporary: entry points not written yet.
#include "pal_common.h"
extern "C" {
size_t pal_recurrent_bwd_workspace_bytes(const PalDims*) { return 0; }
int pal_recurrent_bwd(const PalDims*, const PalFwdTensors*, const PalBwdTensors*, void*, size_t, void*) { return PAL_E_WORKSPACE; }
}
