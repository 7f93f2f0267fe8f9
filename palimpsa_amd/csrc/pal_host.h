// Host-side declarations shared by the entry points of the C ABI.
#pragma once
#include "../../include/palimpsa_hip.h"

namespace pal {
// Pointer / flag consistency checks; PAL_OK or a PAL_E_* code, no HIP call.
int check_fwd_common(const PalDims* d, const PalFwdTensors* t);
int check_chunk_common(const PalDims* d, const PalFwdTensors* t);
int check_bwd_common(const PalDims* d, const PalBwdTensors* gr);
}  // namespace pal
