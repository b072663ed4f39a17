// Internal (not exported): the library's allocation-free scratch memory.  No HIP types, so host-side translation units can
// include it.
#pragma once

#include <cstddef>

// Size of the scratch block every GPU holds (4 MiB).
#define THORHIP_STATIC_SCRATCH_BYTES (4u << 20)

namespace thorhip {

// Address and size of the current device's copy of the scratch block.  The first call on a device looks the address up
// (hipGetSymbolAddress); later calls return the remembered one.  Performs no allocation.  Returns 0, or a negative value
// with thorhip_last_error() set.  Every user of the block on one GPU shares it: calls that overlap in time race.
int staticScratch(void** ptr, size_t* capacity_bytes);

}  // namespace thorhip
