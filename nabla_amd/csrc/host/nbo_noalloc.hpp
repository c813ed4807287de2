// The library's statically allocated device scratch (nbo_noalloc.hip).
#ifndef NBO_NOALLOC_HPP
#define NBO_NOALLOC_HPP

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

// Layout of the 32 KiB array: [0, 16 KiB) f64 partial sums, [16 KiB, 24 KiB) u32 flags,
// the rest unused.  2048 is the norm pass's largest grid.
#define NBO_NOALLOC_SCRATCH_BYTES (32u * 1024u)
#define NBO_NOALLOC_MAX_PARTIALS 2048u
#define NBO_NOALLOC_FLAGS_OFFSET (NBO_NOALLOC_MAX_PARTIALS * 8u)
#define NBO_NOALLOC_MAX_DEVICES 64

namespace nbo {

// Looks up the device address of the scratch array on the current device (once per device;
// later calls return at once).  *device_out receives the current device.  Allocates nothing.
hipError_t noalloc_setup(int *device_out);
// The address noalloc_setup found for `device`, or null if it has not run there.
void *noalloc_scratch(int device);

} // namespace nbo

#endif
