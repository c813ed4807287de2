// Scratch memory for the entry point that allocates nothing (nbo_fused_step_noalloc).
//
// The fused step's norm pass needs device memory beyond the caller's tensors and the
// optimizer's state: one partial sum of squares and one found-inf flag per workgroup of its
// fixed grid.  The ordinary entry points take that from a hipMalloc made by nbo_init.  Callers
// that cannot tolerate any allocation -- code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc -- get the same memory from the file-scope array below,
// which is part of this library's device image: every GPU the library runs on holds its own
// copy, at its own address, from the moment the image is loaded until the process ends.
//
// In host code the array's name is only a handle for hipGetSymbolAddress, never an address a
// kernel may be given: the address is looked up once per device (noalloc_setup, called by the
// runtime's constructor with that device current) and everything else -- kernel arguments,
// clears -- uses the looked-up pointer.
#include <hip/hip_runtime.h>

#include "nbo_noalloc.hpp"

static_assert(NBO_NOALLOC_SCRATCH_BYTES % 256 == 0, "scratch size is a whole number of 256-byte lines");
static_assert(NBO_NOALLOC_MAX_PARTIALS * (sizeof(double) + sizeof(uint32_t)) <= NBO_NOALLOC_SCRATCH_BYTES,
              "scratch holds one f64 partial sum and one u32 flag per workgroup of the norm grid");

static __device__ __align__(256) unsigned char scratch[NBO_NOALLOC_SCRATCH_BYTES];

namespace nbo {

namespace {
void *g_scratch_ptr[NBO_NOALLOC_MAX_DEVICES] = {}; // device address of `scratch`, per device
}

hipError_t noalloc_setup(int *device_out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (device_out) *device_out = dev;
    if (dev < 0 || dev >= NBO_NOALLOC_MAX_DEVICES) return hipErrorInvalidDevice;
    if (g_scratch_ptr[dev]) return hipSuccess;
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!ptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = ptr;
    return hipSuccess;
}

void *noalloc_scratch(int device)
{
    return device >= 0 && device < NBO_NOALLOC_MAX_DEVICES ? g_scratch_ptr[device] : nullptr;
}

} // namespace nbo
