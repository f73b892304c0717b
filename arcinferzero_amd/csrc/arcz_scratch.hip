// The library's static device scratch: one file-scope array in device memory that the allocation-free matmul entry
// point (arcz_engine_matmul_noalloc, include/arcz_engine.h) hands to the short-chunk GEMM as its workspace of partial
// tiles, in place of the buffer the engine allocates for the ordinary entry point.  Each GPU this library runs on
// holds its own copy of the array, at its own address, until the process ends.
//
// In host code the array's name is a host-side stand-in, not a device address.  The address is asked for once per
// device, with that device current (arcz_scratch_setup, called by arcz_init), and kept; everything else -- kernel
// arguments, clears, copies -- uses that pointer.
#include <hip/hip_runtime.h>

#include <cstddef>

#include "arcz_scratch.h"

// (No device code names the array: the kernels get its address as an argument.  The host's use below is what keeps it
//  in the code object, as a symbol the runtime can find; an explicit "used" attribute must not be added -- with it the
//  compiler leaves the symbol local to the code object, and the runtime's lookup then ends the process.)
static __device__ __align__(256) unsigned char scratch[ARCZ_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_ptr[kMaxDevices];  // the array's device address on each device that was set up
}  // namespace

extern "C" int arcz_scratch_setup(int device, void** ptr, size_t* bytes, const char** err) {
  if (device < 0 || device >= kMaxDevices) {
    if (err) *err = "device index past the table of scratch addresses";
    return -1;
  }
  if (!g_ptr[device]) {
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess || cur != device) {
      if (err) *err = "arcz_scratch_setup: the device is not the current one";
      return -1;
    }
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      if (err) *err = hipGetErrorString(e);
      return -1;
    }
    g_ptr[device] = p;
  }
  if (ptr) *ptr = g_ptr[device];
  if (bytes) *bytes = ARCZ_SCRATCH_BYTES;
  return 0;
}
