// Internal to the library (not part of the C ABI): the static device scratch of arcz_scratch.hip.
#pragma once
#include <stddef.h>

// 32 MiB: the most the short-chunk GEMM's partial tiles can take under the engine's launch rule (pieces x tiles within
// two work-groups per compute unit of a 256-unit device, tiles of at most 128 x 128 f32: 512 x 128 x 128 x 4 bytes).
#define ARCZ_SCRATCH_BYTES (32u << 20)

#ifdef __cplusplus
extern "C" {
#endif
// Once per device, with that device current: asks the HIP runtime for the array's address on this device and keeps
// it.  0 and *ptr / *bytes set, or -1 with *err pointing at a static message.
__attribute__((visibility("hidden"))) int arcz_scratch_setup(int device, void** ptr, size_t* bytes, const char** err);
// The runtime's non-owning handle onto the current device's scratch (made by arcz_init), NULL before arcz_init.
struct arcz_mem;
__attribute__((visibility("hidden"))) struct arcz_mem* arcz_scratch_mem(void);
#ifdef __cplusplus
}
#endif
