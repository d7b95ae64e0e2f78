// Host-side state shared by the translation units of libiris_hip: the per-thread error and kernel
// names behind iris_hip_last_error() / iris_hip_last_kernel(), and cached device facts.
#pragma once

#include <hip/hip_runtime.h>

namespace iris_host {

// Record an argument error for the calling thread; returns hipErrorInvalidValue.
int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_last_error();
void set_last_kernel(const char* name);
// CU and XCD count of `device`; returns 0 or a hipError_t value.
int device_facts(int device, int* cu_count, int* xcc_count);
// Workspace of a launch that splits tiles between workgroups: `nwg` slots of `slot_bytes` for partial
// sums, `nwg` flags, and the value the flags take in this launch.  One workspace per (device, stream),
// allocated on the stream's first such launch and kept until the process ends; launches on one stream
// are ordered, so they can share it.  Returns 0, or non-zero when there is none to be had (the stream is
// being captured, a device's eight workspaces are taken, the allocation failed):
// the caller then launches without splitting tiles.
// -1 decide per launch, 0 never split tiles, 1 split whenever the last round of tiles is not full.
int split_tile_mode();
void set_split_tile_mode(int mode);
int split_tile_workspace(int device, hipStream_t stream, int nwg, long long slot_bytes, char** partials, int** flags, int* epoch);

}  // namespace iris_host
