// Host-side state shared by the translation units of libiris_hip: the per-thread error and kernel
// names behind iris_hip_last_error() / iris_hip_last_kernel(), and cached device facts.
#pragma once

namespace iris_host {

// Record an argument error for the calling thread; returns hipErrorInvalidValue.
int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_last_error();
void set_last_kernel(const char* name);
// CU and XCD count of `device`; returns 0 or a hipError_t value.
int device_facts(int device, int* cu_count, int* xcc_count);

}  // namespace iris_host
