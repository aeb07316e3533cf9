// Tuning knobs and device facts shared by the launch code of every format.
//
// Every knob is an environment variable read once per process, the first time it is consulted; the defaults are the
// measured choices and none is needed in production.  mfq_hip_config() lists the effective values.
#pragma once
#include <stddef.h>

namespace mfq {

// Effective value of the knob `name` (must be one of the names in tune.hip's table): the environment's integer when
// set, else `dflt`.
int tune_env(const char *name, int dflt);

// Compute units of the current device (hipDeviceAttributeMultiprocessorCount, queried once per device), or the
// value given to mfq_hip_set_cu_count while that is non-zero.
int device_cu_count();
// the same without mfq_hip_set_cu_count's override: what the device really has
int device_real_cu_count();

// Largest dynamic LDS a block may ask for on gfx950 (160 KB per CU); above 64 KB the kernel has to opt in.
constexpr size_t kMaxDynamicLds = 160 * 1024;
// Opt-in for `lds` bytes of dynamic LDS (no-op up to 64 KB).  Returns an MFQ status.
int allow_dynamic_lds(const void *kernel, size_t lds, const char *what);

}  // namespace mfq
