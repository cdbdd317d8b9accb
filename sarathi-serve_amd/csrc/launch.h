// Host-side helpers shared by the entry points: argument checks and the
// launch-status query.  Entry points never synchronise, allocate or throw.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sarathi_ops.h"

namespace sarathi_hip {

// grid.y / grid.z limit of a launch; token rows above it spill into grid.z
constexpr int kMaxGridY = 65535;

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Status of the launch just issued on this thread (hipGetLastError is
// per-thread and clears the sticky value).
static inline int launch_status() {
  return hipGetLastError() == hipSuccess ? SARATHI_OK : SARATHI_ERR_LAUNCH;
}

}  // namespace sarathi_hip
