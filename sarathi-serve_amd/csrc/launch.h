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

// Compute units of the current device (looked up once; 256 when the query fails).
static inline int compute_units() {
  static const int units = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    return n;
  }();
  return units;
}

// Rows per workgroup for the kernels that put R consecutive rows into one one-wave workgroup
// (fused_add_rms_norm, moe_sum).  Workgroups are dealt to the compute units in turn, so
// the launch lasts as long as the busiest unit: ceil(workgroups / units) * R rows.  Take the
// largest R (fewest weight fetches, fewest workgroups) among those with the shortest busiest
// unit, but keep one row per workgroup while that leaves fewer than two workgroups per unit
// (small batches need the parallelism more).  Measured at 2304 rows of 4096 bf16: R = 3 (768
// workgroups, 3 per unit) 12.4 us, R = 2 (1152, i.e. 4.5 per unit) 15.6 us, R = 1 13.8 us.
static inline int pick_rows_per_workgroup(int64_t rows, int max_rows_per_wg) {
  const int units = compute_units();
  int best = 1;
  int64_t best_cost = (rows + units - 1) / units;
  for (int r = 2; r <= max_rows_per_wg; ++r) {
    const int64_t wgs = (rows + r - 1) / r;
    if (wgs < 2 * (int64_t)units) break;
    const int64_t cost = (wgs + units - 1) / units * r;
    if (cost <= best_cost) {
      best = r;
      best_cost = cost;
    }
  }
  return best;
}

}  // namespace sarathi_hip
