// Kernel-argument block of the wave-scaling kernel and its launcher.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "occupancy.h"

namespace hbt {

// Destinations handled by one launch; more are processed in successive launches.
constexpr int kMaxDestPerLaunch = 8;

// Consecutive records one thread of the kernel's main instantiation owns: each
// of its column accesses is one load or store of this many elements, and the
// columns must be aligned to that many elements (otherwise the one-record
// instantiation runs).  One is fastest at every size tried.
constexpr int kVectorRecords = 1;

// Everything about one (origin, destination) pair that does not depend on the
// record, computed in fp64 on the host in the reference's operation order
// (analyzer/habitat/analysis/wave_scaling/roofline.py:48-64, :107-108).
struct DestArgs {
  OccDevice dev;
  double ridge;                // peak_gflops / mem_bandwidth_gb
  double half_ridge;           // 0.5 * ridge
  double neg_half_over_ridge;  // -0.5 / ridge
  double log2_bw;              // log2(origin.mem_bandwidth_gb / dest.mem_bandwidth_gb)
  double log2_clk;             // log2(origin.base_clock_mhz / dest.base_clock_mhz)
  double log2_clk_sm;          // log2_clk + log2(origin.num_sms / dest.num_sms)
  float inv_sms;               // 1 / num_sms rounded to float

  bool ridge_in_range() const { return ridge >= 0x1p-500 && ridge <= 0x1p500; }
};

// Puts destinations with equal occupancy constants (everything in OccDevice but
// num_sms) next to each other and marks every destination that agrees with the
// one before it (kSameOccAsPrev), so that a kernel walking over dests[0..n)
// evaluates the occupancy model once per run of equal ones.  order[i] is the
// caller's index of the destination now at position i.
void group_by_occupancy(DestArgs* dests, int32_t* order, int n);

// Everything in the two but num_sms (and the kSameOccAsPrev mark) is equal.
bool same_occupancy_constants(OccDevice a, OccDevice b);

// The origin device's share of the constants.
struct OriginArgs {
  OccDevice dev;
  double peak_gflops;  // origin.peak_gflops_per_second
  float inv_sms;       // 1 / origin.num_sms rounded to float
};

// Where one destination's results go (row d of the [n_dest][n] outputs).  Kept
// per destination so that the kernel fetches these pointers when it reaches that
// destination's stores rather than holding them from its first instruction.
struct DestOut {
  double* time_ns;
  int32_t* occ;     // nullable
  int32_t* wave;    // nullable
  uint8_t* status;  // nullable
};

struct WaveScaleArgs {
  int64_t n;
  int32_t n_dest;
  int32_t write_origin;  // 1: this launch writes the per-record origin outputs
  const int32_t* num_blocks;
  const int32_t* block_size;
  const int32_t* dynamic_smem;
  const int32_t* static_smem;
  const int32_t* regs;
  const int32_t* dest_regs;    // nullable
  const double* run_time_ns;
  const double* flop_sp_efficiency;
  const double* dram_read_bytes;
  const double* dram_write_bytes;
  const uint8_t* has_metrics;  // nullable
  int32_t* out_occ_origin;     // [n], nullable
  int32_t* out_wave_origin;    // [n], nullable
  OriginArgs origin;
  DestArgs dest[kMaxDestPerLaunch];
  DestOut out[kMaxDestPerLaunch];
};

OriginArgs make_origin_args(const hbt_device_spec& origin);
DestArgs make_dest_args(const hbt_device_spec& origin, const hbt_device_spec& dest);

// Host side of a kernel that publishes `value` in host-visible memory when its
// results are in place (a system-scope release store after them): watches
// `flag` for up to about 200 microseconds.  False when the value did not show
// up; the caller then waits for the stream instead.
bool wait_published(const uint32_t* flag, uint32_t value);

// `vectorised` needs every column, and every destination's row of the outputs,
// aligned to kVectorRecords elements of its type.
hipError_t launch_wave_scale(const WaveScaleArgs& args, bool vectorised, hipStream_t stream);

}  // namespace hbt
