// Thread-block occupancy model, shared by the host entry points and the HIP
// wave-scaling kernel.
//
// Computes what the reference obtains from KernelMetadata::threadBlockOccupancy
// (cpp/src/cuda/kernel.cpp:29-56), i.e. the minimum of four per-multiprocessor
// block limits (registers, shared memory, warp slots, block slots) under the
// default device state and function attributes that kernel.cpp:35-41 sets up.
// The behaviour is specified by cpp/src/cuda/cuda_occupancy.h:573-694 (per-
// architecture constants), :699-792 (shared-memory pool sizes on cc 7.x),
// :922-990 (input checks), :1016-1062 (warps), :1066-1162 (shared memory),
// :1165-1282 (registers) and :1289-1420 (combination, GP100 re-check).
//
// Layout of the work: everything that depends on the device alone is folded
// into an OccDevice on the host once per launch; the per-record part is a
// handful of integer operations and five divisions.  The divisions go through
// a policy: ExactDiv is plain 64-bit C division (host, and the kernel's rare
// slow path), FastDiv is a float-reciprocal division that is exact for
// operands below 2^22 (the kernel's fast path).
#pragma once

#include <climits>
#include <cstdint>

#include "../../include/habitat_mi.h"

#if defined(__HIPCC__)
#define HBT_HD __host__ __device__ __forceinline__
#else
#define HBT_HD inline
#endif

namespace hbt {

enum SmemArch : int32_t { kFixedPool = 0, kVolta = 1, kTuring = 2 };

// Device-only constants of the occupancy model.
struct OccDevice {
  int32_t ok;                 // 0: the model rejects this device -> occupancy 0 everywhere
  int32_t fast_ok;            // 1: every constant below is < 2^22 (FastDiv may be used)
  int32_t warp_size;
  int32_t warp_shift;         // log2(warp_size) when it is a power of two, else -1
  int32_t max_threads_per_block;
  int32_t max_warps_per_sm;   // max_threads_per_sm / warp_size
  int32_t regs_per_block;
  int32_t regs_per_subpart;   // regs_per_sm / subparts
  int32_t regs_per_subpart4;  // regs_per_sm / 4 (GP100 re-check)
  int32_t subparts;           // 4, or 2 on cc 6.0
  int32_t gp100;              // 1 on cc 6.0
  int32_t block_slots;
  int32_t smem_arch;          // SmemArch
  int32_t num_sms;
  int64_t smem_per_block;
  int64_t smem_per_sm;
  int64_t pref_pool;          // cc 7.x: the pool the default carve-out selects
};

HBT_HD int64_t volta_pool(int32_t arch, int64_t smem_per_sm, int64_t size) {
  if (arch == kTuring) return size <= 32768 ? 32768 : smem_per_sm;
  if (size == 0) return 0;
  if (size <= 8192) return 8192;
  if (size <= 16384) return 16384;
  if (size <= 32768) return 32768;
  if (size <= 65536) return 65536;
  return smem_per_sm;
}

// Host-side folding of a device spec (cuda_occupancy.h:922-958 for the checks).
inline OccDevice make_occ_device(const hbt_device_spec& s) {
  OccDevice d{};
  const int major = s.compute_major, minor = s.compute_minor;
  const bool known = (major == 3 || major == 5 || major == 6 || major == 7);
  const bool limits_ok = s.max_threads_per_block > 0 && s.max_threads_per_sm > 0 &&
                         s.regs_per_block > 0 && s.regs_per_sm > 0 && s.warp_size > 0 &&
                         s.smem_per_block != 0 && s.smem_per_sm != 0 && s.num_sms > 0;
  d.ok = (known && limits_ok) ? 1 : 0;
  d.warp_size = s.warp_size > 0 ? s.warp_size : 1;
  d.warp_shift = -1;
  if ((d.warp_size & (d.warp_size - 1)) == 0) {
    int sh = 0;
    while ((1 << sh) < d.warp_size) ++sh;
    d.warp_shift = sh;
  }
  d.max_threads_per_block = s.max_threads_per_block;
  d.max_warps_per_sm = s.max_threads_per_sm / d.warp_size;
  d.regs_per_block = s.regs_per_block;
  d.gp100 = (major == 6 && minor == 0) ? 1 : 0;
  d.subparts = d.gp100 ? 2 : 4;
  d.regs_per_subpart = s.regs_per_sm / d.subparts;
  d.regs_per_subpart4 = s.regs_per_sm / 4;
  d.block_slots = (major == 3) ? 16 : (major == 7 && minor == 5) ? 16 : 32;
  d.smem_arch = (major == 7) ? (minor == 5 ? kTuring : kVolta) : kFixedPool;
  d.num_sms = s.num_sms;
  d.smem_per_block = s.smem_per_block;
  d.smem_per_sm = s.smem_per_sm;
  d.pref_pool = (major == 7) ? volta_pool(d.smem_arch, s.smem_per_sm, s.smem_per_sm)
                             : s.smem_per_sm;
  const int64_t lim = (int64_t)1 << 22;
  d.fast_ok = (d.warp_size < lim && d.max_warps_per_sm < lim && d.regs_per_subpart < lim &&
               d.smem_per_sm < lim && d.smem_per_sm > 0 && d.pref_pool < lim &&
               d.smem_per_block > 0)
                  ? 1 : 0;
  return d;
}

struct ExactDiv {
  static HBT_HD int64_t div(int64_t a, int64_t b) { return a / b; }
};

#if defined(__HIPCC__)
// a / b for 0 <= a < 2^22, 0 < b < 2^22.  float(a), float(b) are exact, the
// hardware reciprocal is within 1 ulp and the product rounds once more, so the
// estimate is within 1 of the quotient; one correction step makes it exact.
struct FastDiv {
  static __device__ __forceinline__ int64_t div(int64_t a64, int64_t b64) {
    const int a = (int)a64, b = (int)b64;
    int q = (int)(__int2float_rn(a) * __builtin_amdgcn_rcpf(__int2float_rn(b)));
    int r = a - q * b;
    q += (r >= b) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return q;
  }
};
#endif

// The per-record part.  `regs` is already narrowed to 16 bits by the caller.
// Preconditions for FastDiv: d.fast_ok, block < 2^22, 0 <= static+dyn < 2^22 and
// regs * warp_size + 255 < 2^22 (callers test these and fall back to ExactDiv).
template <class Div>
HBT_HD int32_t occupancy_core(const OccDevice& d, int32_t block, int32_t smem_total, int32_t regs) {
  if (!d.ok || block <= 0) return 0;
  // Block too large: the warp limit is 0 and every limit is >= 0.
  if (block > d.max_threads_per_block) return 0;

  const int64_t warps = (d.warp_shift >= 0)
                            ? (((int64_t)block + d.warp_size - 1) >> d.warp_shift)
                            : Div::div((int64_t)block + d.warp_size - 1, d.warp_size);

  // --- registers -----------------------------------------------------------
  int64_t lim_regs;
  {
    const int64_t per_warp = (((int64_t)regs * d.warp_size + 255) >> 8) << 8;
    const int64_t sub = d.subparts;
    const int64_t assumed = per_warp * ((warps + sub - 1) & ~(sub - 1));
    if (d.regs_per_block < assumed || regs > 256) {
      lim_regs = 0;  // `assumed` >= the per-block allocation, one test covers both
    } else if (per_warp == 0) {
      lim_regs = INT_MAX;
    } else {
      lim_regs = Div::div(Div::div(d.regs_per_subpart, per_warp) * sub, warps);
      if (d.gp100 && lim_regs != 0) {
        // cc 6.0 must also fit a 4-sub-partition Pascal SM.
        const int64_t assumed4 = per_warp * ((warps + 3) & ~(int64_t)3);
        if (d.regs_per_block < assumed4 ||
            Div::div(d.regs_per_subpart4, per_warp) * 4 < warps)
          lim_regs = 0;
      }
    }
  }
  if (lim_regs == 0) return 0;

  // --- warp slots ------------------------------------------------------------
  const int64_t lim_warps = Div::div(d.max_warps_per_sm, warps);

  // --- shared memory ---------------------------------------------------------
  int64_t lim_smem;
  {
    // C division truncates toward zero: (total + 255) / 256 * 256.
    const int64_t t255 = (int64_t)smem_total + 255;
    const int64_t alloc = (t255 >= 0 ? (t255 >> 8) : -((-t255) >> 8)) << 8;
    if (alloc < 0 || alloc > d.smem_per_block) {
      lim_smem = 0;
    } else if (alloc == 0) {
      lim_smem = INT_MAX;
    } else {
      int64_t pool = d.pref_pool;
      if (d.smem_arch != kFixedPool && pool < alloc)
        pool = volta_pool(d.smem_arch, d.smem_per_sm, alloc);
      lim_smem = (int32_t)Div::div(pool, alloc);
    }
  }

  int64_t m = lim_regs;
  m = lim_smem < m ? lim_smem : m;
  m = lim_warps < m ? lim_warps : m;
  m = d.block_slots < m ? d.block_slots : m;
  return (int32_t)m;
}

// Wrap-around sum of the two shared-memory sizes: both reach the reference's
// routine as size_t and the sum is cast to int (cuda_occupancy.h:1101-1102).
HBT_HD int32_t smem_sum(int32_t static_smem, int32_t dynamic_smem) {
  return (int32_t)((uint32_t)static_smem + (uint32_t)dynamic_smem);
}

// Host / slow-path occupancy: no preconditions.
HBT_HD int32_t occupancy_exact(const OccDevice& d, int32_t block, int32_t dynamic_smem,
                               int32_t static_smem, int32_t regs) {
  return occupancy_core<ExactDiv>(d, block, smem_sum(static_smem, dynamic_smem),
                                  (int32_t)(uint16_t)regs);
}

}  // namespace hbt
