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
// into an OccDevice on the host once per launch (14 dwords, held in SGPRs by
// the kernel); the per-record part is a handful of integer operations and
// three divisions.  Two implementations of that part: occupancy_core in 64-bit
// arithmetic with plain C division (host, and the kernel variant for devices
// with huge limits), and occupancy_fast in 32-bit arithmetic with a
// float-reciprocal division that is exact for operands below 2^20 (the kernel's
// normal path, taken when every device constant is small enough — which every
// real device is).
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

// OccDevice::flags
enum : uint32_t {
  kOk = 1u << 0,         // the model accepts this device (else occupancy 0 everywhere)
  kFastOk = 1u << 1,     // every constant is below 2^20: occupancy_fast applies
  kGp100 = 1u << 2,      // cc 6.0: 2 sub-partitions, re-checked with 4
  kVolta = 1u << 3,      // cc 7.0/7.2: pool steps 0/8/16/32/64 KB/all
  kTuring = 1u << 4,     // cc 7.5: pool steps 32 KB/all
  kPoolSteps = 1u << 5,  // cc 7.x and a block's allocation can exceed pref_pool
  kWarpPow2 = 1u << 6,   // warp_size is a power of two: warp_shift is valid
  kCdna = 1u << 7,       // AMD compute-unit model (HBT_COMPUTE_MAJOR_CDNA): occupancy_cdna
  // Set by a launcher, not by make_occ_device: in the launch's array of
  // destinations this one has the occupancy constants of the one before it.
  kSameOccAsPrev = 1u << 8,
};

// Device-only constants of the occupancy model (14 dwords).  Every field fits 32 bits:
// hbt_device_spec_check bounds the shared-memory sizes below 2^31.
struct OccDevice {
  uint32_t flags;
  int32_t warp_size;
  int32_t warp_shift;         // log2(warp_size) when kWarpPow2
  int32_t sub_shift;          // log2(sub-partitions): 2, or 1 on cc 6.0
  int32_t max_threads_per_block;
  int32_t max_warps_per_sm;   // max_threads_per_sm / warp_size
  int32_t regs_per_block;
  int32_t regs_per_subpart;   // regs_per_sm / sub-partitions
  int32_t regs_per_subpart4;  // regs_per_sm / 4 (GP100 re-check)
  int32_t block_slots;
  int32_t num_sms;
  int32_t smem_per_block;
  int32_t smem_per_sm;
  int32_t pref_pool;          // cc 7.x: the pool the default carve-out selects

  // kCdna reuses two fields the compute-unit model has no other use for (the
  // struct stays at 14 dwords of kernel-argument space and SGPRs per device):
  // VGPRs per lane one SIMD holds (regs_per_sm / 4 / warp_size) ...
  HBT_HD int32_t vgprs_per_simd() const { return regs_per_subpart4; }
  // ... and the LDS allocation granule in bytes.
  HBT_HD int32_t lds_granule() const { return regs_per_block; }

  HBT_HD bool ok() const { return (flags & kOk) != 0; }
  HBT_HD bool fast_ok() const { return (flags & kFastOk) != 0; }
  // the kernels' lean instantiation: an accepted NVIDIA-rule device whose
  // model is straight-line code in 32-bit arithmetic (power-of-two warp size,
  // no cc 6.0 re-check, no cc 7.x pool steps)
  HBT_HD bool lean_ok() const {
    return (flags & (kOk | kFastOk | kWarpPow2 | kCdna | kGp100 | kPoolSteps)) ==
           (kOk | kFastOk | kWarpPow2);
  }
  // lean_ok, or that but for the cc 6.0 re-check (the P100), which the kernels
  // then apply by a select on the flag instead of a branch
  HBT_HD bool lean_gp_ok() const {
    return (flags & (kOk | kFastOk | kWarpPow2 | kCdna | kPoolSteps)) ==
           (kOk | kFastOk | kWarpPow2);
  }
  // likewise for the compute-unit model: an accepted AMD description with
  // small limits and a power-of-two wavefront size
  HBT_HD bool cdna_lean_ok() const {
    return (flags & (kOk | kFastOk | kWarpPow2 | kCdna)) == (kOk | kFastOk | kWarpPow2 | kCdna);
  }
};

// Shared-memory pool a cc 7.x SM is configured to for an allocation of `size`
// (written with selects: `size` differs per lane in the kernel).
HBT_HD int32_t volta_pool(uint32_t flags, int32_t smem_per_sm, int32_t size) {
  if (flags & kTuring) return size <= 32768 ? 32768 : smem_per_sm;
  int32_t p = smem_per_sm;
  p = size <= 65536 ? 65536 : p;
  p = size <= 32768 ? 32768 : p;
  p = size <= 16384 ? 16384 : p;
  p = size <= 8192 ? 8192 : p;
  p = size == 0 ? 0 : p;
  return p;
}

// Host-side folding of a device spec (cuda_occupancy.h:922-958 for the checks).
// Expects smem fields in [0, 2^31) and warp_size <= 32768 (callers check).
inline OccDevice make_occ_device(const hbt_device_spec& s) {
  OccDevice d{};
  const int major = s.compute_major, minor = s.compute_minor;
  const bool cdna = major == HBT_COMPUTE_MAJOR_CDNA;
  const bool known = (major == 3 || major == 5 || major == 6 || major == 7 || cdna);
  const bool limits_ok = s.max_threads_per_block > 0 && s.max_threads_per_sm > 0 &&
                         s.regs_per_block > 0 && s.regs_per_sm > 0 && s.warp_size > 0 &&
                         s.smem_per_block != 0 && s.smem_per_sm != 0 && s.num_sms > 0;
  const bool ok = known && limits_ok;
  const bool gp100 = (major == 6 && minor == 0);
  d.warp_size = s.warp_size > 0 ? s.warp_size : 1;
  const bool pow2 = (d.warp_size & (d.warp_size - 1)) == 0;
  if (pow2) {
    int sh = 0;
    while ((1 << sh) < d.warp_size) ++sh;
    d.warp_shift = sh;
  }
  d.sub_shift = gp100 ? 1 : 2;
  d.max_threads_per_block = s.max_threads_per_block;
  d.max_warps_per_sm = s.max_threads_per_sm / d.warp_size;
  d.regs_per_block = s.regs_per_block;
  d.regs_per_subpart = s.regs_per_sm >> d.sub_shift;
  d.regs_per_subpart4 = s.regs_per_sm / 4;
  d.block_slots = (major == 3) ? 16 : (major == 7 && minor == 5) ? 16 : 32;
  d.num_sms = s.num_sms;
  d.smem_per_block = (int32_t)s.smem_per_block;
  d.smem_per_sm = (int32_t)s.smem_per_sm;
  uint32_t flags = 0;
  if (ok) flags |= kOk;
  if (gp100) flags |= kGp100;
  if (major == 7) flags |= (minor == 5) ? kTuring : kVolta;
  if (pow2) flags |= kWarpPow2;
  d.pref_pool = (major == 7) ? volta_pool(flags, d.smem_per_sm, d.smem_per_sm) : d.smem_per_sm;
  if (major == 7 && d.pref_pool < d.smem_per_block) flags |= kPoolSteps;
  if (cdna) {
    flags |= kCdna;
    d.sub_shift = 2;    // 4 SIMDs per CU
    d.block_slots = 16; // work-groups of more than one wave a CU holds (barrier resources)
    d.regs_per_subpart4 = (s.regs_per_sm / 4) / d.warp_size;  // vgprs_per_simd()
    d.regs_per_block = (minor == 5) ? 1280 : 512;             // lds_granule()
  }
  // every division operand below 2^20 (so that dividend + divisor <= 2^21)
  const int32_t lim = 1 << 20;
  bool fast = !ok ||  // a rejected device needs no arithmetic at all
              (d.warp_size <= 1024 && d.max_threads_per_block < lim - 1024 &&
               d.max_warps_per_sm < lim && d.regs_per_subpart < lim &&
               d.smem_per_sm < lim && d.pref_pool < lim && d.smem_per_block < lim &&
               d.num_sms <= (1 << 14));
  // LDS sizes are rounded up to the granule before they divide the CU's LDS
  if (ok && cdna) fast = fast && d.smem_per_sm < lim / 2 && d.smem_per_block < lim / 2;
  if (fast) flags |= kFastOk;
  d.flags = flags;
  return d;
}

// Exact a / b for a >= 0, b > 0 and a + b <= 2^21, given rb = 1 / float(b) to
// within 1 ulp: floor((a + 1/2) * rb) in float arithmetic.  (a + 1/2) / b lies
// in [k + 1/(2b), k + 1 - 1/(2b)] for the quotient k; the computed value is off
// by a relative 1.5 * 2^-23 at most (reciprocal within an ulp, one rounding of
// the product), i.e. by less than (k + 1) * 1.5 * 2^-23 <= 1/(2b) as long as
// (k + 1) * b <= a + b <= 2^21, so truncation gives k with no correction step.
// On the host (used to test the 32-bit model) it is plain division.
HBT_HD float fast_rcp(int32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_rcpf(__int2float_rn(b));
#else
  return 1.0f / (float)b;
#endif
}

HBT_HD int32_t fast_div_r(int32_t a, int32_t b, float rb) {
#if defined(__HIP_DEVICE_COMPILE__)
  (void)b;
  return (int32_t)((__int2float_rn(a) + 0.5f) * rb);
#else
  (void)rb;
  return a / b;
#endif
}

HBT_HD int32_t fast_div(int32_t a, int32_t b) { return fast_div_r(a, b, fast_rcp(b)); }

HBT_HD int32_t mul_small(int32_t a, int32_t b) {  // both below 2^23, product below 2^31
#if defined(__HIP_DEVICE_COMPILE__)
  return __mul24(a, b);
#else
  return a * b;
#endif
}

// Wrap-around sum of the two shared-memory sizes: both reach the reference's
// routine as size_t and the sum is cast to int (cuda_occupancy.h:1101-1102).
HBT_HD int32_t smem_sum(int32_t static_smem, int32_t dynamic_smem) {
  return (int32_t)((uint32_t)static_smem + (uint32_t)dynamic_smem);
}

// The shared-memory allocation of a block: the same on every architecture the
// model knows (256-byte granularity), so it is computed once per record.
// The rounding is C division (truncating) and the rounded size is compared as
// an unsigned 64-bit value: (total + 255) / 256 is 0 for total in -510..0
// (nothing allocated) and negative, hence enormous, below that.  A sum the
// 32-bit model cannot hold (enormous, or 2^20 and more) is represented by an
// allocation of 2^20 bytes, which exceeds the per-block limit of every fast_ok
// device and so gives occupancy 0 there, as the true value would.
struct SmemAlloc {
  int32_t alloc;  // rounded allocation in bytes
  float rcp;      // 1 / max(alloc, 1)
};

HBT_HD SmemAlloc smem_alloc(int32_t smem_total) {
  SmemAlloc s;
  const bool representable = smem_total >= -510 && smem_total < (1 << 20) - 255;
  const int32_t t = smem_total > 0 ? smem_total : 0;
  s.alloc = representable ? ((t + 255) & ~255) : (1 << 20);
  s.rcp = fast_rcp(s.alloc > 0 ? s.alloc : 1);
  return s;
}

// The occupancy model in 32-bit arithmetic, for devices with kFastOk (every
// device constant below 2^20, warp size <= 1024).  Any int32 record is
// accepted: fields outside the range the divisions are exact for have
// closed-form answers on such a device.  `regs` is already narrowed to 16 bits.
//
// Written without data-dependent branches (a wavefront holds 64 different
// records): an invalid record keeps computing on clamped operands and its
// budget is zeroed.  Branches on device constants are wave-uniform.  The
// register and warp-slot limits share their divisor, and floor division is
// monotonic, so min(floor(a / w), floor(b / w)) is taken as floor(min(a, b) / w).
//
// LEAN: the device has lean_ok(), so none of the wave-uniform branches is
// compiled in and the whole model is one basic block.  GP_SELECT (with LEAN):
// the device has lean_gp_ok(); the cc 6.0 re-check is computed for every
// record and applied where the device's flag says so, still without a branch.
template <bool LEAN = false, bool GP_SELECT = false>
HBT_HD int32_t occupancy_fast(const OccDevice& d, int32_t block, const SmemAlloc& sm,
                              int32_t regs) {
  if (!LEAN && !d.ok()) return 0;
  // regs <= 256 is the per-thread limit; it also keeps regs * warp_size below 2^19
  const bool in_range = block > 0 && block <= d.max_threads_per_block && regs <= 256;
  block = in_range ? block : 1;
  regs = in_range ? regs : 0;

  const int32_t ws = d.warp_size;
  const int32_t warps = (LEAN || (d.flags & kWarpPow2)) ? ((block + ws - 1) >> d.warp_shift)
                                                      : fast_div(block + ws - 1, ws);
  const float rcp_warps = fast_rcp(warps);

  // registers: 256 per-warp granularity, allocated per sub-partition; a block
  // must fit the per-block limit with its warps rounded up to the sub-partitions
  // (in units of 256 registers the per-warp allocation is at most 2^10 and the
  // rounded warp count below 2^21: their product fits 32 bits, and comparing it
  // with floor(regs_per_block / 256) is the comparison of the full sizes)
  const int32_t per_warp256 = (mul_small(regs, ws) + 255) >> 8;
  const int32_t per_warp = per_warp256 << 8;
  const int32_t sub_mask = (1 << d.sub_shift) - 1;
  const int32_t warps_up = (warps + sub_mask) & ~sub_mask;
  const int32_t block_regs256 = d.regs_per_block >> 8;
  bool fits = mul_small(per_warp256, warps_up) <= block_regs256;
  const int32_t per_warp1 = per_warp > 0 ? per_warp : 1;
  const float rcp_per_warp = fast_rcp(per_warp1);
  const int32_t reg_warps = fast_div_r(d.regs_per_subpart, per_warp1, rcp_per_warp) << d.sub_shift;
  if (GP_SELECT || (!LEAN && (d.flags & kGp100))) {
    // cc 6.0 must also fit a 4-sub-partition Pascal SM
    const int32_t warps_up4 = (warps + 3) & ~3;
    const bool fits4 = mul_small(per_warp256, warps_up4) <= block_regs256 &&
                       (per_warp == 0 ||
                        (fast_div_r(d.regs_per_subpart4, per_warp1, rcp_per_warp) << 2) >= warps);
    fits = fits && (fits4 || (GP_SELECT && !(d.flags & kGp100)));
  }
  int32_t warp_budget = d.max_warps_per_sm;
  warp_budget = (per_warp > 0 && reg_warps < warp_budget) ? reg_warps : warp_budget;
  warp_budget = (in_range && fits) ? warp_budget : 0;
  int32_t lim = fast_div_r(warp_budget, warps, rcp_warps);
  lim = d.block_slots < lim ? d.block_slots : lim;

  // shared memory: an allocation above the per-block limit leaves no pool
  int32_t pool = d.pref_pool;
  if (!LEAN && (d.flags & kPoolSteps)) {
    const int32_t stepped = volta_pool(d.flags, d.smem_per_sm, sm.alloc);
    pool = pool < sm.alloc ? stepped : pool;
  }
  pool = sm.alloc <= d.smem_per_block ? pool : 0;
  const int32_t lim_smem = fast_div_r(pool, sm.alloc > 0 ? sm.alloc : 1, sm.rcp);
  lim = (sm.alloc > 0 && lim_smem < lim) ? lim_smem : lim;
  return lim;
}

// Work-groups per compute unit on an AMD CDNA device (kCdna), after the
// public occupancy rules of LLVM's AMDGPU backend (llvm/lib/Target/AMDGPU/Utils/
// AMDGPUBaseInfo.cpp: getNumWavesPerEUWithNumVGPRs, getMaxWorkGroupsPerCU,
// getLdsDwGranularity) for gfx90a and later, where a SIMD holds one unified file
// of 512 VGPRs per lane allocated in granules of 8:
//   waves per SIMD   = min(wave slots per SIMD, vgprs_per_simd / max(roundup(regs, 8), 8))
//   by waves         = 4 * waves per SIMD / waves per work-group
//   by work-group slots = all wave slots for one-wave work-groups, else 16
//   by LDS           = smem_per_sm / roundup(bytes, granule), if any is used
// and 0 for a launch the device cannot run (block size, registers per lane or
// LDS per work-group beyond the limits, or a negative size).  There is no
// counterpart in the reference.  `regs` is already narrowed to 16 bits.
// EXACT_DIV: plain integer division (host; devices outside kFastOk).
// LEAN: the caller has checked cdna_lean_ok(), so the tests that are uniform
// over a launch are not compiled in.
template <bool EXACT_DIV, bool LEAN = false>
HBT_HD int32_t occupancy_cdna(const OccDevice& d, int32_t block, int32_t smem_total, int32_t regs) {
  static_assert(!(EXACT_DIV && LEAN), "the lean form is the 32-bit one");
  if (!LEAN && !d.ok()) return 0;
  const bool in_range = block > 0 && block <= d.max_threads_per_block &&
                        regs <= d.vgprs_per_simd() && smem_total >= 0 &&
                        smem_total <= d.smem_per_block;
  block = in_range ? block : 1;
  regs = in_range ? regs : 0;
  const int32_t lds_bytes = in_range ? smem_total : 0;
  const int32_t slots_per_simd = d.max_warps_per_sm >> 2;
  int32_t alloc = (regs + 7) & ~7;
  alloc = alloc < 8 ? 8 : alloc;
  int32_t lim, lds, lim_lds;
  if (EXACT_DIV) {
    const int64_t waves = ((int64_t)block + d.warp_size - 1) / d.warp_size;
    int64_t per_simd = d.vgprs_per_simd() / alloc;
    per_simd = per_simd < slots_per_simd ? per_simd : slots_per_simd;
    int64_t l = (per_simd * 4) / waves;
    const int64_t group_slots = waves == 1 ? d.max_warps_per_sm : d.block_slots;
    lim = (int32_t)(group_slots < l ? group_slots : l);
    const int64_t rounded =
        (((int64_t)lds_bytes + d.lds_granule() - 1) / d.lds_granule()) * d.lds_granule();
    lds = rounded > 0 ? 1 : 0;
    lim_lds = (int32_t)(d.smem_per_sm / (rounded > 0 ? rounded : 1));
  } else {
    const int32_t ws = d.warp_size;
    const int32_t waves = (LEAN || (d.flags & kWarpPow2)) ? ((block + ws - 1) >> d.warp_shift)
                                                          : fast_div(block + ws - 1, ws);
    int32_t per_simd = fast_div(d.vgprs_per_simd(), alloc);
    per_simd = per_simd < slots_per_simd ? per_simd : slots_per_simd;
    lim = fast_div(per_simd << 2, waves);
    const int32_t group_slots = waves == 1 ? d.max_warps_per_sm : d.block_slots;
    lim = group_slots < lim ? group_slots : lim;
    const int32_t granules = fast_div(lds_bytes + d.lds_granule() - 1, d.lds_granule());
    lds = mul_small(granules, d.lds_granule());
    lim_lds = fast_div(d.smem_per_sm, lds > 0 ? lds : 1);
  }
  lim = (lds > 0 && lim_lds < lim) ? lim_lds : lim;
  return in_range ? lim : 0;
}

// The model without preconditions, in 64-bit arithmetic with C division (host,
// and the kernel variant for devices outside kFastOk).  `regs` is already
// narrowed to 16 bits; `smem_total` is smem_sum() of the two sizes.
HBT_HD int32_t occupancy_core(const OccDevice& d, int32_t block, int32_t smem_total, int32_t regs) {
  if (!d.ok() || block <= 0) return 0;
  // Block too large: the warp limit is 0 and every limit is >= 0.
  if (block > d.max_threads_per_block) return 0;

  const int64_t warps = ((int64_t)block + d.warp_size - 1) / d.warp_size;

  // --- registers -----------------------------------------------------------
  int64_t lim_regs;
  {
    const int64_t per_warp = (((int64_t)regs * d.warp_size + 255) >> 8) << 8;
    const int64_t sub = (int64_t)1 << d.sub_shift;
    const int64_t assumed = per_warp * ((warps + sub - 1) & ~(sub - 1));
    if (d.regs_per_block < assumed || regs > 256) {
      lim_regs = 0;  // `assumed` >= the per-block allocation, one test covers both
    } else if (per_warp == 0) {
      lim_regs = INT_MAX;
    } else {
      lim_regs = ((d.regs_per_subpart / per_warp) * sub) / warps;
      if ((d.flags & kGp100) && lim_regs != 0) {
        // cc 6.0 must also fit a 4-sub-partition Pascal SM.
        const int64_t assumed4 = per_warp * ((warps + 3) & ~(int64_t)3);
        if (d.regs_per_block < assumed4 || (d.regs_per_subpart4 / per_warp) * 4 < warps)
          lim_regs = 0;
      }
    }
  }
  if (lim_regs == 0) return 0;

  // --- warp slots ------------------------------------------------------------
  const int64_t lim_warps = d.max_warps_per_sm / warps;

  // --- shared memory ---------------------------------------------------------
  int64_t lim_smem;
  {
    // C division truncates toward zero: (total + 255) / 256 * 256.
    const int64_t t255 = (int64_t)smem_total + 255;
    const int64_t alloc = (t255 >= 0 ? (t255 >> 8) : -((-t255) >> 8)) * 256;
    if (alloc < 0 || alloc > d.smem_per_block) {
      lim_smem = 0;
    } else if (alloc == 0) {
      lim_smem = INT_MAX;
    } else {
      int64_t pool = d.pref_pool;
      if ((d.flags & (kVolta | kTuring)) && pool < alloc)
        pool = volta_pool(d.flags, d.smem_per_sm, (int32_t)alloc);  // alloc <= smem_per_block < 2^31
      lim_smem = (int32_t)(pool / alloc);
    }
  }

  int64_t m = lim_regs;
  m = lim_smem < m ? lim_smem : m;
  m = lim_warps < m ? lim_warps : m;
  m = d.block_slots < m ? d.block_slots : m;
  return (int32_t)m;
}

// Host / slow-path occupancy: no preconditions.
HBT_HD int32_t occupancy_exact(const OccDevice& d, int32_t block, int32_t dynamic_smem,
                               int32_t static_smem, int32_t regs) {
  const int32_t smem_total = smem_sum(static_smem, dynamic_smem);
  if (d.flags & kCdna) return occupancy_cdna<true>(d, block, smem_total, (int32_t)(uint16_t)regs);
  return occupancy_core(d, block, smem_total, (int32_t)(uint16_t)regs);
}

}  // namespace hbt
