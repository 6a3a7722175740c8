// C ABI of the library (include/habitat_mi.h): argument checking, host-side
// folding of device constants, launches.  No allocation happens here.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "../../include/habitat_mi.h"
#include "occupancy.h"
#include "wave_scale.h"

namespace hbt {

OriginArgs make_origin_args(const hbt_device_spec& o) {
  OriginArgs a{};
  a.dev = make_occ_device(o);
  a.peak_gflops = o.peak_gflops;
  a.inv_sms = 1.0f / (float)o.num_sms;
  return a;
}

DestArgs make_dest_args(const hbt_device_spec& o, const hbt_device_spec& d) {
  DestArgs p{};
  p.dev = make_occ_device(d);
  p.inv_sms = 1.0f / (float)d.num_sms;
  p.ridge = d.peak_gflops / d.mem_bandwidth_gb;
  p.half_ridge = 0.5 * p.ridge;
  p.neg_half_over_ridge = -0.5 / p.ridge;
  const double bw_ratio = o.mem_bandwidth_gb / d.mem_bandwidth_gb;
  const double clk_ratio = o.base_clock_mhz / d.base_clock_mhz;
  const double sm_ratio = (double)o.num_sms / (double)d.num_sms;
  p.log2_bw = std::log2(bw_ratio);
  p.log2_clk = std::log2(clk_ratio);
  p.log2_clk_sm = p.log2_clk + std::log2(sm_ratio);
  return p;
}

bool same_occupancy_constants(OccDevice a, OccDevice b) {
  a.num_sms = b.num_sms = 0;
  a.flags &= ~kSameOccAsPrev;
  b.flags &= ~kSameOccAsPrev;
  return std::memcmp(&a, &b, sizeof(OccDevice)) == 0;
}

void group_by_occupancy(DestArgs* dests, int32_t* order, int n) {
  if (n <= 1) {
    if (n == 1) {
      order[0] = 0;
      dests[0].dev.flags &= ~kSameOccAsPrev;
    }
    return;
  }
  // class of a destination = position of the first one with its constants;
  // a stable sort by class keeps the caller's order within a class
  std::vector<int32_t> cls((size_t)n);
  for (int i = 0; i < n; ++i) {
    cls[i] = i;
    for (int j = 0; j < i; ++j)
      if (cls[j] == j && same_occupancy_constants(dests[j].dev, dests[i].dev)) {
        cls[i] = j;
        break;
      }
  }
  std::vector<int32_t> idx((size_t)n);
  for (int i = 0; i < n; ++i) idx[i] = i;
  std::stable_sort(idx.begin(), idx.end(), [&](int32_t a, int32_t b) { return cls[a] < cls[b]; });
  std::vector<DestArgs> sorted((size_t)n);
  for (int i = 0; i < n; ++i) {
    sorted[i] = dests[idx[i]];
    sorted[i].dev.flags &= ~kSameOccAsPrev;
    if (i > 0 && cls[idx[i]] == cls[idx[i - 1]]) sorted[i].dev.flags |= kSameOccAsPrev;
    order[i] = idx[i];
  }
  for (int i = 0; i < n; ++i) dests[i] = sorted[i];
}

// What make_occ_device needs: 32-bit shared-memory sizes and a bounded warp size.
static bool occupancy_spec_in_domain(const hbt_device_spec& s) {
  const int64_t two31 = (int64_t)1 << 31;
  return s.warp_size <= 32768 && s.smem_per_block >= 0 && s.smem_per_block < two31 &&
         s.smem_per_sm >= 0 && s.smem_per_sm < two31;
}

static bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

}  // namespace hbt

extern "C" {

int hbt_version(void) { return HBT_VERSION; }

const char* hbt_strerror(int code) {
  switch (code) {
    case HBT_OK: return "ok";
    case HBT_EINVAL: return "invalid argument (null pointer, negative count or bad value)";
    case HBT_ESPEC: return "device spec outside the supported domain";
    case HBT_EHIP: return "HIP runtime error (no GPU, bad stream or failed launch)";
    case HBT_ENOMEM: return "device memory allocation failed";
    case HBT_EALIGN: return "column pointer not aligned to its element size";
    case HBT_ESIZE: return "size beyond what this entry point supports";
    default: return "unknown error code";
  }
}

int hbt_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

int hbt_device_spec_check(const hbt_device_spec* s) {
  if (s == nullptr) return HBT_EINVAL;
  const int64_t two31 = (int64_t)1 << 31;
  if (s->smem_per_block < 0 || s->smem_per_block >= two31) return HBT_ESPEC;
  if (s->smem_per_sm < 0 || s->smem_per_sm >= two31) return HBT_ESPEC;
  if (s->smem_per_block_optin < 0 || s->smem_per_block_optin >= two31) return HBT_ESPEC;
  if (s->warp_size > 32768) return HBT_ESPEC;
  // wave size = num_sms x occupancy (at most 63) is formed in 24-bit arithmetic
  if (s->num_sms > (1 << 20)) return HBT_ESPEC;
  // An AMD compute-unit description holds as many one-wave work-groups as it
  // has wave slots; the small-kernel factor's logarithm table ends at 63.
  if (s->compute_major == HBT_COMPUTE_MAJOR_CDNA && s->warp_size > 0 &&
      s->max_threads_per_sm / s->warp_size > 63)
    return HBT_ESPEC;
  const double f[3] = {s->mem_bandwidth_gb, s->base_clock_mhz, s->peak_gflops};
  for (double v : f)
    if (!(v > 0) || !std::isfinite(v)) return HBT_ESPEC;
  return HBT_OK;
}

int hbt_occupancy_host(const hbt_device_spec* spec, int32_t block_size, int32_t dynamic_smem,
                       int32_t static_smem, int32_t regs, uint32_t* out) {
  if (spec == nullptr || out == nullptr) return HBT_EINVAL;
  if (!hbt::occupancy_spec_in_domain(*spec)) return HBT_ESPEC;
  const hbt::OccDevice d = hbt::make_occ_device(*spec);
  *out = (uint32_t)hbt::occupancy_exact(d, block_size, dynamic_smem, static_smem, regs);
  return HBT_OK;
}

int hbt_occupancy_host_batch(const hbt_device_spec* spec, int64_t n, const int32_t* block_size,
                             const int32_t* dynamic_smem, const int32_t* static_smem,
                             const int32_t* regs, int32_t* out) {
  if (spec == nullptr || n < 0) return HBT_EINVAL;
  if (n > 0 && (!block_size || !dynamic_smem || !static_smem || !regs || !out)) return HBT_EINVAL;
  if (!hbt::occupancy_spec_in_domain(*spec)) return HBT_ESPEC;
  const hbt::OccDevice d = hbt::make_occ_device(*spec);
  for (int64_t i = 0; i < n; ++i)
    out[i] = hbt::occupancy_exact(d, block_size[i], dynamic_smem[i], static_smem[i], regs[i]);
  return HBT_OK;
}

int hbt_occupancy_host_model32_batch(const hbt_device_spec* spec, int64_t n,
                                     const int32_t* block_size, const int32_t* dynamic_smem,
                                     const int32_t* static_smem, const int32_t* regs,
                                     int32_t* out) {
  if (spec == nullptr || n < 0) return HBT_EINVAL;
  if (n > 0 && (!block_size || !dynamic_smem || !static_smem || !regs || !out)) return HBT_EINVAL;
  if (!hbt::occupancy_spec_in_domain(*spec)) return HBT_ESPEC;
  const hbt::OccDevice d = hbt::make_occ_device(*spec);
  if (!d.fast_ok()) return HBT_ESPEC;
  // the form the kernels run for this device: the straight-line one where the
  // device allows it
  const bool lean = d.lean_ok(), lean_gp = d.lean_gp_ok(), cdna_lean = d.cdna_lean_ok();
  for (int64_t i = 0; i < n; ++i) {
    const int32_t smem_total = hbt::smem_sum(static_smem[i], dynamic_smem[i]);
    const int32_t r = regs[i] & 0xFFFF;
    const int32_t b = block_size[i];
    if (d.flags & hbt::kCdna)
      out[i] = cdna_lean ? hbt::occupancy_cdna<false, true>(d, b, smem_total, r)
                         : hbt::occupancy_cdna<false>(d, b, smem_total, r);
    else
      out[i] = lean      ? hbt::occupancy_fast<true>(d, b, hbt::smem_alloc(smem_total), r)
               : lean_gp ? hbt::occupancy_fast<true, true>(d, b, hbt::smem_alloc(smem_total), r)
                         : hbt::occupancy_fast<false>(d, b, hbt::smem_alloc(smem_total), r);
  }
  return HBT_OK;
}

int hbt_wave_scale(const hbt_device_spec* origin, const hbt_device_spec* dests, int32_t n_dest,
                   int64_t n, const int32_t* num_blocks, const int32_t* block_size,
                   const int32_t* dynamic_smem, const int32_t* static_smem, const int32_t* regs,
                   const int32_t* dest_regs, const double* run_time_ns,
                   const double* flop_sp_efficiency, const double* dram_read_bytes,
                   const double* dram_write_bytes, const uint8_t* has_metrics,
                   double* out_time_ns, int32_t* out_occ_origin, int32_t* out_occ_dest,
                   int32_t* out_wave_origin, int32_t* out_wave_dest, uint8_t* out_status,
                   void* hip_stream) {
  using namespace hbt;
  if (origin == nullptr || dests == nullptr || n_dest < 0 || n < 0) return HBT_EINVAL;
  int rc = hbt_device_spec_check(origin);
  if (rc != HBT_OK) return rc;
  for (int32_t d = 0; d < n_dest; ++d)
    if ((rc = hbt_device_spec_check(&dests[d])) != HBT_OK) return rc;
  if (n == 0 || n_dest == 0) return HBT_OK;
  if (!num_blocks || !block_size || !dynamic_smem || !static_smem || !regs || !run_time_ns ||
      !flop_sp_efficiency || !dram_read_bytes || !dram_write_bytes || !out_time_ns)
    return HBT_EINVAL;
  if (n > ((int64_t)1 << 36)) return HBT_ESIZE;  // 128 records per workgroup: the grid stays far below 2^31

  const void* i32_cols[] = {num_blocks, block_size, dynamic_smem, static_smem, regs, dest_regs,
                            out_occ_origin, out_occ_dest, out_wave_origin, out_wave_dest};
  const void* f64_cols[] = {run_time_ns, flop_sp_efficiency, dram_read_bytes, dram_write_bytes,
                            out_time_ns};
  // The main instantiation accesses kVectorRecords elements at a time: every
  // column, and every destination's row of an output ([n_dest][n]), must be
  // aligned to that many elements (with one record per thread that is the
  // element alignment already required).
  bool vec = true;
  for (const void* p : i32_cols) {
    if (!aligned(p, 4)) return HBT_EALIGN;
    vec = vec && aligned(p, 4 * kVectorRecords);
  }
  for (const void* p : f64_cols) {
    if (!aligned(p, 8)) return HBT_EALIGN;
    vec = vec && aligned(p, 8 * kVectorRecords);
  }
  vec = vec && aligned(has_metrics, kVectorRecords) && aligned(out_status, kVectorRecords);
  if (n_dest > 1 && (n % kVectorRecords) != 0) vec = false;

  if (hbt_device_count() <= 0) return HBT_EHIP;

  WaveScaleArgs a{};
  a.n = n;
  a.num_blocks = num_blocks; a.block_size = block_size; a.dynamic_smem = dynamic_smem;
  a.static_smem = static_smem; a.regs = regs; a.dest_regs = dest_regs;
  a.run_time_ns = run_time_ns; a.flop_sp_efficiency = flop_sp_efficiency;
  a.dram_read_bytes = dram_read_bytes; a.dram_write_bytes = dram_write_bytes;
  a.has_metrics = has_metrics;
  a.out_occ_origin = out_occ_origin; a.out_wave_origin = out_wave_origin;
  a.origin = make_origin_args(*origin);

  // Within a launch, destinations with equal occupancy constants go next to
  // each other: the kernel evaluates the occupancy model once per run of them.
  // Every destination keeps its own row of the outputs.
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  for (int32_t d0 = 0; d0 < n_dest; d0 += kMaxDestPerLaunch) {
    const int32_t nd = (n_dest - d0 < kMaxDestPerLaunch) ? (n_dest - d0) : kMaxDestPerLaunch;
    int32_t order[kMaxDestPerLaunch];
    for (int32_t k = 0; k < nd; ++k) a.dest[k] = make_dest_args(*origin, dests[d0 + k]);
    group_by_occupancy(a.dest, order, nd);
    a.n_dest = nd;
    a.write_origin = (d0 == 0) ? 1 : 0;
    for (int32_t k = 0; k < nd; ++k) {
      const int64_t off = (int64_t)(d0 + order[k]) * n;
      a.out[k].time_ns = out_time_ns + off;
      a.out[k].occ = out_occ_dest ? out_occ_dest + off : nullptr;
      a.out[k].wave = out_wave_dest ? out_wave_dest + off : nullptr;
      a.out[k].status = out_status ? out_status + off : nullptr;
    }
    if (launch_wave_scale(a, vec, stream) != hipSuccess) return HBT_EHIP;
  }
  return HBT_OK;
}

}  // extern "C"
