// TEST INFRASTRUCTURE — builds only where the reference tree is mounted.
//
// A C-callable face for the reference's own occupancy routine, so that the
// oracle in occupancy.c (and the product) can be compared with the real thing.
// This file contains no reference code: it includes the reference's kernel.h
// from where it lies and is linked with the reference's kernel.cpp by
// oracle/Makefile.  The argument order follows the DeviceProperties
// constructor (cpp/src/cuda/kernel.h:14-46) and the KernelMetadata
// constructor (cpp/src/cuda/kernel.h:66-79).
#include <cstdint>
#include <string>

#include "kernel.h"

extern "C" {

struct ref_device {
  int32_t compute_major, compute_minor;
  int32_t max_threads_per_block, max_threads_per_sm;
  int32_t regs_per_block, regs_per_sm;
  int32_t warp_size, num_sms;
  int64_t smem_per_block, smem_per_sm, smem_per_block_optin;
  double mem_bandwidth_gb, base_clock_mhz, peak_gflops;
};

static habitat::cuda::DeviceProperties make_device(const ref_device* d) {
  return habitat::cuda::DeviceProperties(
      "dev", d->compute_major, d->compute_minor, d->max_threads_per_block,
      d->max_threads_per_sm, d->regs_per_block, d->regs_per_sm, d->warp_size,
      (size_t)d->smem_per_block, (size_t)d->smem_per_sm, d->num_sms,
      (size_t)d->smem_per_block_optin, (int)d->mem_bandwidth_gb,
      (size_t)d->base_clock_mhz, (size_t)d->peak_gflops);
}

// registers < 0 selects the kernel's own register count, as the Python binding
// does (cpp/src/frontend/model_bindings.cpp:75-82).
uint32_t ref_occupancy(const ref_device* d, int32_t block, int32_t dyn_smem,
                       int32_t static_smem, int32_t own_regs, int32_t registers) {
  habitat::cuda::DeviceProperties dev = make_device(d);
  habitat::cuda::KernelMetadata k("k", 1, block, dyn_smem, static_smem,
                                  (uint16_t)own_regs);
  if (registers < 0) return k.threadBlockOccupancy(dev);
  return k.threadBlockOccupancy(dev, (uint16_t)registers);
}

void ref_occupancy_batch(const ref_device* d, int64_t n, const int32_t* block,
                         const int32_t* dyn_smem, const int32_t* static_smem,
                         const int32_t* own_regs, const int32_t* registers,
                         int32_t* out) {
  habitat::cuda::DeviceProperties dev = make_device(d);
  for (int64_t i = 0; i < n; ++i) {
    habitat::cuda::KernelMetadata k("k", 1, block[i], dyn_smem[i], static_smem[i],
                                    (uint16_t)own_regs[i]);
    if (registers == nullptr || registers[i] < 0)
      out[i] = (int32_t)k.threadBlockOccupancy(dev);
    else
      out[i] = (int32_t)k.threadBlockOccupancy(dev, (uint16_t)registers[i]);
  }
}

}  // extern "C"
