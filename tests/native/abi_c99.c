/* The C ABI used from plain C99, without Python: the header compiles as C, the
 * structures have the sizes the kernels assume, and the host-only entry points
 * answer (occupancy of a known launch on a V100-like device, error strings,
 * argument checks).  Linked against libhabitat_mi.so by tests/test_host.py. */
#include <stdio.h>
#include <string.h>

#include "habitat_mi.h"

int main(void) {
  hbt_device_spec v100;
  uint32_t occ = 0;
  memset(&v100, 0, sizeof v100);
  v100.compute_major = 7;
  v100.compute_minor = 0;
  v100.max_threads_per_block = 1024;
  v100.max_threads_per_sm = 2048;
  v100.regs_per_block = 65536;
  v100.regs_per_sm = 65536;
  v100.warp_size = 32;
  v100.num_sms = 80;
  v100.smem_per_block = 49152;
  v100.smem_per_sm = 98304;
  v100.mem_bandwidth_gb = 739;
  v100.base_clock_mhz = 1312;
  v100.peak_gflops = 6716;

  if (sizeof(hbt_kernel_record) != 64 || sizeof(hbt_device_spec) != 80) return 1;
  if (hbt_version() != HBT_VERSION) return 2;
  if (hbt_device_spec_check(&v100) != HBT_OK) return 3;
  /* 256 threads, 32 registers, no shared memory: 8 blocks of 8 warps fill 64 warp slots */
  if (hbt_occupancy_host(&v100, 256, 0, 0, 32, &occ) != HBT_OK || occ != 8) return 4;
  /* 1024 threads x 255 registers do not fit the register file */
  if (hbt_occupancy_host(&v100, 1024, 0, 0, 255, &occ) != HBT_OK || occ != 0) return 5;
  if (hbt_occupancy_host(NULL, 256, 0, 0, 32, &occ) != HBT_EINVAL) return 6;
  v100.mem_bandwidth_gb = 0;
  if (hbt_device_spec_check(&v100) != HBT_ESPEC) return 7;
  if (strcmp(hbt_strerror(HBT_OK), "ok") != 0 || hbt_strerror(HBT_ESIZE)[0] == '\0') return 8;
  if (hbt_wave_scale_host_records(&v100, &v100, 0, NULL, NULL, NULL, NULL, NULL, NULL) != HBT_ESPEC)
    return 9;
  printf("ok: habitat_mi ABI %d from C99\n", hbt_version());
  return 0;
}
