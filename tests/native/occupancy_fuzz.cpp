// Host-side fuzz of the library's occupancy code under AddressSanitizer and
// UndefinedBehaviorSanitizer (built and run by tests/test_host_sanitized.py).
//
// Includes habitat_amd/csrc/occupancy.h as plain C++ (no HIP): the 64-bit model
// (occupancy_exact: what hbt_occupancy_host* run), the 32-bit model the kernels
// run (occupancy_fast, with the host's exact divisions) and the compute-unit
// model, over random device descriptions and launch configurations that include
// zeros, negatives, INT_MIN / INT_MAX and values around every limit.  The 64-bit
// and 32-bit models are compared with each other and, for NVIDIA-rule devices,
// with the CPU oracle (oracle/occupancy.c, linked in).  Any signed overflow,
// out-of-range shift or bad memory access in the host code aborts the run.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>

#include "../../habitat_amd/csrc/occupancy.h"

extern "C" {
typedef struct {
  int32_t compute_major, compute_minor;
  int32_t max_threads_per_block, max_threads_per_sm;
  int32_t regs_per_block, regs_per_sm;
  int32_t warp_size, num_sms;
  int64_t smem_per_block, smem_per_sm, smem_per_block_optin;
  double mem_bandwidth_gb, base_clock_mhz, peak_gflops;
} orc_device;
uint32_t orc_occupancy(const orc_device* d, int32_t block, int32_t dyn_smem, int32_t static_smem,
                       int32_t regs);
}

namespace {

template <class T, size_t N>
T pick(std::mt19937_64& rng, const T (&values)[N]) {
  return values[rng() % N];
}

int32_t odd_int(std::mt19937_64& rng, int32_t ordinary_max) {
  static const int32_t odd[] = {0, -1, 1, 31, 32, 33, 255, 256, 257, 1023, 1024, 1025, 65535, 65536,
                                65537, 1 << 20, (1 << 20) - 1, INT32_MAX, INT32_MIN, -256, -510, -511,
                                49152, 49153, 98304, 163840, 163841};
  if (rng() % 5 == 0) return pick(rng, odd);
  return (int32_t)(rng() % (uint64_t)(ordinary_max + 1));
}

}  // namespace

int main(int argc, char** argv) {
  const long devices = argc > 1 ? std::atol(argv[1]) : 400;
  const long launches = argc > 2 ? std::atol(argv[2]) : 2000;
  std::mt19937_64 rng(12345);
  long compared_oracle = 0, compared_fast = 0, nonzero = 0;
  for (long dv = 0; dv < devices; ++dv) {
    static const int32_t majors[] = {3, 5, 6, 6, 7, 7, 7, 8, 2, 9, 0, HBT_COMPUTE_MAJOR_CDNA,
                                     HBT_COMPUTE_MAJOR_CDNA};
    static const int32_t minors[] = {0, 0, 1, 2, 5, 7, 4};
    static const int32_t warps[] = {32, 32, 32, 64, 64, 16, 24, 48, 96, 128, 1, 1000, 32768};
    static const int32_t threads_block[] = {1024, 1024, 512, 2048, 1536, 100, 0, 65536, -4, 1 << 24};
    static const int32_t threads_sm[] = {2048, 1024, 1536, 4096, 768, 64, 0, 1 << 20, 2560, 1 << 26};
    static const int32_t regs_block[] = {65536, 32768, 131072, 4096, 0, 1 << 22, 100000, 1 << 30, -1};
    static const int32_t regs_sm[] = {65536, 131072, 262144, 32768, 100000, 0, 1 << 22, 1 << 30};
    static const int64_t smem_block[] = {49152, 65536, 98304, 16384, 163840, 1000, 0, 1 << 21,
                                         ((int64_t)1 << 31) - 1};
    static const int64_t smem_sm[] = {65536, 98304, 102400, 163840, 49152, 32768, 8192, 100, 0,
                                      1 << 21, ((int64_t)1 << 31) - 1};
    static const int32_t sms[] = {1, 14, 80, 256, 1000, 1 << 14, (1 << 14) + 1, 1 << 20};
    hbt_device_spec s{};
    s.compute_major = pick(rng, majors);
    s.compute_minor = pick(rng, minors);
    s.max_threads_per_block = pick(rng, threads_block);
    s.max_threads_per_sm = pick(rng, threads_sm);
    s.regs_per_block = pick(rng, regs_block);
    s.regs_per_sm = pick(rng, regs_sm);
    s.warp_size = pick(rng, warps);
    s.num_sms = pick(rng, sms);
    s.smem_per_block = pick(rng, smem_block);
    s.smem_per_sm = pick(rng, smem_sm);
    s.smem_per_block_optin = 0;
    s.mem_bandwidth_gb = 900; s.base_clock_mhz = 1300; s.peak_gflops = 14000;
    const hbt::OccDevice d = hbt::make_occ_device(s);
    const bool cdna = s.compute_major == HBT_COMPUTE_MAJOR_CDNA;
    orc_device o{};
    o.compute_major = s.compute_major; o.compute_minor = s.compute_minor;
    o.max_threads_per_block = s.max_threads_per_block; o.max_threads_per_sm = s.max_threads_per_sm;
    o.regs_per_block = s.regs_per_block; o.regs_per_sm = s.regs_per_sm;
    o.warp_size = s.warp_size; o.num_sms = s.num_sms;
    o.smem_per_block = s.smem_per_block; o.smem_per_sm = s.smem_per_sm;
    for (long i = 0; i < launches; ++i) {
      const int32_t block = odd_int(rng, 2100), dyn = odd_int(rng, 120000),
                    stat = odd_int(rng, 60000), regs = odd_int(rng, 300);
      const int32_t exact = hbt::occupancy_exact(d, block, dyn, stat, regs);
      nonzero += exact != 0;
      if (!cdna) {
        const uint32_t want = orc_occupancy(&o, block, dyn, stat, regs);
        if ((uint32_t)exact != want) {
          std::printf("MISMATCH oracle: cc %d.%d block %d dyn %d stat %d regs %d: %d vs %u\n",
                      s.compute_major, s.compute_minor, block, dyn, stat, regs, exact, want);
          return 1;
        }
        ++compared_oracle;
      }
      if (d.fast_ok()) {
        const int32_t total = hbt::smem_sum(stat, dyn);
        const int32_t r16 = regs & 0xFFFF;
        int32_t fast;
        if (cdna) fast = hbt::occupancy_cdna<false>(d, block, total, r16);
        else fast = hbt::occupancy_fast(d, block, hbt::smem_alloc(total), r16);
        if (fast != exact) {
          std::printf("MISMATCH 32-bit model: cc %d.%d block %d dyn %d stat %d regs %d: %d vs %d\n",
                      s.compute_major, s.compute_minor, block, dyn, stat, regs, fast, exact);
          return 1;
        }
        ++compared_fast;
      }
    }
  }
  std::printf("ok: %ld against the oracle, %ld 32-bit against 64-bit, %ld non-zero\n", compared_oracle,
              compared_fast, nonzero);
  return (compared_oracle > 0 && compared_fast > 0 && nonzero > 0) ? 0 : 2;
}
