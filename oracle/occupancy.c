/*
 * TEST INFRASTRUCTURE — CPU oracle, not product code.
 *
 * Plain-C restatement of the thread-block occupancy calculation that the
 * reference reaches through KernelMetadata::threadBlockOccupancy
 * (cpp/src/cuda/kernel.cpp:29-56), written from the behaviour of
 * cudaOccMaxActiveBlocksPerMultiprocessor (cpp/src/cuda/cuda_occupancy.h:1289-1420)
 * as the reference configures it:
 *   - default device state: no cache preference, default carve-out
 *     (cuda_occupancy.h:483-487);
 *   - default function attributes: partitioned global caching off, default
 *     shared-memory limit (cuda_occupancy.h:444-452), then
 *     maxThreadsPerBlock = maxDynamicSharedSizeBytes = INT_MAX,
 *     numRegs = registers, sharedSizeBytes = static shared memory
 *     (kernel.cpp:37-41);
 *   - any error status is reported as occupancy 0 (kernel.cpp:45-53).
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this file's library.  It is checked against the compiled reference
 * (oracle/_ref, built by oracle/Makefile from the reference's own kernel.cpp)
 * and against the committed golden vectors in tests/golden/.
 *
 * Arithmetic is done in 64-bit so that no intermediate can overflow; wherever
 * the reference's 32-bit arithmetic does not overflow (which is undefined
 * behaviour there) the results are identical.
 */
#include <stdint.h>
#include <limits.h>
#include <stddef.h>

typedef struct {
  int32_t compute_major, compute_minor;
  int32_t max_threads_per_block, max_threads_per_sm;
  int32_t regs_per_block, regs_per_sm;
  int32_t warp_size, num_sms;
  int64_t smem_per_block, smem_per_sm, smem_per_block_optin;
  double mem_bandwidth_gb, base_clock_mhz, peak_gflops;
} orc_device;

typedef struct {
  int32_t regs, smem, warps, blocks; /* the four per-SM block limits */
  int32_t error;                     /* 1 when the reference returns an error status */
} orc_limits;

static int64_t ceil_div(int64_t x, int64_t y) { return (x + (y - 1)) / y; }
static int64_t round_up(int64_t x, int64_t y) { return y * ceil_div(x, y); }

/* Shared-memory pool sizes a cc 7.x SM can be configured to
 * (cuda_occupancy.h:699-746). */
static int64_t volta_align(const orc_device *d, int64_t size) {
  if (d->compute_minor == 5) {               /* Turing: 32 KB or everything */
    return size <= 32768 ? 32768 : d->smem_per_sm;
  }
  if (size == 0) return 0;                   /* Volta: 0/8/16/32/64 KB or everything */
  if (size <= 8192) return 8192;
  if (size <= 16384) return 16384;
  if (size <= 32768) return 32768;
  if (size <= 65536) return 65536;
  return d->smem_per_sm;
}

/* Register limit (cuda_occupancy.h:1165-1282) with `subparts` sub-partitions. */
static int64_t reg_limit(const orc_device *d, int64_t regs, int64_t warps_per_block,
                         int64_t subparts) {
  const int64_t gran = 256;                  /* cuda_occupancy.h:621-639 */
  const int64_t max_regs_per_thread = 256;   /* 3/5/6 fall through to 256: :600-608 */
  int64_t per_warp = round_up(regs * d->warp_size, gran);
  int64_t per_block = per_warp * warps_per_block;
  int64_t assumed = per_warp * round_up(warps_per_block, subparts);
  if (d->regs_per_block < assumed || d->regs_per_block < per_block ||
      regs > max_regs_per_thread)
    return 0;
  if (per_warp <= 0) return INT_MAX;
  /* caching is off, so the "try again" branch (:1262-1269) is the one taken */
  int64_t warps_per_subpart = (d->regs_per_sm / subparts) / per_warp;
  return (warps_per_subpart * subparts) / warps_per_block;
}

int orc_occupancy_limits(const orc_device *d, int32_t block, int32_t dyn_smem,
                         int32_t static_smem, int32_t registers, orc_limits *out) {
  out->regs = out->smem = out->warps = out->blocks = 0;
  out->error = 1;
  const int64_t regs = (uint16_t)registers;  /* kernel.h:108 narrows to uint16_t */

  /* input checks: cuda_occupancy.h:1307, :922-990.  The size_t fields can only
   * fail the "<= 0" test by being 0; sharedMemPerBlockOptin is not checked. */
  if (block <= 0) return 0;
  if (d->max_threads_per_block <= 0 || d->max_threads_per_sm <= 0 ||
      d->regs_per_block <= 0 || d->regs_per_sm <= 0 || d->warp_size <= 0 ||
      d->smem_per_block == 0 || d->smem_per_sm == 0 || d->num_sms <= 0)
    return 0;

  /* every architecture switch knows majors 3, 5, 6, 7 only (:573-694) */
  const int major = d->compute_major, minor = d->compute_minor;
  if (major != 3 && major != 5 && major != 6 && major != 7) return 0;

  const int64_t warps_per_block = ceil_div(block, d->warp_size);

  /* registers; GP100 (6.0) has 2 sub-partitions and is re-checked as GP10x
   * with 4 (:644-664, :1344-1361) */
  int64_t subparts = (major == 6 && minor == 0) ? 2 : 4;
  int64_t lim_regs = reg_limit(d, regs, warps_per_block, subparts);
  if (major == 6 && minor == 0 && lim_regs != 0) {
    if (reg_limit(d, regs, warps_per_block, 4) == 0) lim_regs = 0;
  }

  /* warps (:1016-1062) */
  int64_t lim_warps = 0;
  if (block <= d->max_threads_per_block)
    lim_warps = (d->max_threads_per_sm / d->warp_size) / warps_per_block;

  /* block slots (:670-694) */
  int64_t lim_blocks;
  if (major == 3) lim_blocks = 16;
  else if (major == 7) lim_blocks = (minor == 5) ? 16 : 32;
  else lim_blocks = 32;

  /* shared memory (:1066-1162).  Both sizes reach the routine as size_t and
   * their sum is cast to int (:1101-1102): that is 32-bit wrap-around. */
  int64_t lim_smem;
  {
    int32_t total = (int32_t)((uint32_t)static_smem + (uint32_t)dyn_smem);
    int64_t alloc = round_up((int64_t)total, 256);        /* C division truncates */
    /* per-block limit: default config → sharedMemPerBlock (:866-897).  The
     * rounded size becomes a size_t again, so a negative one is enormous. */
    int exceeded = (alloc < 0) || ((uint64_t)alloc > (uint64_t)d->smem_per_block);
    if (exceeded) {
      lim_smem = 0;
    } else {
      int64_t pool;
      if (major == 7) {
        int64_t pref = volta_align(d, d->smem_per_sm);    /* :751-792, default carve-out */
        pool = (pref >= alloc) ? pref : volta_align(d, alloc);
      } else {
        pool = d->smem_per_sm;                            /* :818-840; fallback :1143-1146 is the same value */
      }
      if (alloc > 0) {
        int64_t q = pool / alloc;
        lim_smem = (int32_t)q;                            /* (int) cast at :1150 */
      } else {
        lim_smem = INT_MAX;
      }
    }
  }

  out->regs = (int32_t)lim_regs;
  out->smem = (int32_t)lim_smem;
  out->warps = (int32_t)lim_warps;
  out->blocks = (int32_t)lim_blocks;
  out->error = 0;
  int64_t m = lim_regs;
  if (lim_smem < m) m = lim_smem;
  if (lim_warps < m) m = lim_warps;
  if (lim_blocks < m) m = lim_blocks;
  return (int)m;
}

uint32_t orc_occupancy(const orc_device *d, int32_t block, int32_t dyn_smem,
                       int32_t static_smem, int32_t registers) {
  orc_limits l;
  return (uint32_t)orc_occupancy_limits(d, block, dyn_smem, static_smem, registers, &l);
}

/* Vector form for the numpy restatement of wave scaling: one occupancy per
 * record, `registers[i] < 0` meaning "use own_regs[i]" as in
 * cpp/src/frontend/model_bindings.cpp:75-82. */
void orc_occupancy_batch(const orc_device *d, int64_t n, const int32_t *block,
                         const int32_t *dyn_smem, const int32_t *static_smem,
                         const int32_t *own_regs, const int32_t *registers,
                         int32_t *out) {
  for (int64_t i = 0; i < n; ++i) {
    int32_t r = own_regs[i];
    if (registers != NULL && registers[i] >= 0) r = registers[i];
    out[i] = (int32_t)orc_occupancy(d, block[i], dyn_smem[i], static_smem[i], r);
  }
}
