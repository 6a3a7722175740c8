// Trace-level prediction for a sweep of destination devices: the sums the
// reference forms in Python after scaling each kernel, fused into the scaling.
//
//   hbt_wave_scale_sum   per destination d and segment s (one segment per
//                        forward/backward pass of an operation):
//                        sum over the segment's kernel records of the scaled
//                        time t'(d)  — the sum in RunTimePrediction.run_time_ms
//                        (analyzer/habitat/analysis/run_time.py:50-58) over the
//                        kernels Predictor._wave_scale predicted
//                        (analyzer/habitat/analysis/predictor.py:116-124).
//                        Scaled times never reach HBM: traffic is the record
//                        columns once per destination row of the grid (they stay
//                        in L2) plus 8 bytes per (destination, segment).  Sums of
//                        runs that span wavefronts meet in floating-point atomics.
//   hbt_wave_scale_sum_ordered
//                        the same sums for segments that are runs of consecutive
//                        records, added in the records' order as the reference
//                        adds them, without atomics: the scaled times pass
//                        through a caller's workspace and one thread per
//                        (segment, destination) adds them up.
//   hbt_ratio_scale      per destination and MLP-predicted operation:
//                        run_time_ms * pred_dest / pred_origin, negative -> 0
//                        (predictor.py:132-148 and :182,218,238,283), the
//                        per-destination sum of those and the number replaced.
//
// Destinations live in a device-resident table (hbt_device_table) so that one
// launch covers all of them: blockIdx.y is a group of destinations, and their
// constants come through scalar loads.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <new>
#include <vector>

#include "../../include/habitat_mi.h"
#include "occupancy.h"
#include "wave_scale.h"

#pragma clang fp contract(off)

#include "wave_scale_device.h"

struct hbt_device_table {
  int32_t n_dest;
  int32_t model;           // dev::kModel...: which occupancy models the kernel needs
  int device;
  hbt::OriginArgs origin;
  hbt::DestArgs* dests;    // device memory, [n_dest]
};

namespace hbt {
namespace {

using namespace dev;

constexpr int kBlock = 256;
// Destinations one thread of wave_scale_sum_kernel walks over (blockIdx.y counts
// groups of this many): the record is loaded and its origin part computed once
// per group, and the occupancy model runs once per run of destinations with
// equal occupancy constants within the group.
constexpr int kSumGroup = 8;

struct SumArgs {
  int64_t n;
  int32_t n_segments;
  int32_t n_dest;
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
  const int32_t* segment;      // nullable: all records in segment 0
  double* out_sum;             // [n_dest][n_segments]
  int32_t* out_bad;            // [n_dest], nullable
  double* work;                // ORDERED: [n_dest][n]
  const DestArgs* dests;
  OriginArgs origin;
};

__global__ void fill_zero_kernel(double* sums, int64_t n_sums, int32_t* bad, int32_t n_bad) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_sums) sums[i] = 0.0;
  if (bad != nullptr && i < n_bad) bad[i] = 0;
}

// One thread per record and group of kSumGroup destinations.  Within a
// wavefront, consecutive records of the same segment are summed with a
// segmented scan and the last lane of each run adds the run's total to the
// segment's sum, per destination.
// ORDERED: no sums here; each scaled time (+0 where the reference would raise)
// goes to a.work[destination][record] for segment_sum_ordered_kernel to add up
// in the records' order.
template <int MODEL, bool ORDERED>
__global__ __launch_bounds__(kBlock) void wave_scale_sum_kernel(const SumArgs a) {
  const int d0 = blockIdx.y * kSumGroup;
  const int d1 = d0 + kSumGroup < a.n_dest ? d0 + kSumGroup : a.n_dest;
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const bool in_range = i < a.n;
  const int64_t j = in_range ? i : 0;

  RecordIn r;
  r.nb = a.num_blocks[j];
  r.block = a.block_size[j];
  r.smem_total = smem_sum(a.static_smem[j], a.dynamic_smem[j]);
  r.regs = a.regs[j];
  r.dest_regs = a.dest_regs != nullptr ? a.dest_regs[j] : -1;
  r.metrics = a.has_metrics != nullptr ? a.has_metrics[j] != 0 : true;
  r.t = a.run_time_ns[j];
  r.eff = a.flop_sp_efficiency[j];
  r.rd = a.dram_read_bytes[j];
  r.wr = a.dram_write_bytes[j];
  // lanes past the end form a run of their own so that they never swallow a tail
  const int32_t seg = (in_range && !ORDERED) ? (a.segment != nullptr ? a.segment[j] : 0) : -1;

  RecordMid m = origin_part<MODEL>(a.origin, r);
  if (__builtin_expect(m.redo_gflops, 0))
    m.num_gflops = origin_gflops_exact(a.origin.peak_gflops, r.eff, r.t);
  finish_mid<false>(m, 0.0);

  // Runs of equal segment ids get increasing run numbers, so that equal run
  // numbers at any distance mean "same run" even if a segment id repeats later.
  const int32_t prev_seg = __shfl_up(seg, 1);
  const bool head = lane == 0 || prev_seg != seg;
  const unsigned long long heads = __ballot(head);
  const int32_t run = (int32_t)__popcll(heads & ((2ull << lane) - 1ull));
  const int32_t next_run = __shfl_down(run, 1);
  const bool tail = lane == 63 || next_run != run;
  const bool adds = tail && in_range && seg >= 0 && seg < a.n_segments;

  int32_t occ_d = 0;
  for (int d = d0; d < d1; ++d) {
    const DestArgs& p = a.dests[d];
    // the first destination of a group never carries the mark
    if (!(p.dev.flags & kSameOccAsPrev)) occ_d = dest_occupancy<MODEL>(p, r, m);
    const double gamma = roofline_gamma(p, m.num_gflops, m.total_gb, r.metrics);
    RecordOut o = dest_scale<MODEL, false>(p, r, m, occ_d, gamma, 0.0);
    if (__builtin_expect(o.in_order, 0))
      o.t = scaled_time_in_order(r.t, o.gamma, p.log2_bw, p.log2_clk, p.log2_clk_sm);

    const bool ok = in_range && o.status == HBT_ST_OK;
    double v = ok ? o.t : 0.0;
    if (a.out_bad != nullptr) {
      const unsigned long long bad = __ballot(in_range && o.status != HBT_ST_OK);
      if (lane == 0 && bad != 0) atomicAdd(a.out_bad + d, (int32_t)__popcll(bad));
    }
    if (ORDERED) {
      if (in_range) a.work[(int64_t)d * a.n + i] = v;
      continue;
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const double other = __shfl_up(v, off);
      const int32_t other_run = __shfl_up(run, off);
      if (lane >= off && other_run == run) v += other;
    }
    if (adds) unsafeAtomicAdd(a.out_sum + (int64_t)d * a.n_segments + seg, v);
  }
}

struct OrderedSumArgs {
  int64_t n;
  int32_t n_segments;
  const double* work;            // [n_dest][n], from wave_scale_sum_kernel<., true>
  const int64_t* segment_start;  // [n_segments + 1]
  double* out_sum;               // [n_dest][n_segments]
};

// One thread per (segment, destination = blockIdx.y): it adds the segment's
// scaled times one after the other in the records' order, as the reference
// adds a pass's kernels (run_time.py:50-58).  No floating-point atomics: the
// sum is the same every time, and the same as a sequential sum of the
// per-record kernel's times.  (The loads do not depend on the running sum, so
// they run ahead of the additions.)
__global__ __launch_bounds__(kBlock) void segment_sum_ordered_kernel(const OrderedSumArgs a) {
  const int s = blockIdx.x * kBlock + threadIdx.x;
  if (s >= a.n_segments) return;
  // (clamped to the columns: a wrong boundary must not become a stray read)
  int64_t begin = a.segment_start[s], end = a.segment_start[s + 1];
  begin = begin < 0 ? 0 : begin;
  end = end > a.n ? a.n : end;
  const double* v = a.work + (int64_t)blockIdx.y * a.n;
  double sum = 0.0;
#pragma unroll 8
  for (int64_t j = begin; j < end; ++j) sum += v[j];
  a.out_sum[(int64_t)blockIdx.y * a.n_segments + s] = sum;
}

struct GammaArgs {
  int64_t n;
  const double* run_time_ns;
  const double* flop_sp_efficiency;
  const double* dram_read_bytes;
  const double* dram_write_bytes;
  double* out_gamma;
  double peak_gflops;   // origin
  DestArgs dest;
};

// gamma alone (roofline.py:68-104), one thread per record; NaN where the
// reference's assertion 0 <= gamma <= 1 fails.
__global__ __launch_bounds__(kBlock) void roofline_gamma_kernel(const GammaArgs a) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= a.n) return;
  const double t = a.run_time_ns[i], eff = a.flop_sp_efficiency[i];
  const double total_gb = (a.dram_read_bytes[i] + a.dram_write_bytes[i]) * 0x1p-30;
  const double scaled = div_const<C100>(eff) * a.peak_gflops * t;
  double num_gflops = div_const<C1e9>(scaled);
  if (!(div_const_safe(eff) && div_const_safe(scaled)))
    num_gflops = origin_gflops_exact(a.peak_gflops, eff, t);
  const double gamma = roofline_gamma(a.dest, num_gflops, total_gb, true);
  a.out_gamma[i] = (gamma >= 0 && gamma <= 1) ? gamma : __builtin_nan("");
}

struct RatioArgs {
  const float* pred;          // [(n_dest + 1)][n_rows]; the last row is the origin
  const double* run_time_ms;  // [n_ops]
  const int32_t* op_row;      // [n_ops], nullable: operation o reads column o
  int32_t n_dest, n_rows, n_ops;
  double* out_ms;             // [n_dest][n_ops], nullable
  double* out_total;          // [n_dest], nullable; added to
  int32_t* out_clamped;       // [n_dest], nullable; added to
};

// blockIdx.x = destination; the block's threads stride over the operations.
// Operations with equal features share one column of pred.
__global__ __launch_bounds__(kBlock) void ratio_scale_kernel(const RatioArgs a) {
  const int d = blockIdx.x;
  const float* dest = a.pred + (int64_t)d * a.n_rows;
  const float* orig = a.pred + (int64_t)a.n_dest * a.n_rows;
  double acc = 0.0;
  int32_t clamped = 0;
  for (int o = threadIdx.x; o < a.n_ops; o += kBlock) {
    const int32_t row = a.op_row != nullptr ? a.op_row[o] : o;
    double ms = __builtin_nan("");
    if (row >= 0 && row < a.n_rows) {
      // predictor.py:182: operation.run_time_ms * pred_dest / pred_orig, in fp64
      ms = a.run_time_ms[o] * (double)dest[row] / (double)orig[row];
      if (ms < 0) {   // predictor.py:135-141: warned about and replaced by 0
        ms = 0.;
        ++clamped;
      }
    }
    if (a.out_ms != nullptr) a.out_ms[(int64_t)d * a.n_ops + o] = ms;
    acc += ms;
  }
  if (a.out_total == nullptr && a.out_clamped == nullptr) return;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    acc += __shfl_down(acc, off);
    clamped += __shfl_down(clamped, off);
  }
  __shared__ double part[kBlock / 64];
  __shared__ int32_t part_clamped[kBlock / 64];
  if ((threadIdx.x & 63) == 0) {
    part[threadIdx.x >> 6] = acc;
    part_clamped[threadIdx.x >> 6] = clamped;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = 0.0;
    int32_t count = 0;
    for (int w = 0; w < kBlock / 64; ++w) {
      total += part[w];
      count += part_clamped[w];
    }
    if (a.out_total != nullptr) a.out_total[d] += total;
    if (a.out_clamped != nullptr) a.out_clamped[d] += count;
  }
}

}  // namespace
}  // namespace hbt

extern "C" {

hbt_device_table* hbt_device_table_create(const hbt_device_spec* origin,
                                          const hbt_device_spec* dests, int32_t n_dest,
                                          int* err) {
  using namespace hbt;
  int dummy;
  if (err == nullptr) err = &dummy;
  *err = HBT_OK;
  if (origin == nullptr || dests == nullptr || n_dest <= 0) {
    *err = HBT_EINVAL;
    return nullptr;
  }
  if (n_dest > 65535) {
    *err = HBT_ESIZE;
    return nullptr;
  }
  int rc = hbt_device_spec_check(origin);
  for (int32_t d = 0; d < n_dest && rc == HBT_OK; ++d) rc = hbt_device_spec_check(&dests[d]);
  if (rc != HBT_OK) {
    *err = rc;
    return nullptr;
  }
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    *err = HBT_EHIP;
    return nullptr;
  }
  hbt_device_table* t = new (std::nothrow) hbt_device_table();
  if (t == nullptr) {
    *err = HBT_ENOMEM;
    return nullptr;
  }
  t->n_dest = n_dest;
  t->device = device;
  t->origin = make_origin_args(*origin);
  std::vector<DestArgs> host((size_t)n_dest);
  for (int32_t d = 0; d < n_dest; ++d) {
    host[d] = make_dest_args(*origin, dests[d]);
    // within a group of kSumGroup destinations, one that has the occupancy
    // constants of the one before it shares that one's occupancies
    if (d % kSumGroup != 0 && same_occupancy_constants(host[d - 1].dev, host[d].dev))
      host[d].dev.flags |= kSameOccAsPrev;
  }
  t->model = dev::model_for(t->origin.dev, host.data(), n_dest);
  t->dests = nullptr;
  const size_t bytes = sizeof(DestArgs) * (size_t)n_dest;
  if (hipMalloc(reinterpret_cast<void**>(&t->dests), bytes) != hipSuccess) {
    (void)hipGetLastError();
    delete t;
    *err = HBT_ENOMEM;
    return nullptr;
  }
  if (hipMemcpy(t->dests, host.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(t->dests);
    delete t;
    *err = HBT_EHIP;
    return nullptr;
  }
  return t;
}

void hbt_device_table_destroy(hbt_device_table* table) {
  if (table == nullptr) return;
  if (table->dests != nullptr) (void)hipFree(table->dests);
  delete table;
}

int32_t hbt_device_table_size(const hbt_device_table* table) {
  return table != nullptr ? table->n_dest : 0;
}

int hbt_wave_scale_sum(const hbt_device_table* table, int64_t n, const int32_t* num_blocks,
                       const int32_t* block_size, const int32_t* dynamic_smem,
                       const int32_t* static_smem, const int32_t* regs, const int32_t* dest_regs,
                       const double* run_time_ns, const double* flop_sp_efficiency,
                       const double* dram_read_bytes, const double* dram_write_bytes,
                       const uint8_t* has_metrics, const int32_t* segment, int32_t n_segments,
                       double* out_sum, int32_t* out_bad, void* hip_stream) {
  using namespace hbt;
  if (table == nullptr || n < 0 || n_segments <= 0 || out_sum == nullptr) return HBT_EINVAL;
  if (n > 0 && (!num_blocks || !block_size || !dynamic_smem || !static_smem || !regs ||
                !run_time_ns || !flop_sp_efficiency || !dram_read_bytes || !dram_write_bytes))
    return HBT_EINVAL;
  const int64_t blocks = (n + kBlock - 1) / kBlock;
  // (the clearing launch covers n_dest * n_segments sums with 256 threads per block)
  if (blocks > 0x7fffffff || (int64_t)n_segments * table->n_dest > ((int64_t)1 << 38))
    return HBT_ESIZE;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (device != table->device) return HBT_EINVAL;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);

  const int64_t n_sums = (int64_t)table->n_dest * n_segments;
  const int64_t fill = n_sums > table->n_dest ? n_sums : table->n_dest;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((fill + kBlock - 1) / kBlock)), dim3(kBlock),
                     0, stream, out_sum, n_sums, out_bad, table->n_dest);
  if (hipGetLastError() != hipSuccess) return HBT_EHIP;
  if (n == 0) return HBT_OK;

  SumArgs a{};
  a.n = n;
  a.n_segments = n_segments;
  a.n_dest = table->n_dest;
  a.num_blocks = num_blocks; a.block_size = block_size; a.dynamic_smem = dynamic_smem;
  a.static_smem = static_smem; a.regs = regs; a.dest_regs = dest_regs;
  a.run_time_ns = run_time_ns; a.flop_sp_efficiency = flop_sp_efficiency;
  a.dram_read_bytes = dram_read_bytes; a.dram_write_bytes = dram_write_bytes;
  a.has_metrics = has_metrics; a.segment = segment;
  a.out_sum = out_sum; a.out_bad = out_bad;
  a.dests = table->dests;
  a.origin = table->origin;
  const dim3 grid((unsigned)blocks, (unsigned)((table->n_dest + kSumGroup - 1) / kSumGroup));
  dev::with_model(table->model, [&](auto m) {
    hipLaunchKernelGGL((wave_scale_sum_kernel<decltype(m)::value, false>), grid, dim3(kBlock), 0,
                       stream, a);
  });
  return hipGetLastError() == hipSuccess ? HBT_OK : HBT_EHIP;
}

int hbt_wave_scale_sum_ordered(const hbt_device_table* table, int64_t n, const int32_t* num_blocks,
                               const int32_t* block_size, const int32_t* dynamic_smem,
                               const int32_t* static_smem, const int32_t* regs,
                               const int32_t* dest_regs, const double* run_time_ns,
                               const double* flop_sp_efficiency, const double* dram_read_bytes,
                               const double* dram_write_bytes, const uint8_t* has_metrics,
                               const int64_t* segment_start, int32_t n_segments, double* workspace,
                               double* out_sum, int32_t* out_bad, void* hip_stream) {
  using namespace hbt;
  if (table == nullptr || n < 0 || n_segments <= 0 || out_sum == nullptr ||
      segment_start == nullptr)
    return HBT_EINVAL;
  if (n > 0 && (!num_blocks || !block_size || !dynamic_smem || !static_smem || !regs ||
                !run_time_ns || !flop_sp_efficiency || !dram_read_bytes || !dram_write_bytes ||
                !workspace))
    return HBT_EINVAL;
  const int64_t blocks = (n + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffff || (int64_t)n_segments * table->n_dest > ((int64_t)1 << 38))
    return HBT_ESIZE;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (device != table->device) return HBT_EINVAL;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  if (out_bad != nullptr) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((table->n_dest + kBlock - 1) / kBlock)),
                       dim3(kBlock), 0, stream, static_cast<double*>(nullptr), (int64_t)0, out_bad,
                       table->n_dest);
    if (hipGetLastError() != hipSuccess) return HBT_EHIP;
  }
  if (n > 0) {
    SumArgs a{};
    a.n = n;
    a.n_segments = n_segments;
    a.n_dest = table->n_dest;
    a.num_blocks = num_blocks; a.block_size = block_size; a.dynamic_smem = dynamic_smem;
    a.static_smem = static_smem; a.regs = regs; a.dest_regs = dest_regs;
    a.run_time_ns = run_time_ns; a.flop_sp_efficiency = flop_sp_efficiency;
    a.dram_read_bytes = dram_read_bytes; a.dram_write_bytes = dram_write_bytes;
    a.has_metrics = has_metrics;
    a.out_bad = out_bad;
    a.work = workspace;
    a.dests = table->dests;
    a.origin = table->origin;
    const dim3 grid((unsigned)blocks, (unsigned)((table->n_dest + kSumGroup - 1) / kSumGroup));
    dev::with_model(table->model, [&](auto m) {
      hipLaunchKernelGGL((wave_scale_sum_kernel<decltype(m)::value, true>), grid, dim3(kBlock), 0,
                         stream, a);
    });
    if (hipGetLastError() != hipSuccess) return HBT_EHIP;
  }
  OrderedSumArgs b{};
  b.n = n;
  b.n_segments = n_segments;
  b.work = workspace;
  b.segment_start = segment_start;
  b.out_sum = out_sum;
  hipLaunchKernelGGL(segment_sum_ordered_kernel,
                     dim3((unsigned)((n_segments + kBlock - 1) / kBlock), (unsigned)table->n_dest),
                     dim3(kBlock), 0, stream, b);
  return hipGetLastError() == hipSuccess ? HBT_OK : HBT_EHIP;
}

int hbt_roofline_gamma(const hbt_device_spec* origin, const hbt_device_spec* dest, int64_t n,
                       const double* run_time_ns, const double* flop_sp_efficiency,
                       const double* dram_read_bytes, const double* dram_write_bytes,
                       double* out_gamma, void* hip_stream) {
  using namespace hbt;
  if (origin == nullptr || dest == nullptr || n < 0) return HBT_EINVAL;
  int rc = hbt_device_spec_check(origin);
  if (rc == HBT_OK) rc = hbt_device_spec_check(dest);
  if (rc != HBT_OK) return rc;
  if (n == 0) return HBT_OK;
  if (!run_time_ns || !flop_sp_efficiency || !dram_read_bytes || !dram_write_bytes || !out_gamma)
    return HBT_EINVAL;
  const void* cols[] = {run_time_ns, flop_sp_efficiency, dram_read_bytes, dram_write_bytes,
                        out_gamma};
  for (const void* p : cols)
    if (reinterpret_cast<uintptr_t>(p) % 8 != 0) return HBT_EALIGN;
  const int64_t blocks = (n + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffff) return HBT_ESIZE;
  if (hbt_device_count() <= 0) return HBT_EHIP;
  GammaArgs a{};
  a.n = n;
  a.run_time_ns = run_time_ns; a.flop_sp_efficiency = flop_sp_efficiency;
  a.dram_read_bytes = dram_read_bytes; a.dram_write_bytes = dram_write_bytes;
  a.out_gamma = out_gamma;
  a.peak_gflops = origin->peak_gflops;
  a.dest = make_dest_args(*origin, *dest);
  hipLaunchKernelGGL(roofline_gamma_kernel, dim3((unsigned)blocks), dim3(kBlock), 0,
                     static_cast<hipStream_t>(hip_stream), a);
  return hipGetLastError() == hipSuccess ? HBT_OK : HBT_EHIP;
}

int hbt_ratio_scale(const float* pred, int32_t n_dest, int32_t n_rows, const int32_t* op_row,
                    int32_t n_ops, const double* run_time_ms, double* out_ms, double* out_total,
                    int32_t* out_clamped, void* hip_stream) {
  using namespace hbt;
  if (n_dest < 0 || n_ops < 0 || n_rows < 0) return HBT_EINVAL;
  if (op_row == nullptr && n_rows != n_ops) return HBT_EINVAL;
  if (n_dest == 0 || n_ops == 0) return HBT_OK;
  if (pred == nullptr || run_time_ms == nullptr ||
      (out_ms == nullptr && out_total == nullptr && out_clamped == nullptr))
    return HBT_EINVAL;
  if (n_rows == 0) return HBT_EINVAL;
  RatioArgs a{pred, run_time_ms, op_row, n_dest, n_rows, n_ops, out_ms, out_total, out_clamped};
  hipLaunchKernelGGL(ratio_scale_kernel, dim3((unsigned)n_dest), dim3(kBlock), 0,
                     static_cast<hipStream_t>(hip_stream), a);
  return hipGetLastError() == hipSuccess ? HBT_OK : HBT_EHIP;
}

}  // extern "C"
