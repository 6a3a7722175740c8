// Wave scaling of kernel records on gfx950: one fused, HBM-bound kernel.
//
// Per record and destination device it evaluates what the reference evaluates
// with a Python call chain per kernel (analyzer/habitat/analysis/predictor.py:116-124
// -> wave_scaling/unified.py:8-35 -> roofline.py:8-108 | resimplified.py:7-40 ->
// common.py:3-20 -> two occupancy calls into cpp/src/cuda/kernel.cpp:29-56):
// both occupancies, both wave sizes, the roofline gamma, the small-kernel test
// and the scaled time.
//
// Data layout: structure of arrays, one column per record field.  A thread owns
// four consecutive records, so every int32 column is one 16-byte load per lane
// (1 KiB per wavefront) and every fp64 column two; stores likewise.  Device
// constants travel in the kernel-argument segment and live in SGPRs.  The
// algorithmic traffic is 52 B read + 16 B written per record (5 x i32 + 4 x f64
// in; f64 time + 2 x i32 occupancy out); optional columns add to that.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include "occupancy.h"
#include "wave_scale.h"

// Keep a*b+c as two roundings where the reference (CPython floats) has two.
#pragma clang fp contract(off)

namespace hbt {

namespace {

constexpr int kRecPerThread = 4;
constexpr int kBlock = 256;

struct RecordIn {
  int32_t nb, block, smem_total, regs, dest_regs;
  bool metrics;
  double t, eff, rd, wr;
};

// Destination-independent part of one record.
struct RecordMid {
  int32_t occ_o, wave_o;
  bool small_o;       // num_blocks // origin_wave == 0
  bool fast;          // operands small enough for the float-reciprocal division
  double num_gflops, total_gb, intensity;
  double origin_max_occ;  // ceil(num_blocks / origin.num_sms)
};

__device__ __forceinline__ int32_t occupancy_dev(const OccDevice& d, bool fast, int32_t block,
                                                 int32_t smem_total, int32_t regs) {
  regs &= 0xFFFF;  // uint16_t narrowing, cpp/src/cuda/kernel.h:108
  if (fast && d.fast_ok && (int64_t)regs * d.warp_size + 255 < (1 << 22))
    return occupancy_core<FastDiv>(d, block, smem_total, regs);
  return occupancy_core<ExactDiv>(d, block, smem_total, regs);
}

__device__ __forceinline__ RecordMid origin_part(const WaveScaleArgs& a, const RecordIn& r) {
  RecordMid m;
  m.fast = r.block < (1 << 22) && r.smem_total >= 0 && r.smem_total < (1 << 22);
  m.occ_o = occupancy_dev(a.origin, m.fast, r.block, r.smem_total, r.regs);
  m.wave_o = a.origin.num_sms * m.occ_o;
  m.small_o = r.nb >= 0 && r.nb < m.wave_o;
  // roofline.py:72-76, same operation order
  m.total_gb = (r.rd + r.wr) / 1024 / 1024 / 1024;
  const double gflops_per_second = r.eff / 100 * a.origin_peak_gflops;
  m.num_gflops = gflops_per_second * r.t / 1e9;
  m.intensity = m.num_gflops / m.total_gb;
  m.origin_max_occ = ceil((double)r.nb / a.origin_sms);
  return m;
}

struct RecordOut {
  double t;
  int32_t occ_d, wave_d;
  uint8_t status;
};

__device__ __forceinline__ RecordOut dest_part(const DestArgs& p, const RecordIn& r,
                                               const RecordMid& m) {
  RecordOut o;
  const int32_t regs_d = r.dest_regs >= 0 ? r.dest_regs : r.regs;
  o.occ_d = occupancy_dev(p.dev, m.fast, r.block, r.smem_total, regs_d);
  o.wave_d = p.dev.num_sms * o.occ_d;
  o.t = __builtin_nan("");

  double gamma = 1.0;
  if (r.metrics) {
    // roofline.py:86-101
    if (m.num_gflops < 1e-9) gamma = 1.;
    else if (m.total_gb == 0) gamma = 0.;
    else if (m.intensity > p.ridge) gamma = p.half_ridge / m.intensity;
    else gamma = p.neg_half_over_ridge * m.intensity + 1.;
    if (!(gamma >= 0 && gamma <= 1)) { o.status = HBT_ST_BAD_GAMMA; return o; }
  }
  if (m.wave_o == 0) { o.status = HBT_ST_ORIGIN_WAVE_ZERO; return o; }
  bool small = m.small_o;
  if (small) {
    if (o.wave_d == 0) { o.status = HBT_ST_DEST_WAVE_ZERO; return o; }
    small = r.nb < o.wave_d;
  }
  o.status = HBT_ST_OK;

  if (!r.metrics) {  // resimplified.py:25-40
    o.t = small ? r.t : r.t * p.bw_ratio;
    return o;
  }
  const double gamma_compl = 1.0 - gamma;
  if (small) {       // roofline.py:32-45
    if (m.origin_max_occ == 0) { o.status = HBT_ST_ZERO_BLOCKS; return o; }
    const double dest_max_occ = ceil((double)r.nb / p.sms);
    const double factor = p.clk_ratio * (dest_max_occ / m.origin_max_occ);
    o.t = r.t * exp2(gamma_compl * log2(factor));
    return o;
  }
  // roofline.py:48-64: t * bw^gamma * clk^(1-gamma) * sm^(1-gamma), with the
  // three logarithms taken once on the host.
  o.t = r.t * exp2(gamma * p.log2_bw + gamma_compl * p.log2_clk_sm);
  return o;
}

template <class T, int N>
struct alignas(sizeof(T) * N) Pack { T v[N]; };

// Load R consecutive elements starting at i (vectorised when all are in range).
template <class T, int R>
__device__ __forceinline__ void load_r(const T* __restrict__ p, int64_t i, int64_t n, T fill,
                                       T (&out)[R]) {
  if (R > 1 && i + R <= n) {
    const Pack<T, R> v = *reinterpret_cast<const Pack<T, R>*>(p + i);
#pragma unroll
    for (int k = 0; k < R; ++k) out[k] = v.v[k];
  } else {
#pragma unroll
    for (int k = 0; k < R; ++k) out[k] = (i + k < n) ? p[i + k] : fill;
  }
}

template <class T, int R>
__device__ __forceinline__ void store_r(T* __restrict__ p, int64_t i, int64_t n, const T (&in)[R]) {
  if (R > 1 && i + R <= n) {
    Pack<T, R> v;
#pragma unroll
    for (int k = 0; k < R; ++k) v.v[k] = in[k];
    *reinterpret_cast<Pack<T, R>*>(p + i) = v;
  } else {
#pragma unroll
    for (int k = 0; k < R; ++k)
      if (i + k < n) p[i + k] = in[k];
  }
}

template <int R>
__global__ __launch_bounds__(kBlock) void wave_scale_kernel(const WaveScaleArgs a) {
  const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * R;
  if (i >= a.n) return;
  const int64_t n = a.n;

  int32_t nb[R], block[R], dyn[R], stat[R], regs[R], dregs[R];
  uint8_t hm[R];
  double t[R], eff[R], rd[R], wr[R];
  load_r<int32_t, R>(a.num_blocks, i, n, 1, nb);
  load_r<int32_t, R>(a.block_size, i, n, 1, block);
  load_r<int32_t, R>(a.dynamic_smem, i, n, 0, dyn);
  load_r<int32_t, R>(a.static_smem, i, n, 0, stat);
  load_r<int32_t, R>(a.regs, i, n, 0, regs);
  load_r<double, R>(a.run_time_ns, i, n, 0.0, t);
  load_r<double, R>(a.flop_sp_efficiency, i, n, 0.0, eff);
  load_r<double, R>(a.dram_read_bytes, i, n, 0.0, rd);
  load_r<double, R>(a.dram_write_bytes, i, n, 0.0, wr);
  if (a.dest_regs != nullptr) {
    load_r<int32_t, R>(a.dest_regs, i, n, -1, dregs);
  } else {
#pragma unroll
    for (int k = 0; k < R; ++k) dregs[k] = -1;
  }
  if (a.has_metrics != nullptr) {
    load_r<uint8_t, R>(a.has_metrics, i, n, 1, hm);
  } else {
#pragma unroll
    for (int k = 0; k < R; ++k) hm[k] = 1;
  }

  RecordIn rin[R];
  RecordMid mid[R];
#pragma unroll
  for (int k = 0; k < R; ++k) {
    rin[k] = RecordIn{nb[k], block[k], smem_sum(stat[k], dyn[k]), regs[k], dregs[k],
                      hm[k] != 0, t[k], eff[k], rd[k], wr[k]};
    mid[k] = origin_part(a, rin[k]);
  }

  if (a.write_origin) {
    int32_t occ_o[R], wave_o[R];
#pragma unroll
    for (int k = 0; k < R; ++k) { occ_o[k] = mid[k].occ_o; wave_o[k] = mid[k].wave_o; }
    if (a.out_occ_origin != nullptr) store_r<int32_t, R>(a.out_occ_origin, i, n, occ_o);
    if (a.out_wave_origin != nullptr) store_r<int32_t, R>(a.out_wave_origin, i, n, wave_o);
  }

  for (int d = 0; d < a.n_dest; ++d) {
    const DestArgs& p = a.dest[d];
    const int64_t row = (int64_t)d * n;
    double ot[R];
    int32_t occ_d[R], wave_d[R];
    uint8_t st[R];
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const RecordOut o = dest_part(p, rin[k], mid[k]);
      ot[k] = o.t; occ_d[k] = o.occ_d; wave_d[k] = o.wave_d; st[k] = o.status;
    }
    store_r<double, R>(a.out_time_ns + row, i, n, ot);
    if (a.out_occ_dest != nullptr) store_r<int32_t, R>(a.out_occ_dest + row, i, n, occ_d);
    if (a.out_wave_dest != nullptr) store_r<int32_t, R>(a.out_wave_dest + row, i, n, wave_d);
    if (a.out_status != nullptr) store_r<uint8_t, R>(a.out_status + row, i, n, st);
  }
}

}  // namespace

hipError_t launch_wave_scale(const WaveScaleArgs& args, bool vectorised, hipStream_t stream) {
  if (args.n <= 0) return hipSuccess;
  if (vectorised) {
    const int64_t threads = (args.n + kRecPerThread - 1) / kRecPerThread;
    const int64_t blocks = (threads + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(wave_scale_kernel<kRecPerThread>, dim3((unsigned)blocks), dim3(kBlock), 0,
                       stream, args);
  } else {
    const int64_t blocks = (args.n + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(wave_scale_kernel<1>, dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                       args);
  }
  return hipGetLastError();
}

}  // namespace hbt
