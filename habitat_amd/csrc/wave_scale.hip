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
// kVectorRecords consecutive records (one; the code is written for any
// number), so a wavefront reads 256 contiguous bytes of every int32
// column and 512 of every fp64 column; stores likewise.  All loads of a
// thread are issued before any arithmetic and all stores after it, so that no
// wait for a load also waits for a store.  Device constants travel in the
// kernel-argument segment and live in SGPRs.  The algorithmic traffic is 52 B
// read + 16 B written per record (5 x i32 + 4 x f64 in; f64 time + 2 x i32
// occupancy out); optional columns add to that.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include "occupancy.h"
#include "wave_scale.h"

// Keep a*b+c as two roundings where the reference (CPython floats) has two.
#pragma clang fp contract(off)

#include "wave_scale_device.h"

namespace hbt {

namespace {

using namespace dev;

constexpr int kRecPerThread = kVectorRecords;
// Two wavefronts per workgroup: fresh short waves taking consecutive 128-record
// chunks keep the chip on one contiguous window of every column.
constexpr int kBlock = 128;

// N consecutive elements as one register group (a scalar when N is 1).
template <class T, int N>
struct VecOf { using type = T __attribute__((ext_vector_type(N))); };
template <class T>
struct VecOf<T, 1> { using type = T; };

template <class T, int N>
__device__ __forceinline__ T vec_get(const typename VecOf<T, N>::type& v, int k) {
  if constexpr (N == 1) return v;
  else return v[k];
}

template <class T, int N>
__device__ __forceinline__ void vec_set(typename VecOf<T, N>::type& v, int k, T x) {
  if constexpr (N == 1) v = x;
  else v[k] = x;
}

// R consecutive elements starting at element i, all in range: one vector
// access.  Index is uint32_t when every byte offset of the launch fits 32 bits
// (the address is then a uniform 64-bit base plus a 32-bit lane offset, which
// costs no 64-bit vector arithmetic), else uint64_t.
//
// Every column is read once and every output written once, so both directions
// carry the non-temporal hint: the lines are not kept in L2 or the last-level
// cache at the expense of each other.
template <class T, int R, class Index>
__device__ __forceinline__ void load_r(const T* __restrict__ p, Index i, T (&out)[R]) {
  using V = typename VecOf<T, R>::type;
  const Index byte = i * (Index)sizeof(T);
  const V v = __builtin_nontemporal_load(
      reinterpret_cast<const V*>(reinterpret_cast<const char*>(p) + (size_t)byte));
#pragma unroll
  for (int k = 0; k < R; ++k) out[k] = vec_get<T, R>(v, k);
}

template <class T, int R, class Index>
__device__ __forceinline__ void store_r(T* __restrict__ p, Index i, const T (&in)[R]) {
  using V = typename VecOf<T, R>::type;
  V v;
#pragma unroll
  for (int k = 0; k < R; ++k) vec_set<T, R>(v, k, in[k]);
  const Index byte = i * (Index)sizeof(T);
  __builtin_nontemporal_store(v, reinterpret_cast<V*>(reinterpret_cast<char*>(p) + (size_t)byte));
}

// An optional output column (null = the caller does not want it).
template <class T, int R, class Index>
__device__ __forceinline__ void store_out(T* __restrict__ p, Index i, const T (&in)[R]) {
  if (p != nullptr) store_r<T, R>(p, i, in);
}

// Records i .. i+R-1 (all below n) for every destination of the launch.
// SINGLE: the launch has one destination; its constants then sit at fixed
// offsets of the argument segment and are fetched once, up front, instead of
// inside a loop over destinations.
template <int R, int MODEL, bool PERMUTE, bool SINGLE, class Index>
__device__ __forceinline__ void process(const WaveScaleArgs& a, Index i) {
  const double log2_lane = PERMUTE ? kLog2Int[threadIdx.x & 63] : 0.0;
  int32_t nb[R], block[R], dyn[R], stat[R], regs[R], dregs[R];
  double t[R], eff[R], rd[R], wr[R];
  load_r<int32_t, R>(a.num_blocks, i, nb);
  load_r<int32_t, R>(a.block_size, i, block);
  load_r<int32_t, R>(a.dynamic_smem, i, dyn);
  load_r<int32_t, R>(a.static_smem, i, stat);
  load_r<int32_t, R>(a.regs, i, regs);
  load_r<double, R>(a.run_time_ns, i, t);
  load_r<double, R>(a.flop_sp_efficiency, i, eff);
  load_r<double, R>(a.dram_read_bytes, i, rd);
  load_r<double, R>(a.dram_write_bytes, i, wr);
  if (a.dest_regs != nullptr) {
    load_r<int32_t, R>(a.dest_regs, i, dregs);
  } else {
#pragma unroll
    for (int k = 0; k < R; ++k) dregs[k] = -1;
  }
  // The metrics flags stay packed in one register until the destination part
  // needs them (see below), so that nothing waits for this load, the last one
  // issued, before the arithmetic on the other columns starts.
  uint32_t hm_bits = 0x01010101u;
  if (a.has_metrics != nullptr) {
    uint8_t v[R];
    load_r<uint8_t, R>(a.has_metrics, i, v);
    hm_bits = 0;
#pragma unroll
    for (int k = 0; k < R; ++k) hm_bits |= (uint32_t)v[k] << (8 * k);
  }

  RecordIn rin[R];
  RecordMid mid[R];
#pragma unroll
  for (int k = 0; k < R; ++k) {
    rin[k] = RecordIn{nb[k], block[k], smem_sum(stat[k], dyn[k]), regs[k], dregs[k],
                      true, t[k], eff[k], rd[k], wr[k]};
    mid[k] = origin_part<MODEL>(a.origin, rin[k]);
  }
  bool redo = false;
#pragma unroll
  for (int k = 0; k < R; ++k) redo = redo || mid[k].redo_gflops;
  if (__builtin_expect(redo, 0)) {
#pragma unroll
    for (int k = 0; k < R; ++k)
      if (mid[k].redo_gflops)
        mid[k].num_gflops = origin_gflops_exact(a.origin.peak_gflops, rin[k].eff, rin[k].t);
  }
  // Opaque to the optimiser: keeps the unpacking of the flags from moving up
  // to the load.
  asm volatile("" : "+v"(hm_bits));
#pragma unroll
  for (int k = 0; k < R; ++k) rin[k].metrics = ((hm_bits >> (8 * k)) & 0xffu) != 0;

  // With several destinations the two divisions of gamma that do not depend on
  // the destination are made once per record (the general instantiation keeps
  // the one-division form, which has no precondition on the ridge point).
  constexpr bool SHARED = !SINGLE && MODEL != kModelGeneral;
  Intensity intensity[R];
#pragma unroll
  for (int k = 0; k < R; ++k) {
    finish_mid<PERMUTE>(mid[k], log2_lane);
    if (SHARED) intensity[k] = record_intensity(mid[k].num_gflops, mid[k].total_gb);
  }

  const int n_dest = SINGLE ? 1 : a.n_dest;
  int32_t occ_d[R];
  for (int d = 0; d < n_dest; ++d) {
    const DestArgs& p = a.dest[d];
    double ot[R], gamma[R];
    int32_t wave_d[R];
    uint8_t st[R];
    bool in_order = false;
    // the destination's occupancy, unless it has the constants of the one before
    if (SINGLE || !(p.dev.flags & kSameOccAsPrev)) {
#pragma unroll
      for (int k = 0; k < R; ++k) occ_d[k] = dest_occupancy<MODEL>(p, rin[k], mid[k]);
    }
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const double g =
          SHARED ? roofline_gamma_shared(p, mid[k].num_gflops, mid[k].total_gb, intensity[k],
                                         rin[k].metrics)
                 : roofline_gamma(p, mid[k].num_gflops, mid[k].total_gb, rin[k].metrics);
      const RecordOut o = dest_scale<MODEL, PERMUTE>(p, rin[k], mid[k], occ_d[k], g, log2_lane);
      ot[k] = o.t; wave_d[k] = o.wave_d; st[k] = o.status;
      gamma[k] = o.in_order ? o.gamma : __builtin_nan("");
      in_order = in_order || o.in_order;
    }
    const DestOut& w = a.out[d];
    store_r<double, R>(w.time_ns, i, ot);
    store_out<int32_t, R>(w.occ, i, occ_d);
    store_out<int32_t, R>(w.wave, i, wave_d);
    store_out<uint8_t, R>(w.status, i, st);
    // Run times beyond 2^+-500 ns (see dest_scale): the time is formed again in
    // the reference's order of operations and stored over the first one, after
    // everything else, where the rare call costs the other records nothing.
    if (__builtin_expect(in_order, 0)) {
#pragma unroll
      for (int k = 0; k < R; ++k)
        if (gamma[k] == gamma[k])
          ot[k] = scaled_time_in_order(rin[k].t, gamma[k], p.log2_bw, p.log2_clk, p.log2_clk_sm);
      store_r<double, R>(w.time_ns, i, ot);
    }
  }

  // Origin columns last: a store issued between the loads and the arithmetic
  // that consumes them would have to be waited for together with the loads
  // (one counter tracks both).
  if (a.write_origin) {
    int32_t occ_o[R], wave_o[R];
#pragma unroll
    for (int k = 0; k < R; ++k) { occ_o[k] = mid[k].occ_o; wave_o[k] = mid[k].wave_o; }
    store_out<int32_t, R>(a.out_occ_origin, i, occ_o);
    store_out<int32_t, R>(a.out_wave_origin, i, wave_o);
  }
}

template <int R, int MODEL, bool SINGLE, class Index>
__global__ __launch_bounds__(kBlock) void wave_scale_kernel(const WaveScaleArgs a) {
  const Index thread = (Index)blockIdx.x * kBlock + threadIdx.x;
  const Index i = thread * R;
  const Index n = (Index)a.n;
  // A wavefront whose 64 * R records are all in range takes the vector path
  // with every lane active; the last, partial wavefront of the batch goes one
  // record at a time.
  const Index wave_end = ((thread | 63) + 1) * R;
  if (wave_end <= n) {
    process<R, MODEL, true, SINGLE, Index>(a, i);
  } else {
    const Index end = (i + R < n) ? i + R : n;
    for (Index j = i; j < end; ++j) process<1, MODEL, false, SINGLE, Index>(a, j);
  }
}

template <int R, int MODEL, class Index>
void launch(const WaveScaleArgs& args, hipStream_t stream) {
  const int64_t threads = (args.n + R - 1) / R;
  const int64_t blocks = (threads + kBlock - 1) / kBlock;
  if (args.n_dest == 1)
    hipLaunchKernelGGL((wave_scale_kernel<R, MODEL, true, Index>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, stream, args);
  else
    hipLaunchKernelGGL((wave_scale_kernel<R, MODEL, false, Index>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, stream, args);
}

template <int R, int MODEL>
void launch(const WaveScaleArgs& args, hipStream_t stream) {
  // 32-bit byte offsets when the widest column (8 bytes per record) and the
  // thread numbering stay below 2^32 with room for the last wavefront.
  if (args.n < ((int64_t)1 << 28)) launch<R, MODEL, uint32_t>(args, stream);
  else launch<R, MODEL, uint64_t>(args, stream);
}

}  // namespace

hipError_t launch_wave_scale(const WaveScaleArgs& args, bool vectorised, hipStream_t stream) {
  if (args.n <= 0) return hipSuccess;
  const int model = model_for(args.origin.dev, args.dest, args.n_dest);
  const bool vec = vectorised && kRecPerThread > 1;
  with_model(model, [&](auto m) {
    if (vec) launch<kRecPerThread, decltype(m)::value>(args, stream);
    else launch<1, decltype(m)::value>(args, stream);
  });
  return hipGetLastError();
}

}  // namespace hbt
