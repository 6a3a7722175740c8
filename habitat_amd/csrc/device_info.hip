// Describing and calibrating the GPU this process runs on.
//
//   hbt_local_device_spec      the fields the reference's `device_info` tool
//                              prints from cudaDeviceProp
//                              (cpp/src/device_info.cpp:16-30), from hipDeviceProp_t
//   hbt_measure_fp32_fma_gflops   the role of the reference's flop_test kernel
//                              (cpp/src/cuda/diagnostics.cu:9-25, driven by
//                              tools/device-metadata/measure_peak_flops.py:10-18):
//                              a kernel of nothing but fp32 FMAs, timed
//   hbt_measure_fp32_mfma_gflops  the same for v_mfma_f32_32x32x2_f32, the
//                              instruction the MLP kernel is bound by
//   hbt_measure_copy_gbps      device-to-device copy bandwidth, the achievable
//                              ceiling under the published HBM peak
//
// These are calibration tools, not part of the prediction path: they allocate
// their own scratch memory, run on the default stream and synchronise.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>

#include "../../include/habitat_mi.h"

namespace hbt {
namespace {

using f32x16 = float __attribute__((ext_vector_type(16)));

// 16 independent accumulators per lane, 2 FLOP per FMA.
__global__ __launch_bounds__(256) void fma_peak_kernel(float* out, int iters, float a, float b) {
  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = (float)(threadIdx.x + i);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = __builtin_fmaf(acc[i], a, b);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// 4 independent 32x32 accumulators per wave, 4096 FLOP per instruction.
__global__ __launch_bounds__(256) void mfma_peak_kernel(float* out, int iters, float a, float b) {
  f32x16 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = (float)(threadIdx.x + t);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[t], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[t][i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

struct StreamArgs {
  const int32_t* ints[5];
  const double* dbls[4];
  double* out_time;
  int32_t* out_occ[2];
  uint8_t* out_status;
  uint32_t n;
};

// The data movement of the wave-scaling kernel and nothing else: the same nine
// input and four output columns, one record per thread, 128-thread workgroups,
// non-temporal accesses; the arithmetic is a few additions so that no load can
// be dropped.
__global__ __launch_bounds__(128) void record_stream_kernel(const StreamArgs a) {
  const uint32_t i = blockIdx.x * 128u + threadIdx.x;
  if (i >= a.n) return;
  int32_t s = 0;
  double d = 0;
#pragma unroll
  for (int k = 0; k < 5; ++k) s += __builtin_nontemporal_load(a.ints[k] + i);
#pragma unroll
  for (int k = 0; k < 4; ++k) d += __builtin_nontemporal_load(a.dbls[k] + i);
  __builtin_nontemporal_store(d, a.out_time + i);
  __builtin_nontemporal_store(s, a.out_occ[0] + i);
  __builtin_nontemporal_store(s + 1, a.out_occ[1] + i);
  __builtin_nontemporal_store((uint8_t)s, a.out_status + i);
}

struct MultiStreamArgs {
  const int32_t* ints[5];
  const double* dbls[4];
  double* out_time;     // [n_dest][n]
  int32_t* out_occ;     // [n_dest][n]
  uint8_t* out_status;  // [n_dest][n]
  int32_t* out_occ_origin;
  uint32_t n;
  int32_t n_dest;
};

// The data movement of a launch with several destinations: the record read
// once, per destination one fp64, one int32 and one byte written to that
// destination's rows, the origin occupancy once.
__global__ __launch_bounds__(128) void record_stream_multi_kernel(const MultiStreamArgs a) {
  const uint32_t i = blockIdx.x * 128u + threadIdx.x;
  if (i >= a.n) return;
  int32_t s = 0;
  double d = 0;
#pragma unroll
  for (int k = 0; k < 5; ++k) s += __builtin_nontemporal_load(a.ints[k] + i);
#pragma unroll
  for (int k = 0; k < 4; ++k) d += __builtin_nontemporal_load(a.dbls[k] + i);
  for (int j = 0; j < a.n_dest; ++j) {
    const size_t at = (size_t)j * a.n + i;
    __builtin_nontemporal_store(d + j, a.out_time + at);
    __builtin_nontemporal_store(s + j, a.out_occ + at);
    __builtin_nontemporal_store((uint8_t)(s + j), a.out_status + at);
  }
  __builtin_nontemporal_store(s, a.out_occ_origin + i);
}

struct Timer {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  bool ok = false;
  Timer() { ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess; }
  ~Timer() {
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  }
};

template <class Launch>
int time_kernel(Launch launch, int blocks, double* ms_out) {
  float* scratch = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&scratch), (size_t)blocks * 256 * sizeof(float)) !=
      hipSuccess) {
    (void)hipGetLastError();
    return HBT_ENOMEM;
  }
  Timer t;
  int rc = HBT_OK;
  float ms = 0.f;
  launch(scratch);  // warm-up
  if (!t.ok || hipDeviceSynchronize() != hipSuccess) rc = HBT_EHIP;
  if (rc == HBT_OK) {
    (void)hipEventRecord(t.e0, nullptr);
    launch(scratch);
    (void)hipEventRecord(t.e1, nullptr);
    if (hipEventSynchronize(t.e1) != hipSuccess ||
        hipEventElapsedTime(&ms, t.e0, t.e1) != hipSuccess)
      rc = HBT_EHIP;
  }
  (void)hipFree(scratch);
  if (rc != HBT_OK) (void)hipGetLastError();
  *ms_out = ms;
  return rc;
}

int cu_count(int* out) {
  int device = 0;
  hipDeviceProp_t p;
  if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&p, device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  *out = p.multiProcessorCount;
  return HBT_OK;
}

}  // namespace
}  // namespace hbt

extern "C" {

int hbt_local_device_spec(int device, hbt_device_spec* out, char* name, size_t name_len) {
  if (out == nullptr) return HBT_EINVAL;
  hipDeviceProp_t p;
  std::memset(&p, 0, sizeof(p));
  if (hipGetDeviceProperties(&p, device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  std::memset(out, 0, sizeof(*out));
  out->compute_major = p.major;
  out->compute_minor = p.minor;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  out->max_threads_per_sm = p.maxThreadsPerMultiProcessor;
  out->regs_per_block = p.regsPerBlock;
  out->regs_per_sm = p.regsPerMultiprocessor;
  out->warp_size = p.warpSize;
  out->num_sms = p.multiProcessorCount;
  out->smem_per_block = (int64_t)p.sharedMemPerBlock;
  out->smem_per_sm = (int64_t)p.maxSharedMemoryPerMultiProcessor;
  out->smem_per_block_optin = (int64_t)p.sharedMemPerBlockOptin;
  // memoryClockRate is in kHz, the bus width in bits.  HBM2/2e (up to gfx90a)
  // moves two bits per pin and reported clock, HBM3/3E (gfx942, gfx950) four:
  // MI300X reports 1300 MHz x 8192 bit for 5.3 TB/s, MI355X 2000 MHz x 8192 bit
  // for 8 TB/s.
  const double bits_per_clock = (p.major == 9 && p.minor >= 4) ? 4.0 : 2.0;
  out->mem_bandwidth_gb =
      bits_per_clock * p.memoryClockRate * 1e3 * (p.memoryBusWidth / 8.0) / 1e9;
  out->base_clock_mhz = p.clockRate / 1e3;
  // vector fp32 as an ordinary kernel reaches it: 64 lanes x one FMA (2 FLOP)
  // per CU and clock.  The published fp32 figure (157.3 TFLOP/s on MI355X) is
  // twice that: it counts packed fp32 or the matrix cores.
  out->peak_gflops = p.multiProcessorCount * (p.clockRate / 1e6) * 128.0;
  if (name != nullptr && name_len > 0) {
    std::strncpy(name, p.name, name_len - 1);
    name[name_len - 1] = '\0';
  }
  return HBT_OK;
}

int hbt_measure_fp32_fma_gflops(int iters, double* out_gflops) {
  using namespace hbt;
  if (iters <= 0 || out_gflops == nullptr) return HBT_EINVAL;
  int cus = 0;
  int rc = cu_count(&cus);
  if (rc != HBT_OK) return rc;
  const int blocks = cus * 8;  // 8 waves per SIMD
  double ms = 0;
  rc = time_kernel([&](float* s) {
    hipLaunchKernelGGL(fma_peak_kernel, dim3(blocks), dim3(256), 0, nullptr, s, iters, 0.999f, 0.5f);
  }, blocks, &ms);
  if (rc != HBT_OK) return rc;
  *out_gflops = (double)blocks * 256 * iters * 16 * 2.0 / (ms * 1e6);
  return HBT_OK;
}

int hbt_measure_fp32_mfma_gflops(int iters, double* out_gflops) {
  using namespace hbt;
  if (iters <= 0 || out_gflops == nullptr) return HBT_EINVAL;
  int cus = 0;
  int rc = cu_count(&cus);
  if (rc != HBT_OK) return rc;
  const int blocks = cus * 2;  // 2 waves per SIMD
  double ms = 0;
  rc = time_kernel([&](float* s) {
    hipLaunchKernelGGL(mfma_peak_kernel, dim3(blocks), dim3(256), 0, nullptr, s, iters, 1.0f, 0.5f);
  }, blocks, &ms);
  if (rc != HBT_OK) return rc;
  *out_gflops = (double)blocks * 4 * iters * 16 * 4096.0 / (ms * 1e6);
  return HBT_OK;
}

int hbt_measure_copy_gbps(size_t bytes, double* out_gbps) {
  using namespace hbt;
  if (bytes == 0 || out_gbps == nullptr) return HBT_EINVAL;
  void *src = nullptr, *dst = nullptr;
  if (hipMalloc(&src, bytes) != hipSuccess || hipMalloc(&dst, bytes) != hipSuccess) {
    (void)hipGetLastError();
    if (src) (void)hipFree(src);
    return HBT_ENOMEM;
  }
  Timer t;
  int rc = t.ok ? HBT_OK : HBT_EHIP;
  float ms = 0.f;
  const int reps = 10;
  if (rc == HBT_OK && (hipMemsetAsync(src, 1, bytes, nullptr) != hipSuccess ||
                       hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, nullptr) != hipSuccess ||
                       hipDeviceSynchronize() != hipSuccess))
    rc = HBT_EHIP;
  if (rc == HBT_OK) {
    (void)hipEventRecord(t.e0, nullptr);
    for (int i = 0; i < reps; ++i)
      (void)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, nullptr);
    (void)hipEventRecord(t.e1, nullptr);
    if (hipEventSynchronize(t.e1) != hipSuccess ||
        hipEventElapsedTime(&ms, t.e0, t.e1) != hipSuccess)
      rc = HBT_EHIP;
  }
  (void)hipFree(src);
  (void)hipFree(dst);
  if (rc != HBT_OK) {
    (void)hipGetLastError();
    return rc;
  }
  *out_gbps = 2.0 * (double)bytes * reps / (ms * 1e6);  // read + write
  return HBT_OK;
}

int hbt_measure_record_stream_gbps(int64_t n, int warmup, int launches, double* out_gbps) {
  using namespace hbt;
  if (n < 2 || n > ((int64_t)1 << 30) || warmup < 0 || launches <= 0 || out_gbps == nullptr)
    return HBT_EINVAL;
  // one allocation: 5 int32 + 4 fp64 input columns, fp64 + 2 int32 + 1 byte output columns
  const size_t col4 = ((size_t)n * 4 + 255) & ~(size_t)255, col8 = ((size_t)n * 8 + 255) & ~(size_t)255;
  const size_t total = 7 * col4 + 5 * col8 + (size_t)n;
  char* base = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&base), total) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_ENOMEM;
  }
  StreamArgs a{};
  char* p = base;
  for (int k = 0; k < 5; ++k) { a.ints[k] = reinterpret_cast<const int32_t*>(p); p += col4; }
  for (int k = 0; k < 4; ++k) { a.dbls[k] = reinterpret_cast<const double*>(p); p += col8; }
  a.out_time = reinterpret_cast<double*>(p); p += col8;
  a.out_occ[0] = reinterpret_cast<int32_t*>(p); p += col4;
  a.out_occ[1] = reinterpret_cast<int32_t*>(p); p += col4;
  a.out_status = reinterpret_cast<uint8_t*>(p);
  a.n = (uint32_t)n;
  const unsigned blocks = (unsigned)((n + 127) / 128);
  Timer t;
  int rc = t.ok ? HBT_OK : HBT_EHIP;
  float ms = 0.f;
  if (rc == HBT_OK && hipMemsetAsync(base, 0, total, nullptr) != hipSuccess) rc = HBT_EHIP;
  if (rc == HBT_OK) {
    for (int i = 0; i < warmup; ++i)
      hipLaunchKernelGGL(record_stream_kernel, dim3(blocks), dim3(128), 0, nullptr, a);
    (void)hipEventRecord(t.e0, nullptr);
    for (int i = 0; i < launches; ++i)
      hipLaunchKernelGGL(record_stream_kernel, dim3(blocks), dim3(128), 0, nullptr, a);
    (void)hipEventRecord(t.e1, nullptr);
    if (hipEventSynchronize(t.e1) != hipSuccess ||
        hipEventElapsedTime(&ms, t.e0, t.e1) != hipSuccess || hipGetLastError() != hipSuccess)
      rc = HBT_EHIP;
  }
  (void)hipFree(base);
  if (rc != HBT_OK) {
    (void)hipGetLastError();
    return rc;
  }
  *out_gbps = 68.0 * (double)n * launches / (ms * 1e6);  // the kernel's algorithmic bytes
  return HBT_OK;
}

int hbt_measure_record_stream_multi_gbps(int64_t n, int32_t n_dest, int warmup, int launches,
                                         double* out_gbps) {
  using namespace hbt;
  if (n < 2 || n > ((int64_t)1 << 28) || n_dest < 1 || n_dest > 64 || warmup < 0 ||
      launches <= 0 || out_gbps == nullptr)
    return HBT_EINVAL;
  const size_t col4 = ((size_t)n * 4 + 255) & ~(size_t)255, col8 = ((size_t)n * 8 + 255) & ~(size_t)255;
  const size_t rows8 = ((size_t)n * 8 * n_dest + 255) & ~(size_t)255;
  const size_t rows4 = ((size_t)n * 4 * n_dest + 255) & ~(size_t)255;
  const size_t total = 6 * col4 + 4 * col8 + rows8 + rows4 + (size_t)n * n_dest;
  char* base = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&base), total) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_ENOMEM;
  }
  MultiStreamArgs a{};
  char* p = base;
  for (int k = 0; k < 5; ++k) { a.ints[k] = reinterpret_cast<const int32_t*>(p); p += col4; }
  for (int k = 0; k < 4; ++k) { a.dbls[k] = reinterpret_cast<const double*>(p); p += col8; }
  a.out_occ_origin = reinterpret_cast<int32_t*>(p); p += col4;
  a.out_time = reinterpret_cast<double*>(p); p += rows8;
  a.out_occ = reinterpret_cast<int32_t*>(p); p += rows4;
  a.out_status = reinterpret_cast<uint8_t*>(p);
  a.n = (uint32_t)n;
  a.n_dest = n_dest;
  const unsigned blocks = (unsigned)((n + 127) / 128);
  Timer t;
  int rc = t.ok ? HBT_OK : HBT_EHIP;
  float ms = 0.f;
  if (rc == HBT_OK && hipMemsetAsync(base, 0, total, nullptr) != hipSuccess) rc = HBT_EHIP;
  if (rc == HBT_OK) {
    for (int i = 0; i < warmup; ++i)
      hipLaunchKernelGGL(record_stream_multi_kernel, dim3(blocks), dim3(128), 0, nullptr, a);
    (void)hipEventRecord(t.e0, nullptr);
    for (int i = 0; i < launches; ++i)
      hipLaunchKernelGGL(record_stream_multi_kernel, dim3(blocks), dim3(128), 0, nullptr, a);
    (void)hipEventRecord(t.e1, nullptr);
    if (hipEventSynchronize(t.e1) != hipSuccess ||
        hipEventElapsedTime(&ms, t.e0, t.e1) != hipSuccess || hipGetLastError() != hipSuccess)
      rc = HBT_EHIP;
  }
  (void)hipFree(base);
  if (rc != HBT_OK) {
    (void)hipGetLastError();
    return rc;
  }
  *out_gbps = (56.0 + 13.0 * n_dest) * (double)n * launches / (ms * 1e6);
  return HBT_OK;
}

}  // extern "C"
