// Wave scaling of kernel records that live in HOST memory as an array of
// structures, results back in host memory: the boundary for callers that hold
// Python (or C++) kernel objects rather than columns on the GPU.
//
//   hbt_wave_scale_host_records   n records, one destination, one call: the
//       reference's per-kernel loop of Predictor._wave_scale
//       (analyzer/habitat/analysis/predictor.py:116-124) over the kernels of a
//       pass, an operation or a whole trace.
//   hbt_wave_scale_one            the same for one record: one call of the
//       strategy signature (wave_scaling/unified.py:8-35).
//
// Records and results travel through a pinned, device-visible staging block the
// library keeps per GPU (allocated on the first call there, kept until the
// process ends); the kernel reads the records and writes the results straight
// through it, so a call is one memcpy into the block, one launch, one wait and
// one memcpy out; arrays longer than the block go through its two halves in
// turn, the copies of one chunk beside the launch of the next.  The arithmetic is the code of wave_scale_device.h that the
// column kernel runs.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstring>
#include <mutex>

#include "../../include/habitat_mi.h"
#include "occupancy.h"
#include "wave_scale.h"

#pragma clang fp contract(off)

#include "wave_scale_device.h"

namespace hbt {
namespace {

using namespace dev;

constexpr int kBlock = 256;
// Records per pass through the staging block; longer arrays take several passes.
constexpr int64_t kChunk = 16384;

static_assert(sizeof(hbt_kernel_record) == 64, "the kernel reads a record as four 16-byte loads");

struct HostRecordArgs {
  int64_t n;
  const hbt_kernel_record* rec;  // device-visible host memory
  double* time_ns;
  int32_t* occ_origin;
  int32_t* occ_dest;
  uint8_t* status;
  // a launch of ONE workgroup stores done_value here (host-visible memory) once
  // its results are in place, so that the caller need not wait for the stream
  uint32_t* done_flag;  // nullable
  uint32_t done_value;
  OriginArgs origin;
  DestArgs dest;
};

using i32x4 = int32_t __attribute__((ext_vector_type(4)));
using f64x2 = double __attribute__((ext_vector_type(2)));

// One thread per record.
template <int MODEL>
__global__ __launch_bounds__(kBlock) void wave_scale_records_kernel(const HostRecordArgs a) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < a.n) {
    const char* p = reinterpret_cast<const char*>(a.rec + i);
    const i32x4 q0 = *reinterpret_cast<const i32x4*>(p);
    const i32x4 q1 = *reinterpret_cast<const i32x4*>(p + 16);
    const f64x2 d0 = *reinterpret_cast<const f64x2*>(p + 32);
    const f64x2 d1 = *reinterpret_cast<const f64x2*>(p + 48);
    RecordIn r;
    r.nb = q0[0];
    r.block = q0[1];
    r.smem_total = smem_sum(q0[3], q0[2]);
    r.regs = q1[0];
    r.dest_regs = q1[1];
    r.metrics = q1[2] != 0;
    r.t = d0[0];
    r.eff = d0[1];
    r.rd = d1[0];
    r.wr = d1[1];

    RecordMid m = origin_part<MODEL>(a.origin, r);
    if (__builtin_expect(m.redo_gflops, 0))
      m.num_gflops = origin_gflops_exact(a.origin.peak_gflops, r.eff, r.t);
    RecordOut o = dest_part<MODEL, false>(a.dest, r, m, 0.0);
    if (__builtin_expect(o.in_order, 0))
      o.t = scaled_time_in_order(r.t, o.gamma, a.dest.log2_bw, a.dest.log2_clk, a.dest.log2_clk_sm);
    a.time_ns[i] = o.t;
    a.occ_origin[i] = m.occ_o;
    a.occ_dest[i] = o.occ_d;
    a.status[i] = o.status;
  }
  if (a.done_flag != nullptr) {       // uniform; the launch is one workgroup
    __threadfence_system();           // this thread's results, then ...
    __syncthreads();                  // ... everybody's
    if (threadIdx.x == 0)
      __hip_atomic_store(a.done_flag, a.done_value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// The staging block of one GPU: two slots of kChunk records in and their
// results out, so that an array of several chunks keeps the GPU on one slot
// while the calling thread empties and refills the other.
struct Staging {
  std::mutex lock;  // one call at a time per device: the block is shared
  unsigned char* host = nullptr;
  unsigned char* device = nullptr;
  hipEvent_t filled[2] = {nullptr, nullptr};  // slot's results are in place
  uint32_t calls = 0;  // numbers the one-workgroup launches: the value they publish
};
constexpr size_t kOffTime = (size_t)kChunk * sizeof(hbt_kernel_record);
constexpr size_t kOffOccOrigin = kOffTime + (size_t)kChunk * sizeof(double);
constexpr size_t kOffOccDest = kOffOccOrigin + (size_t)kChunk * sizeof(int32_t);
constexpr size_t kOffStatus = kOffOccDest + (size_t)kChunk * sizeof(int32_t);
constexpr size_t kSlotBytes = (kOffStatus + (size_t)kChunk + 255) & ~(size_t)255;
constexpr size_t kOffDone = 2 * kSlotBytes;  // one completion word for the block
constexpr size_t kStagingBytes = kOffDone + 64;
constexpr int kMaxDevices = 64;
Staging g_staging[kMaxDevices];

int staging_ready(Staging& st) {
  if (st.host != nullptr) return HBT_OK;
  void* h = nullptr;
  void* d = nullptr;
  hipEvent_t events[2] = {nullptr, nullptr};
  if (hipHostMalloc(&h, kStagingBytes, hipHostMallocDefault) != hipSuccess ||
      hipHostGetDevicePointer(&d, h, 0) != hipSuccess || d == nullptr ||
      hipEventCreateWithFlags(&events[0], hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&events[1], hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    if (events[0] != nullptr) (void)hipEventDestroy(events[0]);
    if (h != nullptr) (void)hipHostFree(h);
    return HBT_ENOMEM;
  }
  st.host = static_cast<unsigned char*>(h);
  st.device = static_cast<unsigned char*>(d);
  st.filled[0] = events[0];
  st.filled[1] = events[1];
  std::memset(st.host + kOffDone, 0, 64);
  return HBT_OK;
}

// Results of `m` records from a slot to the caller's arrays at `done`.
void copy_out(const unsigned char* slot, int64_t done, int64_t m, double* out_time_ns,
              uint8_t* out_status, int32_t* out_occ_origin, int32_t* out_occ_dest) {
  std::memcpy(out_time_ns + done, slot + kOffTime, (size_t)m * sizeof(double));
  std::memcpy(out_status + done, slot + kOffStatus, (size_t)m);
  if (out_occ_origin != nullptr)
    std::memcpy(out_occ_origin + done, slot + kOffOccOrigin, (size_t)m * sizeof(int32_t));
  if (out_occ_dest != nullptr)
    std::memcpy(out_occ_dest + done, slot + kOffOccDest, (size_t)m * sizeof(int32_t));
}

// The stream must be usable for a launch followed by a wait: not under
// capture, and a stream of the current device (whose staging block is used).
int stream_usable(hipStream_t stream, int device) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (capture != hipStreamCaptureStatusNone) return HBT_EINVAL;
  hipDevice_t of_stream = device;
  if (hipStreamGetDevice(stream, &of_stream) == hipSuccess) {
    if ((int)of_stream != device) return HBT_EINVAL;
  } else {
    (void)hipGetLastError();
  }
  return HBT_OK;
}

}  // namespace

bool wait_published(const uint32_t* flag, uint32_t value) {
  using clock = std::chrono::steady_clock;
  const clock::time_point give_up = clock::now() + std::chrono::microseconds(200);
  for (;;) {
    for (int spin = 0; spin < 64; ++spin)
      if (__atomic_load_n(flag, __ATOMIC_ACQUIRE) == value) return true;
    if (clock::now() > give_up) return false;
  }
}

}  // namespace hbt

extern "C" {

int hbt_wave_scale_host_records(const hbt_device_spec* origin, const hbt_device_spec* dest,
                                int64_t n, const hbt_kernel_record* records, double* out_time_ns,
                                uint8_t* out_status, int32_t* out_occ_origin,
                                int32_t* out_occ_dest, void* hip_stream) {
  using namespace hbt;
  if (origin == nullptr || dest == nullptr || n < 0) return HBT_EINVAL;
  int rc = hbt_device_spec_check(origin);
  if (rc == HBT_OK) rc = hbt_device_spec_check(dest);
  if (rc != HBT_OK) return rc;
  if (n == 0) return HBT_OK;
  if (records == nullptr || out_time_ns == nullptr || out_status == nullptr) return HBT_EINVAL;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (device < 0 || device >= kMaxDevices) return HBT_ESIZE;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  if ((rc = stream_usable(stream, device)) != HBT_OK) return rc;

  Staging& st = g_staging[device];
  std::lock_guard<std::mutex> guard(st.lock);
  if ((rc = staging_ready(st)) != HBT_OK) return rc;

  HostRecordArgs a{};
  a.origin = make_origin_args(*origin);
  a.dest = make_dest_args(*origin, *dest);
  const int model = dev::model_for(a.origin.dev, &a.dest, 1);
  const auto launch = [&](int slot, int64_t m, const dim3 grid) {
    unsigned char* base = st.device + (size_t)slot * kSlotBytes;
    a.n = m;
    a.rec = reinterpret_cast<const hbt_kernel_record*>(base);
    a.time_ns = reinterpret_cast<double*>(base + kOffTime);
    a.occ_origin = reinterpret_cast<int32_t*>(base + kOffOccOrigin);
    a.occ_dest = reinterpret_cast<int32_t*>(base + kOffOccDest);
    a.status = base + kOffStatus;
    dev::with_model(model, [&](auto mc) {
      hipLaunchKernelGGL(wave_scale_records_kernel<decltype(mc)::value>, grid, dim3(kBlock), 0,
                         stream, a);
    });
    return hipGetLastError() == hipSuccess;
  };

  if (n <= kChunk) {
    std::memcpy(st.host, records, (size_t)n * sizeof(hbt_kernel_record));
    const dim3 grid((unsigned)((n + kBlock - 1) / kBlock));
    // one workgroup (one kernel, a pass of a few kernels): it publishes its own
    // completion, see wait_published
    const bool publishes = grid.x == 1;
    a.done_flag = publishes ? reinterpret_cast<uint32_t*>(st.device + kOffDone) : nullptr;
    a.done_value = publishes ? ++st.calls : 0;
    if (!launch(0, n, grid)) return HBT_EHIP;
    if (!(publishes &&
          wait_published(reinterpret_cast<const uint32_t*>(st.host + kOffDone), a.done_value)) &&
        hipStreamSynchronize(stream) != hipSuccess) {
      (void)hipGetLastError();
      return HBT_EHIP;
    }
    copy_out(st.host, 0, n, out_time_ns, out_status, out_occ_origin, out_occ_dest);
    return HBT_OK;
  }

  // Several chunks, slots in turn: while the GPU works on one slot the calling
  // thread copies the chunk before out of the other and, in the next turn, the
  // next chunk into it.  A slot is refilled only after its results were taken.
  int64_t before_done = 0, before_m = 0;  // the chunk launched one turn ago
  int turn = 0;
  // (an error with a launch in flight: let the stream drain before the block is used again)
  const auto fail = [&]() {
    (void)hipGetLastError();
    (void)hipStreamSynchronize(stream);
    (void)hipGetLastError();
    return HBT_EHIP;
  };
  for (int64_t done = 0; done < n; done += kChunk, ++turn) {
    const int slot = turn & 1;
    const int64_t m = (n - done < kChunk) ? (n - done) : kChunk;
    std::memcpy(st.host + (size_t)slot * kSlotBytes, records + done,
                (size_t)m * sizeof(hbt_kernel_record));
    a.done_flag = nullptr;
    a.done_value = 0;
    if (!launch(slot, m, dim3((unsigned)((m + kBlock - 1) / kBlock)))) return fail();
    if (hipEventRecord(st.filled[slot], stream) != hipSuccess) return fail();
    if (turn > 0) {
      if (hipEventSynchronize(st.filled[slot ^ 1]) != hipSuccess) return fail();
      copy_out(st.host + (size_t)(slot ^ 1) * kSlotBytes, before_done, before_m, out_time_ns,
               out_status, out_occ_origin, out_occ_dest);
    }
    before_done = done;
    before_m = m;
  }
  const int last = (turn - 1) & 1;
  if (hipEventSynchronize(st.filled[last]) != hipSuccess) return fail();
  copy_out(st.host + (size_t)last * kSlotBytes, before_done, before_m, out_time_ns, out_status,
           out_occ_origin, out_occ_dest);
  return HBT_OK;
}

int hbt_wave_scale_one(const hbt_device_spec* origin, const hbt_device_spec* dest,
                       const hbt_kernel_record* record, double* out_time_ns,
                       int32_t* out_occ_origin, int32_t* out_occ_dest, uint8_t* out_status,
                       void* hip_stream) {
  if (record == nullptr || out_time_ns == nullptr || out_status == nullptr) return HBT_EINVAL;
  return hbt_wave_scale_host_records(origin, dest, 1, record, out_time_ns, out_status,
                                     out_occ_origin, out_occ_dest, hip_stream);
}

}  // extern "C"
