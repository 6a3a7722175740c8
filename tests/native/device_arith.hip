// Test infrastructure, not part of the product: brute-force checks, on the GPU,
// of the arithmetic shortcuts the wave-scaling kernels rely on, each over the
// whole domain its comment claims or over 2^30 operands where the domain is
// the doubles.  The functions under test are the product's own device code,
// included from habitat_amd/csrc; what they are held against is plain integer
// division, IEEE fp64 division and the device library's exp2.
//
//   arith_fast_div    fast_div_r(a, b, fast_rcp(b)) == a / b for every
//                     a >= 0, b > 0 with a + b <= 2^21 (occupancy.h)
//   arith_ceil_div    ceil_div_small<true>(nb, sms, 1/sms) == ceil(nb / sms) for
//                     every 1 <= sms <= 2^14, 0 <= nb < 64 * sms (wave_scale_device.h)
//   arith_div_const   div_const<C>(x) == x / C bit for bit wherever
//                     div_const_safe(x), for C = 100 and 1e9 (but for the sign
//                     of a zero, counted apart)
//   arith_occupancy_lattice  the 32-bit occupancy models the kernels run
//                     (occupancy_fast and its lean forms, occupancy_cdna in 32 bits)
//                     against the 64-bit models with plain division
//                     (occupancy_core, occupancy_cdna<true>) on a lattice of
//                     launch configurations of one device
//   arith_exp2        largest relative error of exp2_poly against exp2 on a grid
//   arith_exp2_at     exp2_poly at given points (saturation, NaN)
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/habitat_mi.h"
#include "../../habitat_amd/csrc/occupancy.h"
#include "../../habitat_amd/csrc/wave_scale.h"

#pragma clang fp contract(off)

#include "../../habitat_amd/csrc/wave_scale_device.h"

namespace {

using namespace hbt;
using namespace hbt::dev;

typedef unsigned long long u64;

struct Report {
  u64 checked, mismatches, first_a, first_b;
};

__device__ void note(Report* rep, u64 checked, u64 bad, u64 a, u64 b) {
  if (checked != 0) atomicAdd(&rep->checked, checked);
  if (bad != 0 && atomicAdd(&rep->mismatches, bad) == 0) {
    rep->first_a = a;
    rep->first_b = b;
  }
}

constexpr int kThreads = 256;

// One workgroup per divisor b; its threads stride over the dividends.  The
// expected quotient is carried along (k, r with a = k * b + r), so the loop
// holds no division of its own.
__global__ __launch_bounds__(kThreads) void fast_div_kernel(int32_t b_begin, int32_t b_end,
                                                            int32_t limit, Report* rep) {
  const int32_t b = b_begin + (int32_t)blockIdx.x;
  if (b >= b_end) return;
  const float rb = fast_rcp(b);
  int32_t a = threadIdx.x;
  int32_t k = a / b, r = a % b;
  const int32_t qt = kThreads / b, rt = kThreads % b;
  u64 checked = 0, bad = 0, bad_a = 0;
  for (; a <= limit - b; a += kThreads) {
    if (fast_div_r(a, b, rb) != k) {
      if (bad == 0) bad_a = (u64)a;
      ++bad;
    }
    ++checked;
    k += qt;
    r += rt;
    if (r >= b) {
      r -= b;
      ++k;
    }
  }
  note(rep, checked, bad, bad_a, (u64)b);
}

// One workgroup per divisor sms.
__global__ __launch_bounds__(kThreads) void ceil_div_kernel(const float* inv, int32_t sms_end,
                                                            Report* rep) {
  const int32_t sms = 1 + (int32_t)blockIdx.x;
  if (sms > sms_end) return;
  const float inv_sms = inv[sms];
  u64 checked = 0, bad = 0, bad_a = 0;
  for (int32_t nb = threadIdx.x; nb < 64 * sms; nb += kThreads) {
    const int32_t want = (nb + sms - 1) / sms;
    if (ceil_div_small<true>(nb, sms, inv_sms) != want) {
      if (bad == 0) bad_a = (u64)nb;
      ++bad;
    }
    ++checked;
  }
  note(rep, checked, bad, bad_a, (u64)sms);
}

__device__ u64 mix(u64 z) {  // splitmix64
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

// Operands are raw bit patterns (every exponent is as likely as any other);
// every fourth gets a short mantissa, where quotients by a constant land on
// or next to rounding boundaries more often.
template <class C>
__global__ __launch_bounds__(kThreads) void div_const_kernel(u64 n, u64 seed, Report* rep) {
  const u64 stride = (u64)gridDim.x * kThreads;
  u64 checked = 0, bad = 0, bad_bits = 0, zero_sign = 0;
  for (u64 i = (u64)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    u64 bits = mix(i ^ seed);
    if ((i & 3) == 3) bits &= ~((1ull << (int)(mix(i) % 52)) - 1ull);
    const double x = __longlong_as_double((long long)bits);
    if (!div_const_safe(x)) continue;
    const double got = div_const<C>(x);
    const double want = x / C::value;
    if (__double_as_longlong(got) != __double_as_longlong(want)) {
      if (got == 0.0 && want == 0.0) {
        ++zero_sign;  // x = -0.0 comes back as +0.0
      } else {
        if (bad == 0) bad_bits = bits;
        ++bad;
      }
    }
    ++checked;
  }
  note(rep, checked, bad, bad_bits, 0);
  if (zero_sign != 0) atomicAdd(&rep->first_b, zero_sign);
}

// The lattice: block sizes -1..1100, registers per thread 0..300 and 65535
// (what a uint16_t can hold at most), shared memory -600..600 bytes one by one
// and from there to 70 000 every size that is 0, 1, 2, 127, 128, 254 or 255
// above a multiple of 256 (all allocation granules are multiples of 256).
constexpr int kLatticeBlocks = 1102, kLatticeRegs = 302;
constexpr int kLatticeSmemDense = 1201, kLatticeSmemRows = 271;
constexpr int kLatticeSmem = kLatticeSmemDense + 7 * kLatticeSmemRows;

__device__ int32_t lattice_smem(int idx) {
  if (idx < kLatticeSmemDense) return idx - 600;
  const int j = idx - kLatticeSmemDense;
  const int residue[7] = {0, 1, 2, 127, 128, 254, 255};
  return 768 + (j / 7) * 256 + residue[j % 7];
}

// blockIdx.x: block size, blockIdx.y: registers; the threads stride over the
// shared-memory sizes.  `variants`: bit 0 occupancy_fast, 1 its lean form, 2 the
// lean form with the cc 6.0 re-check by select, 3 occupancy_cdna in 32 bits,
// 4 its lean form.
__global__ __launch_bounds__(kThreads) void occupancy_lattice_kernel(const OccDevice d,
                                                                     uint32_t variants,
                                                                     Report* rep) {
  const int32_t block = (int32_t)blockIdx.x - 1;
  const int32_t regs = blockIdx.y == kLatticeRegs - 1 ? 65535 : (int32_t)blockIdx.y;
  u64 checked = 0, bad = 0, bad_a = 0, bad_b = 0;
  for (int idx = threadIdx.x; idx < kLatticeSmem; idx += kThreads) {
    const int32_t smem = lattice_smem(idx);
    const SmemAlloc sm = smem_alloc(smem);
    const int32_t want = (d.flags & kCdna) ? occupancy_cdna<true>(d, block, smem, regs)
                                           : occupancy_core(d, block, smem, regs);
    uint32_t wrong = 0;
    if ((variants & 1) && occupancy_fast<false, false>(d, block, sm, regs) != want) wrong |= 1;
    if ((variants & 2) && occupancy_fast<true, false>(d, block, sm, regs) != want) wrong |= 2;
    if ((variants & 4) && occupancy_fast<true, true>(d, block, sm, regs) != want) wrong |= 4;
    if ((variants & 8) && occupancy_cdna<false, false>(d, block, smem, regs) != want) wrong |= 8;
    if ((variants & 16) && occupancy_cdna<false, true>(d, block, smem, regs) != want) wrong |= 16;
    if (wrong != 0) {
      if (bad == 0) {
        bad_a = ((u64)(uint32_t)block << 32) | (uint32_t)smem;
        bad_b = ((u64)(uint32_t)regs << 32) | wrong;
      }
      ++bad;
    }
    ++checked;
  }
  note(rep, checked, bad, bad_a, bad_b);
}

struct Exp2Report {
  u64 worst_err_bits;  // the largest relative error, as the bits of a double
  u64 checked;
};

__global__ __launch_bounds__(kThreads) void exp2_kernel(double lo, double step, u64 n,
                                                        Exp2Report* rep) {
  const u64 stride = (u64)gridDim.x * kThreads;
  double worst = 0.0;
  u64 checked = 0;
  for (u64 i = (u64)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    const double x = lo + step * (double)i;
    const double want = exp2(x);
    const double err = fabs(exp2_poly(x) - want) / want;
    worst = err > worst || err != err ? err : worst;
    ++checked;
  }
  // non-negative doubles order like their bit patterns; a NaN sorts above all
  atomicMax(&rep->worst_err_bits, (u64)__double_as_longlong(worst));
  atomicAdd(&rep->checked, checked);
}

__global__ void exp2_at_kernel(const double* x, int n, double* y) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = exp2_poly(x[i]);
}

template <class T>
struct DeviceBuffer {
  T* p = nullptr;
  explicit DeviceBuffer(size_t count) {
    if (hipMalloc(reinterpret_cast<void**>(&p), count * sizeof(T)) != hipSuccess) p = nullptr;
  }
  ~DeviceBuffer() {
    if (p != nullptr) (void)hipFree(p);
  }
};

int fetch(const Report* device, u64* out4) {
  Report host;
  if (hipDeviceSynchronize() != hipSuccess) return -2;
  if (hipMemcpy(&host, device, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) return -3;
  out4[0] = host.checked;
  out4[1] = host.mismatches;
  out4[2] = host.first_a;
  out4[3] = host.first_b;
  return 0;
}

}  // namespace

extern "C" {

// out4 = {pairs checked, mismatches, dividend and divisor of one mismatch}
int arith_fast_div(int32_t limit, u64* out4) {
  if (limit < 1 || limit > (1 << 21)) return -1;
  DeviceBuffer<Report> rep(1);
  if (rep.p == nullptr || hipMemset(rep.p, 0, sizeof(Report)) != hipSuccess) return -1;
  // a launch per 2^16 divisors keeps each launch well under a second
  for (int32_t b = 1; b <= limit; b += 1 << 16) {
    const int32_t end = b + (1 << 16) <= limit + 1 ? b + (1 << 16) : limit + 1;
    hipLaunchKernelGGL(fast_div_kernel, dim3((unsigned)(end - b)), dim3(kThreads), 0, 0, b, end,
                       limit, rep.p);
    if (hipGetLastError() != hipSuccess) return -2;
  }
  return fetch(rep.p, out4);
}

// out4 = {pairs checked, mismatches, block count and divisor of one mismatch}
int arith_ceil_div(int32_t sms_end, u64* out4) {
  if (sms_end < 1 || sms_end > (1 << 14)) return -1;
  DeviceBuffer<Report> rep(1);
  DeviceBuffer<float> inv((size_t)sms_end + 1);
  if (rep.p == nullptr || inv.p == nullptr || hipMemset(rep.p, 0, sizeof(Report)) != hipSuccess)
    return -1;
  // the reciprocals as the library's host code forms them (api.hip: 1.0f / (float)num_sms)
  float* host = new float[(size_t)sms_end + 1];
  host[0] = 0.f;
  for (int32_t s = 1; s <= sms_end; ++s) host[s] = 1.0f / (float)s;
  const hipError_t copied =
      hipMemcpy(inv.p, host, ((size_t)sms_end + 1) * sizeof(float), hipMemcpyHostToDevice);
  delete[] host;
  if (copied != hipSuccess) return -3;
  hipLaunchKernelGGL(ceil_div_kernel, dim3((unsigned)sms_end), dim3(kThreads), 0, 0, inv.p,
                     sms_end, rep.p);
  if (hipGetLastError() != hipSuccess) return -2;
  return fetch(rep.p, out4);
}

// which: 100 or 1000000000.  out4 = {operands checked (those div_const_safe
// accepts), mismatches, bit pattern of one mismatching operand, zeros that
// differ from the quotient in sign only (not counted as mismatches)}
int arith_div_const(int64_t which, u64 n, u64 seed, u64* out4) {
  DeviceBuffer<Report> rep(1);
  if (rep.p == nullptr || hipMemset(rep.p, 0, sizeof(Report)) != hipSuccess) return -1;
  const dim3 grid(256 * 16);
  if (which == 100)
    hipLaunchKernelGGL(div_const_kernel<C100>, grid, dim3(kThreads), 0, 0, n, seed, rep.p);
  else if (which == 1000000000)
    hipLaunchKernelGGL(div_const_kernel<C1e9>, grid, dim3(kThreads), 0, 0, n, seed, rep.p);
  else
    return -1;
  if (hipGetLastError() != hipSuccess) return -2;
  return fetch(rep.p, out4);
}

// The occupancy models of one device on the lattice.  out4 = {configurations
// checked, mismatches, (block << 32 | shared memory) and (registers << 32 |
// variants that differ) of one mismatch}; *variants_run = the variants that
// apply to this device (bits as in occupancy_lattice_kernel).
int arith_occupancy_lattice(const hbt_device_spec* spec, uint32_t* variants_run, u64* out4) {
  if (spec == nullptr) return -1;  // (a spec hbt_device_spec_check accepts: the caller's part)
  const OccDevice d = make_occ_device(*spec);
  uint32_t variants = 0;
  if (d.flags & kCdna) {
    if (d.fast_ok()) variants |= 8;
    if (d.cdna_lean_ok()) variants |= 16;
  } else {
    if (d.fast_ok()) variants |= 1;
    if (d.lean_ok()) variants |= 2;
    if (d.lean_gp_ok()) variants |= 4;
  }
  *variants_run = variants;
  DeviceBuffer<Report> rep(1);
  if (rep.p == nullptr || hipMemset(rep.p, 0, sizeof(Report)) != hipSuccess) return -1;
  hipLaunchKernelGGL(occupancy_lattice_kernel, dim3(kLatticeBlocks, kLatticeRegs), dim3(kThreads),
                     0, 0, d, variants, rep.p);
  if (hipGetLastError() != hipSuccess) return -2;
  return fetch(rep.p, out4);
}

// n points lo, lo + step, ...; out2 = {largest relative error, points checked}
int arith_exp2(double lo, double step, u64 n, double* out2) {
  DeviceBuffer<Exp2Report> rep(1);
  if (rep.p == nullptr || hipMemset(rep.p, 0, sizeof(Exp2Report)) != hipSuccess) return -1;
  hipLaunchKernelGGL(exp2_kernel, dim3(256 * 16), dim3(kThreads), 0, 0, lo, step, n, rep.p);
  if (hipGetLastError() != hipSuccess) return -2;
  if (hipDeviceSynchronize() != hipSuccess) return -2;
  Exp2Report host;
  if (hipMemcpy(&host, rep.p, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) return -3;
  union {
    u64 bits;
    double value;
  } worst;
  worst.bits = host.worst_err_bits;
  out2[0] = worst.value;
  out2[1] = (double)host.checked;
  return 0;
}

// x, y: HOST arrays of n doubles
int arith_exp2_at(const double* x, int32_t n, double* y) {
  if (n <= 0 || n > 65536) return -1;
  DeviceBuffer<double> dx((size_t)n), dy((size_t)n);
  if (dx.p == nullptr || dy.p == nullptr) return -1;
  if (hipMemcpy(dx.p, x, (size_t)n * sizeof(double), hipMemcpyHostToDevice) != hipSuccess)
    return -3;
  hipLaunchKernelGGL(exp2_at_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0, dx.p, n,
                     dy.p);
  if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess) return -2;
  return hipMemcpy(y, dy.p, (size_t)n * sizeof(double), hipMemcpyDeviceToHost) == hipSuccess ? 0
                                                                                            : -3;
}

}  // extern "C"
