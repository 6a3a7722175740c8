// Device code of wave scaling, shared by the per-record kernel (wave_scale.hip)
// and the fused per-operation sums (trace.hip): per record and destination, both
// occupancies and wave sizes, the roofline gamma, the small-kernel test and the
// scaled time, as the reference computes them one kernel at a time
// (analyzer/habitat/analysis/wave_scaling/unified.py:8-35, roofline.py:8-108,
// resimplified.py:7-40, common.py:3-20, cpp/src/cuda/kernel.cpp:29-56).
//
// Include after `#pragma clang fp contract(off)`: a*b+c must stay two roundings
// where the reference (CPython floats) has two.
#pragma once

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <type_traits>

#include "occupancy.h"
#include "wave_scale.h"

namespace hbt {
namespace dev {

// log2(i) for i = 0..63 (entry 0 unused), one entry per lane.  A kernel that
// fits in one wave on a device has num_blocks < num_sms * occupancy, so
// ceil(num_blocks / num_sms) is an integer in 1..occupancy.  NVIDIA-rule
// devices hold at most 32 blocks per SM; an AMD compute-unit description holds
// as many one-wave work-groups as it has wave slots, and hbt_device_spec_check
// keeps those at 63 or fewer (40 on a CU with 10 waves per SIMD), so the
// logarithm of the small-kernel factor needs no more than this table.  Each
// wavefront keeps it in one register pair (lane i holds entry i) and looks
// entries up with a cross-lane permute: no LDS, no barrier.
__device__ static const double kLog2Int[64] = {
    0x0.0p+0, 0x0.0p+0, 0x1.0000000000000p+0, 0x1.95c01a39fbd68p+0, 0x1.0000000000000p+1,
    0x1.2934f0979a371p+1, 0x1.4ae00d1cfdeb4p+1, 0x1.675767f54042dp+1, 0x1.8000000000000p+1,
    0x1.95c01a39fbd68p+1, 0x1.a934f0979a371p+1, 0x1.bacea7c065d42p+1, 0x1.cae00d1cfdeb4p+1,
    0x1.d9a802391e233p+1, 0x1.e75767f54042dp+1, 0x1.f414fdb498226p+1, 0x1.0000000000000p+2,
    0x1.0598fdbeb244cp+2, 0x1.0ae00d1cfdeb4p+2, 0x1.0fde0b5c81340p+2, 0x1.149a784bcd1b9p+2,
    0x1.191bba891f171p+2, 0x1.1d6753e032ea1p+2, 0x1.21820a01ac755p+2, 0x1.2570068e7ef5ap+2,
    0x1.2934f0979a371p+2, 0x1.2cd4011c8f119p+2, 0x1.305013ab7ce0ep+2, 0x1.33abb3faa0216p+2,
    0x1.36e9291eaa65bp+2, 0x1.3a0a7eda4c113p+2, 0x1.3d118d66c4d4ep+2, 0x1.4000000000000p+2,
    0x1.42d75a6eb1dfbp+2, 0x1.4598fdbeb244cp+2, 0x1.48462c466d3cfp+2, 0x1.4ae00d1cfdeb4p+2,
    0x1.4d67af16da765p+2, 0x1.4fde0b5c81340p+2, 0x1.524407ab0e074p+2, 0x1.549a784bcd1b9p+2,
    0x1.56e221cd9d0cep+2, 0x1.591bba891f171p+2, 0x1.5b47ebf73882ap+2, 0x1.5d6753e032ea1p+2,
    0x1.5f7a8568cb06dp+2, 0x1.61820a01ac755p+2, 0x1.637e623d2ba02p+2, 0x1.6570068e7ef5ap+2,
    0x1.675767f54042dp+2, 0x1.6934f0979a371p+2, 0x1.6b09044d313a6p+2, 0x1.6cd4011c8f119p+2,
    0x1.6e963fac9c0eap+2, 0x1.705013ab7ce0ep+2, 0x1.7201cc2c0005ap+2, 0x1.73abb3faa0216p+2,
    0x1.754e11eb0029ap+2, 0x1.76e9291eaa65bp+2, 0x1.787d3945c340bp+2, 0x1.7a0a7eda4c113p+2,
    0x1.7b9133567feaep+2, 0x1.7d118d66c4d4ep+2, 0x1.7e8bc1179e0cbp+2};

struct RecordIn {
  int32_t nb, block, smem_total, regs, dest_regs;
  bool metrics;
  double t, eff, rd, wr;
};

// Destination-independent part of one record.
struct RecordMid {
  SmemAlloc smem;
  int32_t occ_o, wave_o;
  int32_t origin_max_occ;  // ceil(num_blocks / origin.num_sms) when small_o, else 0
  bool small_o;            // num_blocks // origin_wave == 0
  bool redo_gflops;        // num_gflops needs origin_gflops_exact (see div_const)
  double num_gflops, total_gb;
  double log2_origin_max;  // log2(origin_max_occ), see finish_mid
};

// A double constant held in a scalar register pair.  The compiler would put a
// 64-bit literal that no instruction can encode into a VECTOR register pair
// first (two vector moves per use); an FMA reads one scalar operand for free,
// and the scalar moves that fill it run beside other waves' vector work.
__device__ __forceinline__ double scalar_const(double c) {
  asm("" : "+s"(c));
  return c;
}

// 2^x for finite x, relative error below 1e-13: split x = n + f with
// |f| <= 1/2, evaluate e^(f ln 2) by its Taylor polynomial of degree 11
// ((ln2 / 2)^12 / 12! < 7e-15) and scale by 2^n.
__device__ __forceinline__ double exp2_poly(double x) {
  const double n = rint(x);
  const double z = (x - n) * 0x1.62e42fefa39efp-1;  // f * ln 2
  double p = 1.0 / 39916800.0;
  p = fma(p, z, scalar_const(1.0 / 3628800.0));
  p = fma(p, z, scalar_const(1.0 / 362880.0));
  p = fma(p, z, scalar_const(1.0 / 40320.0));
  p = fma(p, z, scalar_const(1.0 / 5040.0));
  p = fma(p, z, scalar_const(1.0 / 720.0));
  p = fma(p, z, scalar_const(1.0 / 120.0));
  p = fma(p, z, scalar_const(1.0 / 24.0));
  p = fma(p, z, scalar_const(1.0 / 6.0));
  p = fma(p, z, 0.5);
  p = fma(p, z, 1.0);
  p = fma(p, z, 1.0);
  // |x| beyond the exponent range saturates through ldexp (inf or 0)
  const double nc = fmin(fmax(n, -4096.0), 4096.0);
  return ldexp(p, (int)nc);
}

// x / c for a compile-time constant c, correctly rounded like the IEEE
// division it replaces: q = x * (1/c) is within an ulp of the quotient, the
// remainder x - q*c is exact in an FMA, and adding remainder * (1/c) back
// rounds to the nearest double (Markstein's correction; checked against `/`
// on 1e9 operands for each constant used here).  One difference: x = -0.0
// comes back as +0.0 (the zero remainder is positive); the FLOP count this
// feeds is only compared with 1e-9, which no zero passes.  Valid where div_const_safe
// holds; elsewhere the remainder could underflow or overflow and the caller
// must divide for real.
template <class C>
__device__ __forceinline__ double div_const(double x) {
  constexpr double c = C::value, rc = 1.0 / C::value;
  const double q = x * rc;
  const double r = fma(-q, c, x);
  return fma(r, rc, q);
}

// zero, or finite with |x| >= 2^-900 (c > 1, so nothing can overflow)
__device__ __forceinline__ bool div_const_safe(double x) {
  const double ax = fabs(x);
  return (ax >= 0x1p-900 && ax < __builtin_inf()) || ax == 0.0;
}
struct C100 { static constexpr double value = 100.0; };
struct C1e9 { static constexpr double value = 1e9; };

// Which occupancy models a kernel instantiation contains.
//   The lean ones: every destination's ridge point lies within 2^+-500 and the
//     origin and every destination of the launch have OccDevice::lean_ok (the 32-bit NVIDIA-rule model, straight-line) or
//     cdna_lean_ok (the compute-unit model, straight-line), the origin one kind
//     and the destinations all one kind; nothing else is compiled in and no
//     branch is uniform over the launch.  kModelLeanGp: NVIDIA-rule devices
//     with a P100 among them (lean_gp_ok): the cc 6.0 re-check is computed for
//     every record and selected by the device's flag.
//   kModelGeneral: each device picks its model by wave-uniform branches: the
//     compute-unit model for AMD descriptions, the 64-bit model with real
//     divisions for devices with limits of 2^20 and more (not real hardware,
//     but in the domain).
enum : int {
  kModelGeneral = 0,
  kModelLean = 1,            // NVIDIA-rule origin and destinations
  kModelLeanCdnaDest = 2,    // NVIDIA-rule origin, AMD destinations
  kModelLeanCdnaOrigin = 3,  // AMD origin, NVIDIA-rule destinations
  kModelLeanCdna = 4,        // AMD origin and destinations
  kModelLeanGp = 5,          // NVIDIA-rule origin and destinations, cc 6.0 among them
};

// The instantiation for a launch from `origin` to the n_dest devices of `dests`.
inline int model_for(const OccDevice& origin, const DestArgs* dests, int n_dest) {
  bool lean = true, gp = true, cdna = true;
  for (int d = 0; d < n_dest; ++d) {
    // (the lean instantiations also form gamma the shared way, see
    // roofline_gamma_shared, which wants a ridge point of ordinary magnitude)
    if (!dests[d].ridge_in_range()) return kModelGeneral;
    lean = lean && dests[d].dev.lean_ok();
    gp = gp && dests[d].dev.lean_gp_ok();
    cdna = cdna && dests[d].dev.cdna_lean_ok();
  }
  if (origin.lean_ok() && lean) return kModelLean;
  if (origin.lean_ok() && cdna) return kModelLeanCdnaDest;
  if (origin.cdna_lean_ok() && lean) return kModelLeanCdnaOrigin;
  if (origin.cdna_lean_ok() && cdna) return kModelLeanCdna;
  if (origin.lean_gp_ok() && gp) return kModelLeanGp;
  return kModelGeneral;
}

// Calls f with the model as a compile-time constant.
template <class F>
inline void with_model(int model, F&& f) {
  switch (model) {
    case kModelLean: f(std::integral_constant<int, kModelLean>()); break;
    case kModelLeanCdnaDest: f(std::integral_constant<int, kModelLeanCdnaDest>()); break;
    case kModelLeanCdnaOrigin: f(std::integral_constant<int, kModelLeanCdnaOrigin>()); break;
    case kModelLeanCdna: f(std::integral_constant<int, kModelLeanCdna>()); break;
    case kModelLeanGp: f(std::integral_constant<int, kModelLeanGp>()); break;
    default: f(std::integral_constant<int, kModelGeneral>()); break;
  }
}

template <int MODEL, bool DEST>
__device__ __forceinline__ int32_t occupancy_dev(const OccDevice& d, int32_t block,
                                                 int32_t smem_total, const SmemAlloc& sm,
                                                 int32_t regs) {
  regs &= 0xFFFF;  // uint16_t narrowing, cpp/src/cuda/kernel.h:108
  constexpr bool cdna = DEST ? (MODEL == kModelLeanCdnaDest || MODEL == kModelLeanCdna)
                             : (MODEL == kModelLeanCdnaOrigin || MODEL == kModelLeanCdna);
  if (cdna) return occupancy_cdna<false, true>(d, block, smem_total, regs);
  if (MODEL == kModelLeanGp) return occupancy_fast<true, true>(d, block, sm, regs);
  if (MODEL != kModelGeneral) return occupancy_fast<true>(d, block, sm, regs);
  if (d.flags & kCdna)
    return d.fast_ok() ? occupancy_cdna<false>(d, block, smem_total, regs)
                       : occupancy_cdna<true>(d, block, smem_total, regs);
  return d.fast_ok() ? occupancy_fast(d, block, sm, regs)
                     : occupancy_core(d, block, smem_total, regs);
}

// ceil(nb / sms) for 0 <= nb < 32 * sms.  The reference takes math.ceil of the
// fp64 quotient (roofline.py:33-38); for operands below 2^53 that quotient is an
// integer only when the division is exact, so the integer ceiling is the same.
// With sms <= 2^14 (every fast_ok device) nb < 2^19: float(nb) * (1/sms) is within
// 2^-18 of the quotient, which is either an integer or at least 2^-14 away from
// one, so ceil(product - 2^-16) is the exact ceiling.
template <bool FAST>
__device__ __forceinline__ int32_t ceil_div_small(int32_t nb, int32_t sms, float inv_sms) {
  if (FAST || sms <= (1 << 14))
    return (int32_t)ceilf(fmaf(__int2float_rn(nb), inv_sms, -0x1p-16f));
  return (int32_t)(((int64_t)nb + sms - 1) / sms);
}

template <int MODEL>
__device__ __forceinline__ RecordMid origin_part(const OriginArgs& o, const RecordIn& r) {
  RecordMid m;
  m.smem = smem_alloc(r.smem_total);
  m.occ_o = occupancy_dev<MODEL, false>(o.dev, r.block, r.smem_total, m.smem, r.regs);
  m.wave_o = mul_small(o.dev.num_sms, m.occ_o);
  m.small_o = r.nb >= 0 && r.nb < m.wave_o;
  m.origin_max_occ =
      ceil_div_small<MODEL != kModelGeneral>(m.small_o ? r.nb : 0, o.dev.num_sms, o.inv_sms);
  // roofline.py:72-76, same operation order.  The three divisions by 1024 are
  // exact scalings, done here as one by 2^-30.  (Below 2^-992 bytes, where a
  // quotient is subnormal and one rounding is not three, the last bits of
  // total_gb reach no output: gamma is then forced to 1 by num_gflops < 1e-9
  // or lies within 1e-290 of 0.)
  m.total_gb = (r.rd + r.wr) * 0x1p-30;
  // eff / 100 * peak * t / 1e9 with the two constant divisions as corrected
  // multiplications.  No branch here: the caller tests redo_gflops of all its
  // records at once, so that their arithmetic stays in one basic block.
  const double gflops_per_second = div_const<C100>(r.eff) * o.peak_gflops;
  const double scaled = gflops_per_second * r.t;
  m.num_gflops = div_const<C1e9>(scaled);
  m.redo_gflops = !(div_const_safe(r.eff) && div_const_safe(scaled));
  return m;
}

// The same quantity with the divisions the reference performs (roofline.py:73-76),
// for records whose operands div_const cannot take: infinities, NaN, magnitudes
// below 2^-900.
__device__ __noinline__ double origin_gflops_exact(double peak_gflops, double eff, double t) {
  const double gflops_per_second = eff / 100 * peak_gflops;
  return gflops_per_second * t / 1e9;
}

// t * bw^gamma * clk^(1-gamma) * sm^(1-gamma) multiplied out from left to right
// as the reference does (roofline.py:58-63), for run times so large that a
// partial product overflows where the whole product does not: the reference
// then returns inf, and so must this.
__device__ __noinline__ double scaled_time_in_order(double t, double gamma, double log2_bw,
                                                    double log2_clk, double log2_clk_sm) {
  const double gamma_compl = 1.0 - gamma;
  double v = t * exp2_poly(gamma * log2_bw);
  v = v * exp2_poly(gamma_compl * log2_clk);
  return v * exp2_poly(gamma_compl * (log2_clk_sm - log2_clk));
}

struct RecordOut {
  double t;
  double gamma;
  bool in_order;  // t must be replaced by scaled_time_in_order (see there)
  int32_t occ_d, wave_d;
  uint8_t status;
};

// log2 of a small-kernel block count (0..63).  PERMUTE: read it from the lane
// that holds it (needs all 64 lanes of the wavefront active); otherwise gather
// it from the table in memory.
template <bool PERMUTE>
__device__ __forceinline__ double log2_count(double log2_lane, int32_t count) {
  if (PERMUTE) {
    // lane `count` of the wavefront (the hardware takes the lane number modulo 64)
    const int addr = count << 2;
    const int lo = __builtin_amdgcn_ds_bpermute(addr, __double2loint(log2_lane));
    const int hi = __builtin_amdgcn_ds_bpermute(addr, __double2hiint(log2_lane));
    return __hiloint2double(hi, lo);
  }
  return kLog2Int[count & 63];
}

// roofline.py:78-101 for one record and destination.  With I = gflops / gb the
// reference takes 0.5 * R / I above the ridge point R and 1 - 0.5 / R * I
// below; both are formed here from one division by choosing its operands
// first.  The choice compares gflops with R * gb instead of I with R, which can
// differ only within an ulp of the ridge, where the two expressions agree
// (gamma = 1/2).  A record without metrics takes the no-metrics strategy
// (resimplified.py:25-40): unchanged when small, else t * bw_ratio; with gamma = 1
// the roofline expressions reduce to exactly that.
__device__ __forceinline__ double roofline_gamma(const DestArgs& p, double num_gflops,
                                                 double total_gb, bool metrics) {
  const bool above = total_gb > 0 && num_gflops > p.ridge * total_gb;
  const double q = (above ? p.half_ridge * total_gb : num_gflops) /
                   (above ? num_gflops : total_gb);
  double gamma = above ? q : p.neg_half_over_ridge * q + 1.;
  gamma = (total_gb == 0) ? 0. : gamma;
  return (num_gflops < 1e-9 || !metrics) ? 1. : gamma;
}

// The same for a launch with several destinations, where the two divisions
// that do not depend on the destination are made once per record: the
// intensity I = gflops / gb as the reference forms it (the branch on I > R and
// the expression below the ridge are then the reference's own arithmetic) and
// 1 / I = gb / gflops, which gives 0.5 * R / I above the ridge as a product
// (two roundings instead of one: within 2 ulp).  Needs a ridge point within
// 2^+-500 (DestArgs::ridge_in_range), so that 1 / I is finite whenever I > R.
struct Intensity {
  double value, reciprocal;
};

__device__ __forceinline__ Intensity record_intensity(double num_gflops, double total_gb) {
  return Intensity{num_gflops / total_gb, total_gb / num_gflops};
}

__device__ __forceinline__ double roofline_gamma_shared(const DestArgs& p, double num_gflops,
                                                        double total_gb, const Intensity& in,
                                                        bool metrics) {
  // both expressions are formed and one is selected: no branch, and the
  // destination's constants are all fetched at the top of its turn
  const double over = p.half_ridge * in.reciprocal;
  const double under = p.neg_half_over_ridge * in.value + 1.;
  double gamma = in.value > p.ridge ? over : under;
  gamma = (total_gb == 0) ? 0. : gamma;
  return (num_gflops < 1e-9 || !metrics) ? 1. : gamma;
}

// log2 of the origin's small-kernel block count, which every destination of a
// launch uses: looked up once per record.
template <bool PERMUTE>
__device__ __forceinline__ void finish_mid(RecordMid& m, double log2_lane) {
  m.log2_origin_max = log2_count<PERMUTE>(log2_lane, m.origin_max_occ);
}

// Blocks per multiprocessor on the destination.  It depends on the device only
// through the occupancy constants, not through num_sms, bandwidth, clock or
// peak: destinations that agree in those (kSameOccAsPrev) share one evaluation.
template <int MODEL>
__device__ __forceinline__ int32_t dest_occupancy(const DestArgs& p, const RecordIn& r,
                                                  const RecordMid& m) {
  const int32_t regs_d = r.dest_regs >= 0 ? r.dest_regs : r.regs;
  return occupancy_dev<MODEL, true>(p.dev, r.block, r.smem_total, m.smem, regs_d);
}

// Everything after the destination's occupancy.  `gamma` is roofline_gamma or
// roofline_gamma_shared of the record for this destination; finish_mid has run.
template <int MODEL, bool PERMUTE>
__device__ __forceinline__ RecordOut dest_scale(const DestArgs& p, const RecordIn& r,
                                                const RecordMid& m, int32_t occ_d, double gamma,
                                                double log2_lane) {
  RecordOut o;
  o.occ_d = occ_d;
  o.wave_d = mul_small(p.dev.num_sms, o.occ_d);
  const bool bad_gamma = !(gamma >= 0 && gamma <= 1);

  // `a // wave_o == 0 and a // wave_d == 0`: the second test, and its division
  // by zero, happen only when the first holds (roofline.py:29-30).
  const bool small = m.small_o && r.nb < o.wave_d;
  const int32_t dest_max_occ =
      ceil_div_small<MODEL != kModelGeneral>(small ? r.nb : 0, p.dev.num_sms, p.inv_sms);

  int32_t status = HBT_ST_OK;
  status = (r.metrics && small && m.origin_max_occ == 0) ? HBT_ST_ZERO_BLOCKS : status;
  status = (m.small_o && o.wave_d == 0) ? HBT_ST_DEST_WAVE_ZERO : status;
  status = (m.wave_o == 0) ? HBT_ST_ORIGIN_WAVE_ZERO : status;
  status = bad_gamma ? HBT_ST_BAD_GAMMA : status;
  o.status = (uint8_t)status;

  // roofline.py:32-45: (clk_ratio * dest_max_occ / origin_max_occ)^(1-gamma), both
  // counts in 1..63; roofline.py:48-64: bw^gamma * clk^(1-gamma) * sm^(1-gamma)
  const double gamma_compl = 1.0 - gamma;
  const double log2_small =
      p.log2_clk + log2_count<PERMUTE>(log2_lane, dest_max_occ) - m.log2_origin_max;
  // small: (1-gamma) * log2_small; else gamma * L_bw + (1-gamma) * L_clk_sm.  As one
  // expression with selected operands (a zero first term is exact), so that
  // the code stays free of branches.
  const double exponent = (small ? 0.0 : gamma) * p.log2_bw +
                          gamma_compl * (small ? log2_small : p.log2_clk_sm);
  const double t = r.t * exp2_poly(exponent);
  o.t = (status == HBT_ST_OK) ? t : __builtin_nan("");
  // One combined power is the product of the reference's three to rounding,
  // unless a partial product overflows on the way where the whole does not:
  // only possible for run times beyond 2^500 ns (the factors are ratios of
  // device constants).  Those are left to the caller (scaled_time_in_order), so
  // that this function stays free of branches.  (No such case at the other
  // end: with a time small enough to underflow the FLOP count falls below
  // 1e-9, gamma is 1 and one factor is left.)
  o.gamma = gamma;
  o.in_order = status == HBT_ST_OK && !small && fabs(r.t) > 0x1p500;
  return o;
}

// One record, one destination, start to finish.  Written with selects rather
// than branches: the 64 records of a wavefront take all paths between them.
template <int MODEL, bool PERMUTE>
__device__ __forceinline__ RecordOut dest_part(const DestArgs& p, const RecordIn& r,
                                               RecordMid& m, double log2_lane) {
  finish_mid<PERMUTE>(m, log2_lane);
  const double gamma = roofline_gamma(p, m.num_gflops, m.total_gb, r.metrics);
  return dest_scale<MODEL, PERMUTE>(p, r, m, dest_occupancy<MODEL>(p, r, m), gamma, log2_lane);
}

}  // namespace dev
}  // namespace hbt
