/*
 * TEST INFRASTRUCTURE — CPU oracle, not product code.
 *
 * Plain-C restatement of the reference's per-kernel wave scaling, one record at
 * a time and in the reference's own operation order, so that every fp64
 * rounding is the one CPython makes (a Python float is a C double and
 * math.pow is libm's pow):
 *   unified_wave_scaling      analyzer/habitat/analysis/wave_scaling/unified.py:8-35
 *   roofline_wave_scaling     analyzer/habitat/analysis/wave_scaling/roofline.py:8-65
 *   _roofline_gamma           analyzer/habitat/analysis/wave_scaling/roofline.py:68-108
 *   resimplified_wave_scaling analyzer/habitat/analysis/wave_scaling/resimplified.py:7-40
 *   calculate_wave_info       analyzer/habitat/analysis/wave_scaling/common.py:3-20
 *
 * The reference raises where this code sets a status:
 *   1  origin wave size is 0      -> ZeroDivisionError (roofline.py:29, resimplified.py:25)
 *   2  destination wave size is 0 and the origin test did not short-circuit
 *                                 -> ZeroDivisionError (roofline.py:30, resimplified.py:26)
 *   3  gamma outside [0, 1] or NaN -> AssertionError   (roofline.py:103)
 *   4  num_blocks == 0 on the roofline small-kernel branch: ceil(0/sms) = 0 is a
 *      divisor                    -> ZeroDivisionError (roofline.py:40)
 * and the predicted time is NaN for such a record.
 *
 * pins: tests/test_oracle.py checks this file against oracle/wave_scaling.py
 * (a line-by-line Python restatement), against the hand-derived known answers
 * of tests/golden/kat.json (both branches of gamma, below and above the ridge
 * point; the small-kernel factor with unequal ceilings on the two devices;
 * table registers that move a record from one branch to the other; the
 * no-metrics strategy on both branches) and against closed forms (identity,
 * gamma 0 and 1, continuity at the ridge point).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

typedef struct {
  int32_t compute_major, compute_minor;
  int32_t max_threads_per_block, max_threads_per_sm;
  int32_t regs_per_block, regs_per_sm;
  int32_t warp_size, num_sms;
  int64_t smem_per_block, smem_per_sm, smem_per_block_optin;
  double mem_bandwidth_gb, base_clock_mhz, peak_gflops;
} orc_device;

uint32_t orc_occupancy(const orc_device *d, int32_t block, int32_t dyn_smem,
                       int32_t static_smem, int32_t registers);

/* Python's `a // b == 0` for integers with b > 0. */
static int floordiv_is_zero(int64_t a, int64_t b) { return a >= 0 && a < b; }

/* roofline.py:68-104.  Returns 0 and sets *gamma, or 1 when the assert fires. */
static int roofline_gamma(const orc_device *o, const orc_device *d, double t_ns,
                          double flop_eff, double rd, double wr, double *gamma) {
  double total_gb = (rd + wr) / 1024 / 1024 / 1024;
  double gflops_per_second = flop_eff / 100 * o->peak_gflops;
  double num_gflops = gflops_per_second * t_ns / 1e9;
  double g;
  if (num_gflops < 1e-9) {
    g = 1.;
  } else if (total_gb == 0) {
    g = 0.;
  } else {
    double intensity = num_gflops / total_gb;
    double ridge = d->peak_gflops / d->mem_bandwidth_gb;
    if (intensity > ridge)
      g = 0.5 * ridge / intensity;
    else
      g = -0.5 / ridge * intensity + 1.;
  }
  *gamma = g;
  return !(g >= 0 && g <= 1);
}

void orc_wave_scale(const orc_device *o, const orc_device *d, int64_t n,
                    const int32_t *num_blocks, const int32_t *block,
                    const int32_t *dyn_smem, const int32_t *static_smem,
                    const int32_t *regs, const int32_t *dest_regs /* nullable */,
                    const double *t_ns, const double *flop_eff, const double *rd,
                    const double *wr, const uint8_t *has_metrics /* nullable */,
                    double *out_t, int32_t *out_occ_o, int32_t *out_occ_d,
                    int32_t *out_wave_o, int32_t *out_wave_d, uint8_t *out_status,
                    double *out_gamma /* nullable */) {
  for (int64_t i = 0; i < n; ++i) {
    const int metrics = has_metrics == NULL || has_metrics[i] != 0;
    const double t = t_ns[i];
    const int64_t nb = num_blocks[i];
    double gamma = NAN;
    int bad_gamma = 0;
    /* unified.py:14-27 → roofline first computes gamma (roofline.py:14) */
    if (metrics) bad_gamma = roofline_gamma(o, d, t, flop_eff[i], rd[i], wr[i], &gamma);
    if (out_gamma) out_gamma[i] = gamma;

    /* common.py:3-20 */
    int32_t dr = (dest_regs != NULL && dest_regs[i] >= 0) ? dest_regs[i] : regs[i];
    int64_t occ_o = orc_occupancy(o, block[i], dyn_smem[i], static_smem[i], regs[i]);
    int64_t occ_d = orc_occupancy(d, block[i], dyn_smem[i], static_smem[i], dr);
    int64_t wave_o = (int64_t)o->num_sms * occ_o;
    int64_t wave_d = (int64_t)d->num_sms * occ_d;
    out_occ_o[i] = (int32_t)occ_o;
    out_occ_d[i] = (int32_t)occ_d;
    if (out_wave_o) out_wave_o[i] = (int32_t)wave_o;
    if (out_wave_d) out_wave_d[i] = (int32_t)wave_d;

    out_t[i] = NAN;
    if (bad_gamma) { out_status[i] = 3; continue; }
    if (wave_o == 0) { out_status[i] = 1; continue; }
    int small = floordiv_is_zero(nb, wave_o);
    if (small) {                       /* `and` evaluates the second test only now */
      if (wave_d == 0) { out_status[i] = 2; continue; }
      small = floordiv_is_zero(nb, wave_d);
    }
    out_status[i] = 0;

    if (!metrics) {                    /* resimplified.py:25-40 */
      if (small) out_t[i] = t;
      else out_t[i] = t * (o->mem_bandwidth_gb / d->mem_bandwidth_gb);
      continue;
    }

    const double gamma_compl = 1.0 - gamma;
    if (small) {                       /* roofline.py:32-45 */
      double origin_max_occ = ceil((double)nb / (double)o->num_sms);
      double dest_max_occ = ceil((double)nb / (double)d->num_sms);
      if (origin_max_occ == 0) { out_status[i] = 4; continue; }
      double factor = (o->base_clock_mhz / d->base_clock_mhz) *
                      (dest_max_occ / origin_max_occ);
      out_t[i] = t * pow(factor, gamma_compl);
      continue;
    }
    /* roofline.py:48-64, multiplied left to right */
    double bw = o->mem_bandwidth_gb / d->mem_bandwidth_gb;
    double clk = o->base_clock_mhz / d->base_clock_mhz;
    double sm = (double)o->num_sms / (double)d->num_sms;
    out_t[i] = t * pow(bw, gamma) * pow(clk, gamma_compl) * pow(sm, gamma_compl);
  }
}
