/*
 * habitat_mi — C ABI of the MI355X-native batched-prediction path.
 *
 * This is the whole boundary between host code (Python via ctypes, or any
 * other FFI) and the HIP kernels.  Plain pointers and sizes only.  Unless a
 * parameter says "host", every array pointer is DEVICE memory owned by the
 * caller; work is enqueued on the given HIP stream (NULL = the default stream)
 * and the call returns without synchronising.  Functions return 0 or a
 * negative HBT_E* code; hbt_strerror() names it.  There is no CPU fallback:
 * without a GPU the compute entry points return HBT_EHIP.  Only the two
 * *_create calls allocate device memory (and the calibration calls at the
 * end, which say so); the library's only state outside its handles is what
 * hbt_wave_scale_host_records and hbt_mlp_forward_static say they keep per GPU.
 *
 * Each entry point cites the reference interface it stands in for
 * (paths relative to the reference tree).
 */
#ifndef HABITAT_MI_H_
#define HABITAT_MI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HBT_VERSION 103 /* 0.1.3 */

enum {
  HBT_OK = 0,
  HBT_EINVAL = -1, /* null pointer, negative count, bad argument */
  HBT_ESPEC = -2,  /* device spec outside the supported domain (see hbt_device_spec_check) */
  HBT_EHIP = -3,   /* a HIP runtime call failed (no GPU, bad stream, launch error) */
  HBT_ENOMEM = -4, /* allocation failed (the *_create calls only) */
  HBT_EALIGN = -5, /* a column pointer is not aligned to its element size */
  HBT_ESIZE = -6   /* size beyond what the entry point supports */
};

/* Per-record status written by hbt_wave_scale.  Non-zero statuses are the
 * places where the reference's scalar Python raises instead of returning; the
 * predicted time of such a record is NaN. */
enum {
  HBT_ST_OK = 0,
  HBT_ST_ORIGIN_WAVE_ZERO = 1, /* ZeroDivisionError at wave_scaling/roofline.py:29, resimplified.py:25 */
  HBT_ST_DEST_WAVE_ZERO = 2,   /* ZeroDivisionError at wave_scaling/roofline.py:30, resimplified.py:26 */
  HBT_ST_BAD_GAMMA = 3,        /* AssertionError at wave_scaling/roofline.py:103 */
  HBT_ST_ZERO_BLOCKS = 4       /* ZeroDivisionError at wave_scaling/roofline.py:40 (num_blocks == 0) */
};

/*
 * compute_major of a device described by AMD's compute-unit model instead of
 * the reference's NVIDIA one: 100 + the major HIP reports for the gfx9 family
 * (compute_minor = HIP's minor: 0 gfx90a, 4 gfx942, 5 gfx950).  No counterpart
 * in the reference, whose occupancy routine knows compute capabilities 3.x to
 * 7.x and answers 0 for anything else (cpp/src/cuda/cuda_occupancy.h:573-694),
 * plain 9.x included, which this library does too.  With this value the fields
 * read: warp_size = wavefront size, max_threads_per_sm = wave slots of a CU x
 * wavefront size, regs_per_sm = VGPRs of a CU counted per lane (4 SIMDs x 512
 * x 64), smem_per_block / smem_per_sm = LDS a work-group may use / LDS of a
 * CU, num_sms = CUs; regs_per_block is not used.  Occupancy (work-groups per
 * CU) follows the public LLVM AMDGPU rules: VGPRs allocated in granules of 8
 * per lane out of regs_per_sm / (4 x warp_size), a work-group's waves spread
 * over the 4 SIMDs, 16 work-groups with more than one wave per CU, LDS in
 * granules of 512 B (1280 B on gfx950).
 */
#define HBT_COMPUTE_MAJOR_CDNA 109

/*
 * Device description.  Replaces habitat::cuda::DeviceProperties
 * (cpp/src/cuda/kernel.h:14-62; Python constructor
 * cpp/src/frontend/model_bindings.cpp:17-55) minus the name, which stays on
 * the host side.  The three double fields hold integer values, as the
 * reference's fields are integers (kernel.h:59-61).
 */
typedef struct hbt_device_spec {
  int32_t compute_major, compute_minor;
  int32_t max_threads_per_block, max_threads_per_sm;
  int32_t regs_per_block, regs_per_sm;
  int32_t warp_size, num_sms;
  int64_t smem_per_block, smem_per_sm, smem_per_block_optin;
  double mem_bandwidth_gb, base_clock_mhz, peak_gflops;
} hbt_device_spec;

int hbt_version(void);
const char *hbt_strerror(int code);

/* Number of HIP devices visible to the library (0 without a GPU); never fails. */
int hbt_device_count(void);

/*
 * HBT_OK when `spec` (host) is inside the domain the batch kernels accept:
 * smem fields >= 0 and < 2^31, warp_size <= 32768, num_sms <= 2^20,
 * mem_bandwidth_gb, base_clock_mhz, peak_gflops finite and > 0, and for an AMD
 * compute-unit description (HBT_COMPUTE_MAJOR_CDNA) at most 63 wave slots per
 * CU (max_threads_per_sm / warp_size; 32 on gfx90a and later, 40 on CUs with 10
 * waves per SIMD).  A spec the
 * occupancy model rejects (unknown compute capability, a zero limit) is still
 * in the domain: every occupancy on it is 0, as in the reference.
 */
int hbt_device_spec_check(const hbt_device_spec *spec);

/*
 * Thread-block occupancy of one launch configuration on one device, on the
 * HOST (all pointers host).  Replaces KernelMetadata::threadBlockOccupancy
 * (cpp/src/cuda/kernel.h:104-115, cpp/src/cuda/kernel.cpp:29-56) and its Python
 * face KernelInstance.thread_block_occupancy
 * (cpp/src/frontend/model_bindings.cpp:75-82).  `regs` is narrowed to 16 bits
 * as there; any error in the model gives *out = 0.
 */
int hbt_occupancy_host(const hbt_device_spec *spec, int32_t block_size, int32_t dynamic_smem,
                       int32_t static_smem, int32_t regs, uint32_t *out);

/* The same over host arrays (used by data generators and host-side callers). */
int hbt_occupancy_host_batch(const hbt_device_spec *spec, int64_t n, const int32_t *block_size,
                             const int32_t *dynamic_smem, const int32_t *static_smem,
                             const int32_t *regs, int32_t *out);

/*
 * Diagnostic: the 32-bit formulation of the same model that the wave-scaling
 * kernel uses for devices whose limits are all below 2^20, evaluated on the
 * HOST over host arrays (its float-reciprocal divisions replaced by exact
 * ones), in the straight-line form the kernels run where the device allows
 * it.  Lets the kernel's integer logic be checked against
 * hbt_occupancy_host_batch without a GPU.  Returns HBT_ESPEC for a device
 * outside that formulation's domain.  No counterpart in the reference.
 */
int hbt_occupancy_host_model32_batch(const hbt_device_spec *spec, int64_t n,
                                     const int32_t *block_size, const int32_t *dynamic_smem,
                                     const int32_t *static_smem, const int32_t *regs,
                                     int32_t *out);

/*
 * Wave-scale n kernel records measured on `origin` to each of n_dest
 * destination devices.  One launch replaces the per-kernel Python loop of
 * Predictor._wave_scale (analyzer/habitat/analysis/predictor.py:116-124) and,
 * per record, unified_wave_scaling (analysis/wave_scaling/unified.py:8-35) with
 * everything under it: roofline.py:8-108, resimplified.py:7-40,
 * common.py:3-20 and the occupancy routine above.
 *
 * origin, dests: HOST pointers (dests is an array of n_dest specs).
 * Input columns (device, length n): the fields of KernelMetadata /
 * KernelInstance (cpp/src/cuda/kernel.h:64-151) and the three metrics that
 * roofline.py:69-71 reads.
 *   dest_regs    nullable; >= 0 replaces regs for the destination occupancy
 *                (MetadataManager.kernel_registers_for, wave_scaling/metadata.py:12-37;
 *                < 0 = no entry)
 *   has_metrics  nullable (= all present); 0 selects the no-metrics strategy
 * Outputs (device): out_time_ns, out_occ_dest, out_wave_dest, out_status are
 * [n_dest][n] row-major; out_occ_origin, out_wave_origin are [n].
 * out_wave_*, out_status and out_occ_* are nullable.
 */
int hbt_wave_scale(const hbt_device_spec *origin, const hbt_device_spec *dests, int32_t n_dest,
                   int64_t n, const int32_t *num_blocks, const int32_t *block_size,
                   const int32_t *dynamic_smem, const int32_t *static_smem, const int32_t *regs,
                   const int32_t *dest_regs, const double *run_time_ns,
                   const double *flop_sp_efficiency, const double *dram_read_bytes,
                   const double *dram_write_bytes, const uint8_t *has_metrics,
                   double *out_time_ns, int32_t *out_occ_origin, int32_t *out_occ_dest,
                   int32_t *out_wave_origin, int32_t *out_wave_dest, uint8_t *out_status,
                   void *hip_stream);

/*
 * Kernel records held in HOST memory as an array of structures, one
 * destination, results back in host memory, start to finish: the per-kernel
 * loop of Predictor._wave_scale (analysis/predictor.py:116-124), i.e. n calls of
 * strategy(kernel, origin_device, dest_device, metadata_manager)
 * (wave_scaling/unified.py:8-35), as ONE C call.  This is the entry for callers
 * that hold kernel objects on the host (the reference's plug point) rather
 * than columns on the GPU.  `records`, out_time_ns [n], out_status [n],
 * out_occ_origin [n] and out_occ_dest [n] (both nullable) are HOST memory.
 * Per record: dest_regs < 0 = no register-table entry; has_metrics == 0 selects
 * the no-metrics strategy; out_status is one of HBT_ST_* and the time is NaN
 * unless it is HBT_ST_OK.
 *
 * The records go through a pinned, device-visible staging block of the library
 * (about 2.7 MiB per GPU, allocated on the first call there and kept): up to
 * 16384 records in one launch on `hip_stream` and a wait, so the call returns
 * with the results in place (some 15 us for up to a few thousand records);
 * longer arrays in chunks of 16384 through the block's two halves in turn, one
 * chunk on the GPU while the calling thread copies the one before out and the
 * next in.  Calls on one GPU are serialised inside the library.
 * `hip_stream` must be a stream of the current device and must not be under
 * graph capture (HBT_EINVAL): the call waits for it.
 */
typedef struct hbt_kernel_record {
  int32_t num_blocks, block_size, dynamic_smem, static_smem, regs, dest_regs;
  int32_t has_metrics, reserved;
  double run_time_ns, flop_sp_efficiency, dram_read_bytes, dram_write_bytes;
} hbt_kernel_record;
int hbt_wave_scale_host_records(const hbt_device_spec *origin, const hbt_device_spec *dest,
                                int64_t n, const hbt_kernel_record *records, double *out_time_ns,
                                uint8_t *out_status, int32_t *out_occ_origin,
                                int32_t *out_occ_dest, void *hip_stream);

/*
 * One kernel record: hbt_wave_scale_host_records with n = 1, the reference's
 * strategy call (analysis/predictor.py:116-124 invoking
 * wave_scaling/unified.py:8-35) one kernel at a time.  All of its cost is the
 * launch and the wait; callers with many kernels should hand them over together.
 */
int hbt_wave_scale_one(const hbt_device_spec *origin, const hbt_device_spec *dest,
                       const hbt_kernel_record *record, double *out_time_ns,
                       int32_t *out_occ_origin, int32_t *out_occ_dest, uint8_t *out_status,
                       void *hip_stream);

/*
 * A set of destination devices resident on the GPU, for predicting one trace
 * on many devices at once.  hbt_device_table_create takes HOST pointers, folds
 * the per-device constants of (origin, dests[i]) and uploads them to the
 * current HIP device; with hbt_mlp_create it is the only call that allocates.
 * Returns NULL on failure (and sets *err if err is not NULL).  No counterpart
 * in the reference, which handles one destination per Trace.to_device call
 * (analyzer/habitat/analysis/trace.py:38-51).
 */
typedef struct hbt_device_table hbt_device_table;
hbt_device_table *hbt_device_table_create(const hbt_device_spec *origin,
                                          const hbt_device_spec *dests, int32_t n_dest, int *err);
int32_t hbt_device_table_size(const hbt_device_table *table);
void hbt_device_table_destroy(hbt_device_table *table);

/*
 * Wave scaling fused with the per-pass sums: for every destination d of the
 * table and every segment s, out_sum[d][s] = sum of the scaled times of the
 * records k with segment[k] == s.  A segment is one forward or backward pass of
 * one operation, so out_sum is the kernel part of RunTimePrediction.run_time_ms
 * (analyzer/habitat/analysis/run_time.py:50-58) for the kernels that
 * Predictor._wave_scale (analysis/predictor.py:111-130) scales one by one; the
 * caller adds the pass overhead, which does not depend on the destination.
 * Input columns as for hbt_wave_scale; `segment` (device, [n], nullable = one
 * segment) holds values in [0, n_segments), others are ignored.  Records whose
 * status is not HBT_ST_OK on d add nothing and are counted in out_bad[d]
 * (nullable): the reference would have raised for that destination.  out_sum
 * ([n_dest][n_segments]) and out_bad ([n_dest]) are overwritten.  Sums are
 * accumulated with floating-point atomics: their rounding can differ in the
 * last bits from run to run.  Must be called with the table's device current.
 */
int hbt_wave_scale_sum(const hbt_device_table *table, int64_t n, const int32_t *num_blocks,
                       const int32_t *block_size, const int32_t *dynamic_smem,
                       const int32_t *static_smem, const int32_t *regs, const int32_t *dest_regs,
                       const double *run_time_ns, const double *flop_sp_efficiency,
                       const double *dram_read_bytes, const double *dram_write_bytes,
                       const uint8_t *has_metrics, const int32_t *segment, int32_t n_segments,
                       double *out_sum, int32_t *out_bad, void *hip_stream);

/*
 * The same sums for segments that are runs of consecutive records, added up in
 * the records' order like the reference's sequential sum over a pass's kernels
 * (analysis/run_time.py:50-58): segment s holds the records
 * [segment_start[s], segment_start[s + 1]) (device, [n_segments + 1], int64,
 * non-decreasing, segment_start[n_segments] <= n; the caller guarantees that).
 * No floating-point atomics: the scaled times go through `workspace` (device,
 * [n_dest][n] doubles, the caller's; contents afterwards unspecified) and one
 * thread per (segment, destination) adds them up in order, so out_sum[d][s] is
 * the sequential fp64 sum of the times hbt_wave_scale writes for those records
 * on d (a one-destination launch), bit for bit and the same on every run.
 * Everything else as for hbt_wave_scale_sum.
 */
int hbt_wave_scale_sum_ordered(const hbt_device_table *table, int64_t n, const int32_t *num_blocks,
                               const int32_t *block_size, const int32_t *dynamic_smem,
                               const int32_t *static_smem, const int32_t *regs,
                               const int32_t *dest_regs, const double *run_time_ns,
                               const double *flop_sp_efficiency, const double *dram_read_bytes,
                               const double *dram_write_bytes, const uint8_t *has_metrics,
                               const int64_t *segment_start, int32_t n_segments, double *workspace,
                               double *out_sum, int32_t *out_bad, void *hip_stream);

/*
 * The roofline exponent alone, _roofline_gamma
 * (analysis/wave_scaling/roofline.py:68-104) with _ridge_point (:107-108), for n
 * records that all have their three metrics: out_gamma[n] fp64, NaN where the
 * reference's assertion 0 <= gamma <= 1 fails.  hbt_wave_scale computes the
 * same value internally; this entry exists so that it can be inspected.
 */
int hbt_roofline_gamma(const hbt_device_spec *origin, const hbt_device_spec *dest, int64_t n,
                       const double *run_time_ns, const double *flop_sp_efficiency,
                       const double *dram_read_bytes, const double *dram_write_bytes,
                       double *out_gamma, void *hip_stream);

/*
 * The last step of the MLP-predicted operations for a device sweep
 * (analysis/predictor.py:132-148 with :182,218,238,283): pred is
 * [(n_dest + 1)][n_rows] fp32 MLP outputs, the last row evaluated with the
 * origin's device features; operation o reads column op_row[o] (device,
 * [n_ops], nullable = column o, then n_rows must equal n_ops), so operations
 * with equal features share one MLP row.  out_ms[d][o] = run_time_ms[o] *
 * pred[d][r] / pred[n_dest][r] in fp64, negative values replaced by 0 (out_ms
 * nullable); out_total[d] += sum over o of out_ms[d][o] (nullable);
 * out_clamped[d] += the number of operations whose value was negative
 * (nullable): the reference logs a warning for each of them
 * (predictor.py:135-141).  A column index outside [0, n_rows) gives NaN.
 */
int hbt_ratio_scale(const float *pred, int32_t n_dest, int32_t n_rows, const int32_t *op_row,
                    int32_t n_ops, const double *run_time_ms, double *out_ms, double *out_total,
                    int32_t *out_clamped, void *hip_stream);

/*
 * Per-operation MLP (fc1 -> ReLU -> hidden x (Linear, ReLU) -> fc2), the
 * network of analysis/mlp/mlp.py:17-109.  hbt_mlp_create takes HOST pointers:
 * W[0] is fc1.weight [width][in_features], W[1..hidden] are the hidden
 * weights [width][width], W[hidden+1] is fc2.weight [1][width], all row-major
 * fp32 as in a torch state_dict; b[] likewise; mu and sigma are the
 * checkpoint's normalisation vectors [in_features] (mlp.py:133-137).  The
 * weights are copied to the current HIP device in the layout the kernels want
 * (this call and hbt_device_table_create are the only ones that allocate
 * device memory; this one also takes 1 KiB of pinned host memory for
 * hbt_mlp_predict_one).
 * Returns NULL on failure (and sets *err if err is not NULL).
 */
typedef struct hbt_mlp hbt_mlp;
hbt_mlp *hbt_mlp_create(int32_t in_features, int32_t width, int32_t hidden_layers,
                        const float *const *W, const float *const *b, const double *mu,
                        const double *sigma, int *err);

/*
 * Batched RuntimePredictor.predict (analysis/mlp/mlp.py:252-267): rows of raw
 * (un-normalised) features [n][in_features] fp64 — operation features then the
 * four device features — are standardised in fp64, cast to fp32, and run
 * through the network; out[n] receives the fp32 predictions.  Must be called
 * with the device of hbt_mlp_create current.  Large batches go through one
 * fused kernel that runs the whole network with activations on-chip, in whole
 * rounds of 32 rows per compute unit; up to 7168 rows (a single prediction,
 * the operations of one trace, a trace for some devices, or what is left over
 * after the last whole round) each layer is one launch spread over the whole
 * GPU, with activations or partial sums in a scratch buffer that belongs to
 * the handle (2 x 28 MiB, allocated by hbt_mlp_create): calls on ONE handle
 * must therefore not overlap, on any streams; different handles are
 * independent.  Results are reproducible for a given n and position of the
 * row; the paths (per layer with K split over workgroups or waves in several
 * ways by row count, fused) sum in different orders and agree to fp32
 * rounding.
 */
int hbt_mlp_forward(hbt_mlp *mlp, const double *raw_features, int64_t n, float *out,
                    void *hip_stream);
void hbt_mlp_destroy(hbt_mlp *mlp);

/*
 * One prediction from a row in HOST memory, start to finish: the reference's
 * RuntimePredictor.predict (analysis/mlp/mlp.py:252-267), which Predictor calls
 * twice per MLP-predicted operation (analysis/predictor.py:177-180), as one C
 * call.  raw_row [in_features] and out are HOST memory.  The row goes through
 * a pinned, device-visible block of the handle (1 KiB, allocated by
 * hbt_mlp_create), the per-layer kernels of hbt_mlp_forward read it and write
 * the prediction there, and the call waits for `hip_stream` before it returns:
 * about 40 us of GPU time, launch-bound.  The result is bit-identical to
 * hbt_mlp_forward with n = 1.  Uses the handle's scratch like hbt_mlp_forward:
 * the call must not overlap other calls on the same handle from other streams;
 * concurrent hbt_mlp_predict_one calls on one handle are serialised inside the
 * library.  `hip_stream` must not be under graph capture (HBT_EINVAL).  Must be
 * called with the device of hbt_mlp_create current.
 */
int hbt_mlp_predict_one(hbt_mlp *mlp, const double *raw_row, float *out, void *hip_stream);

/*
 * hbt_mlp_forward for callers that cannot allocate device memory or tolerate a
 * library that does: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  The same
 * per-layer kernels as hbt_mlp_forward runs for such row counts (and therefore
 * bit-identical results), but their scratch (activations or partial sums
 * between the layer launches) lives in a static device array of the library, 2
 * x 4 MiB per GPU for the life of the process, not in memory of the handle; the
 * call allocates and frees nothing.  n > HBT_MLP_STATIC_MAX_ROWS returns
 * HBT_ESIZE.  All calls on one GPU share that array, whatever handle or stream
 * they use: calls that overlap on one GPU race; calls that follow each other on
 * one stream, or are otherwise ordered, are fine (nothing is carried over from
 * one call to the next).  The first call on a device looks the array's address
 * up (hipGetSymbolAddress), so make it outside any graph capture.  Must be
 * called with the device of hbt_mlp_create current.
 */
#define HBT_MLP_STATIC_MAX_ROWS 1024
int hbt_mlp_forward_static(hbt_mlp *mlp, const double *raw_features, int64_t n, float *out,
                           void *hip_stream);

/*
 * Calibration of the GPU this process runs on.  Not part of the prediction
 * path: these calls allocate their own scratch memory, use the default stream
 * and synchronise.
 *
 * hbt_local_device_spec fills `out` (host) from hipDeviceProp_t, the fields the
 * reference's device_info tool prints from cudaDeviceProp
 * (cpp/src/device_info.cpp:16-30), plus bandwidth, clock and vector-fp32 peak
 * derived from the reported clocks; `name` (host, nullable) receives the device
 * name.  The compute capability is HIP's, so the spec is a description, not an
 * input the occupancy model accepts as is.
 *
 * hbt_measure_fp32_fma_gflops times a kernel of independent fp32 FMAs, the
 * role of the reference's flop_test kernel (cpp/src/cuda/diagnostics.cu:9-25,
 * tools/device-metadata/measure_peak_flops.py:10-18); hbt_measure_fp32_mfma_gflops
 * does the same with v_mfma_f32_32x32x2_f32; hbt_measure_copy_gbps times a
 * device-to-device copy of `bytes` (read + write counted);
 * hbt_measure_record_stream_gbps times a kernel that performs the loads and
 * stores of hbt_wave_scale on n records (same columns, same access pattern) and
 * no arithmetic, `launches` times after `warmup` untimed ones, and reports
 * 68 bytes per record over the launch time: the data-movement ceiling the
 * wave-scaling kernel can be held against at that size.
 * hbt_measure_record_stream_multi_gbps does the same for a launch with n_dest
 * destinations (the record read once, 13 bytes written per destination to
 * that destination's rows, the origin occupancy once) and reports 52 + 4 + 13
 * x n_dest bytes per record over the launch time.
 */
int hbt_local_device_spec(int device, hbt_device_spec *out, char *name, size_t name_len);
int hbt_measure_fp32_fma_gflops(int iters, double *out_gflops);
int hbt_measure_fp32_mfma_gflops(int iters, double *out_gflops);
int hbt_measure_copy_gbps(size_t bytes, double *out_gbps);
int hbt_measure_record_stream_gbps(int64_t n, int warmup, int launches, double *out_gbps);
int hbt_measure_record_stream_multi_gbps(int64_t n, int32_t n_dest, int warmup, int launches,
                                         double *out_gbps);

#ifdef __cplusplus
}
#endif
#endif /* HABITAT_MI_H_ */
