// Per-operation MLP inference on gfx950: the whole network in one kernel.
//
// Network (analyzer/habitat/analysis/mlp/mlp.py:17-109): fc1 (F -> W), ReLU,
// `hidden` x [Linear(W, W), ReLU], fc2 (W -> 1), with W = 1024.  Input rows are
// standardised as RuntimePredictor.predict does (mlp.py:258-264): (x - mu) /
// sigma in fp64, then cast to fp32.
//
// Design.  A workgroup owns 32 input rows for the whole chain.  Their
// activations (32 x 1024 fp32 = 128 KiB) live in LDS and never touch HBM; the
// only global traffic in steady state is the weight stream, which every
// workgroup reads in the same order and therefore mostly finds in L2.  A layer
// is computed transposed, Out^T[n][m] = sum_k W[n][k] * Act[m][k], with
// v_mfma_f32_32x32x2_f32: the A operand is a 32(n) x 2(k) weight fragment, the
// B operand a 2(k) x 32(m) activation fragment.  The 32 n-tiles of a layer are
// split over the waves; a wave keeps its slice of the output in accumulator
// registers for the whole K loop and only then, after a barrier, overwrites the
// LDS activations in place (bias, staged in LDS during the K loop, and ReLU are
// applied on the way out).
//
// Weights are repacked once, at hbt_mlp_create, so that a wave's fragment for
// 8 consecutive k is one fully coalesced 1 KiB load (16 B per lane) straight
// into the registers the MFMA reads: index [wave][layer][k/8][tile][lane][4]
// holds W_layer[32*tile_global + lane%32][8*(k/8) + 4*(lane/32) + e].  For one
// wave the k-groups of all layers form one contiguous stream, so the prefetch
// ring runs across layer boundaries: the next layer's first weights are already
// in flight while this layer's results are written back.  The matching
// activation fragment is one ds_read_b128 of Act[lane%32][8*(k/8) + 4*(lane/32) ..+3];
// rows are padded by 4 floats so those reads are bank-conflict free.
//
// FLOPs per row: 2 * (F*1024 + hidden*1024^2 + 1024); bound: fp32 MFMA rate.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/habitat_mi.h"
#include "wave_scale.h"

namespace hbt {

namespace {

using u32x4 = unsigned int __attribute__((ext_vector_type(4)));
using f32x2 = float __attribute__((ext_vector_type(2)));
using f32x4 = float __attribute__((ext_vector_type(4)));
using f32x16 = float __attribute__((ext_vector_type(16)));

// ReLU that hands a NaN on, as torch's does (a feature that is NaN or infinite,
// or a zero sigma, must give a NaN prediction as in the reference); the
// hardware's max would return the other operand, 0.
__device__ __forceinline__ float relu(float v) { return v < 0.f ? 0.f : v; }

constexpr int kWidth = 1024;      // hidden width the kernel is built for
constexpr int kRows = 32;         // rows per workgroup (one MFMA tile of m)
constexpr int kStride = kWidth + 4;  // LDS row stride in floats
constexpr int kMaxInPadded = 64;  // in_features padded to a multiple of 32, at most this

struct MlpArgs {
  const double* raw;     // [n][in_features]
  float* out;            // [n]
  int64_t n;
  int32_t in_features;
  int32_t in_padded;     // multiple of 32
  int32_t hidden;
  const double* mu;      // [in_features]
  const double* sigma;   // [in_features]
  const float* w_stream; // packed weights [waves][groups of all layers][tpw][64][4]
  const float* bias;     // [(hidden + 1)][kWidth]: fc1 bias, then hidden biases
  const float* w_last;   // fc2.weight [kWidth]
  float b_last;
};

// Fragments travel through a ring of four register slots.  Weight fragments are
// indexed by the wave's global k-group number (all layers, one stream) and are
// loaded three groups ahead, also across a layer boundary; activation
// fragments are loaded from LDS three groups ahead within the layer.
template <int TPW>
struct Ring {
  f32x4 w[4][TPW];
  f32x4 x[4];
};

// The wave's weight stream as a buffer resource: a load then takes the stream's
// base from scalar registers, the k-group's offset as a scalar and the lane's
// 16 bytes as one 32-bit register, with no 64-bit address arithmetic.
struct WeightStream {
  __amdgpu_buffer_rsrc_t rsrc;
  int lane_bytes;  // 16 * lane
};

__device__ __forceinline__ WeightStream weight_stream(const f32x4* stream, int64_t bytes,
                                                      int lane) {
  WeightStream w;
  w.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<f32x4*>(stream), 0, (int)bytes, 0x00020000);
  w.lane_bytes = 16 * lane;
  return w;
}

template <int TPW, int SLOT>
__device__ __forceinline__ void ring_load_w(Ring<TPW>& r, const WeightStream& stream, int group,
                                            int lane) {
  const int group_bytes = group * (TPW * 64 * 16);
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(stream.rsrc, stream.lane_bytes + t * 1024,
                                                          group_bytes, 0);
    r.w[SLOT][t] = __builtin_bit_cast(f32x4, v);
  }
}

template <int TPW, int SLOT>
__device__ __forceinline__ void ring_load_x(Ring<TPW>& r, const float* act_lane, int g) {
  r.x[SLOT] = *reinterpret_cast<const f32x4*>(act_lane + 8 * g);
}

template <int TPW, int SLOT>
__device__ __forceinline__ void ring_mfma(const Ring<TPW>& r, f32x16 (&acc)[TPW]) {
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int t = 0; t < TPW; ++t)
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(r.w[SLOT][t][e], r.x[SLOT][e], acc[t], 0, 0, 0);
}

// One layer's K loop: kg groups of 8 k (a multiple of 4) starting at global
// group `g0` of the wave's stream; `g_end` is the stream's last valid group.
// On entry ring slots 0..2 hold the weights of groups g0..g0+2.
template <int TPW>
__device__ __forceinline__ void layer_k_loop(Ring<TPW>& r, const WeightStream& stream,
                                             int g0, int kg, int g_end, const float* act_lane,
                                             f32x16 (&acc)[TPW]) {
  const int lane = threadIdx.x & 63;
  const int last = kg - 1;
  ring_load_x<TPW, 0>(r, act_lane, 0);
  ring_load_x<TPW, 1>(r, act_lane, min(1, last));
  ring_load_x<TPW, 2>(r, act_lane, min(2, last));
  for (int j = 0; j < kg; j += 4) {
    // The scheduling barriers keep the compiler from sinking a prefetch below
    // the MFMA block it is meant to overlap with.  Weight groups past the end
    // of the stream, and activation groups past the end of the layer, reload
    // the last valid one (unused values).
    ring_load_w<TPW, 3>(r, stream, min(g0 + j + 3, g_end), lane);
    ring_load_x<TPW, 3>(r, act_lane, min(j + 3, last));
    __builtin_amdgcn_sched_barrier(0);
    ring_mfma<TPW, 0>(r, acc);
    __builtin_amdgcn_sched_barrier(0);
    ring_load_w<TPW, 0>(r, stream, min(g0 + j + 4, g_end), lane);
    ring_load_x<TPW, 0>(r, act_lane, min(j + 4, last));
    __builtin_amdgcn_sched_barrier(0);
    ring_mfma<TPW, 1>(r, acc);
    __builtin_amdgcn_sched_barrier(0);
    ring_load_w<TPW, 1>(r, stream, min(g0 + j + 5, g_end), lane);
    ring_load_x<TPW, 1>(r, act_lane, min(j + 5, last));
    __builtin_amdgcn_sched_barrier(0);
    ring_mfma<TPW, 2>(r, acc);
    __builtin_amdgcn_sched_barrier(0);
    ring_load_w<TPW, 2>(r, stream, min(g0 + j + 6, g_end), lane);
    ring_load_x<TPW, 2>(r, act_lane, min(j + 6, last));
    __builtin_amdgcn_sched_barrier(0);
    ring_mfma<TPW, 3>(r, acc);
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64, 1) void mlp_fused_kernel(const MlpArgs a) {
  constexpr int TPW = (kWidth / 32) / WAVES;  // n-tiles per wave
  constexpr int THREADS = WAVES * 64;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* act = lds;                           // [kRows][kStride]
  float* red = lds + kRows * kStride;         // [THREADS / 32][32]
  float* bias_lds = red + (THREADS / 32) * 32;  // [kWidth]
  static_assert(THREADS * 4 == kWidth, "one float4 of bias per thread");

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  const int64_t row0 = (int64_t)blockIdx.x * kRows;

  // ---- stage standardised inputs: act[r][k], zero beyond in_features / n ----
  for (int idx = tid; idx < kRows * a.in_padded; idx += THREADS) {
    const int r = idx / a.in_padded, k = idx - r * a.in_padded;
    float v = 0.f;
    if (k < a.in_features && row0 + r < a.n) {
      const double x = a.raw[(row0 + r) * a.in_features + k];
      v = (float)((x - a.mu[k]) / a.sigma[k]);
    }
    act[r * kStride + k] = v;
  }
  // fc1's bias, where the accumulators will pick it up
  *reinterpret_cast<f32x4*>(bias_lds + 4 * tid) = *reinterpret_cast<const f32x4*>(a.bias + 4 * tid);
  __syncthreads();

  const float* act_lane = act + m * kStride + 4 * h;
  const int tile0 = wave * TPW;  // first n-tile of this wave

  // This wave's weight stream: fc1's groups, then 128 groups per hidden layer.
  const int kg_first = a.in_padded / 8;
  const int groups = kg_first + a.hidden * (kWidth / 8);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int64_t stream_bytes = (int64_t)groups * TPW * 64 * 16;
  const WeightStream stream = weight_stream(
      reinterpret_cast<const f32x4*>(a.w_stream) + (size_t)wave_u * groups * TPW * 64, stream_bytes,
      lane);
  const int g_end = groups - 1;

  Ring<TPW> ring;
  ring_load_w<TPW, 0>(ring, stream, 0, lane);
  ring_load_w<TPW, 1>(ring, stream, min(1, g_end), lane);
  ring_load_w<TPW, 2>(ring, stream, min(2, g_end), lane);

  f32x16 acc[TPW];
  int g0 = 0;
  for (int layer = 0; layer <= a.hidden; ++layer) {
    // The accumulators start at this layer's bias, which the layer before
    // parked in LDS; every thread fetches four values of the next layer's now
    // and parks them after the K loop.  (Adding the bias here instead of in the
    // write-back leaves room there for a ReLU that hands NaNs on, at no more
    // instructions than add and max.)
    const int next_layer = layer < a.hidden ? layer + 1 : layer;
    const f32x4 bias_part =
        *reinterpret_cast<const f32x4*>(a.bias + (size_t)next_layer * kWidth + 4 * tid);
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 b =
            *reinterpret_cast<const f32x4*>(bias_lds + (tile0 + t) * 32 + 8 * g + 4 * h);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[t][4 * g + e] = b[e];
      }

    const int kg = (layer == 0) ? kg_first : kWidth / 8;
    layer_k_loop<TPW>(ring, stream, g0, kg, g_end, act_lane, acc);
    g0 += kg;

    __syncthreads();  // every wave has finished reading this layer's input and bias
    *reinterpret_cast<f32x4*>(bias_lds + 4 * tid) = bias_part;
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = (tile0 + t) * 32 + 8 * g + 4 * h;
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = relu(acc[t][4 * g + e]);
        *reinterpret_cast<f32x4*>(act + m * kStride + n) = o;
      }
    __syncthreads();
  }

  // ---- fc2: out[r] = sum_n act[r][n] * w_last[n] + b_last ----
  {
    constexpr int PARTS = THREADS / 32;
    constexpr int NPP = kWidth / PARTS;
    const int r = tid & 31, part = tid >> 5;
    const float* ap = act + r * kStride + part * NPP;
    const float* wl = a.w_last + part * NPP;
    float s = 0.f;
#pragma unroll 8
    for (int k = 0; k < NPP; k += 4) {
      const f32x4 x = *reinterpret_cast<const f32x4*>(ap + k);
      const f32x4 w = *reinterpret_cast<const f32x4*>(wl + k);
      s = fmaf(x[0], w[0], s);
      s = fmaf(x[1], w[1], s);
      s = fmaf(x[2], w[2], s);
      s = fmaf(x[3], w[3], s);
    }
    red[part * 32 + r] = s;
    __syncthreads();
    if (tid < 32 && row0 + tid < a.n) {
      float total = a.b_last;
#pragma unroll
      for (int p = 0; p < PARTS; ++p) total += red[p * 32 + tid];
      a.out[row0 + tid] = total;
    }
  }
}

// ---------------------------------------------------------------------------
// Up to kLayerMaxRows rows (one prediction, the operations of one trace, a trace
// for some devices): one launch per layer.
//
// The fused kernel gives each workgroup 32 rows and the whole network, so a
// batch of up to 32 rows runs on ONE compute unit, which has to pull all
// 33.6 MB of weights through by itself (about 1 ms), and any batch below 8192
// rows leaves compute units idle for that long.  Here a layer is spread over
// the chip instead, in one of three shapes:
//
//   For a few rows (up to kSplitMaxRows) mlp_layer_kernel with four waves: a
//   workgroup takes one n-tile x one m-tile and an eighth of K (kSplit: 256
//   workgroups per layer), its waves split that eighth, each multiplies its
//   k-groups straight from global memory (no loop, no LDS staging), the waves
//   add their 32 x 32 accumulators through LDS, and the K-partials are written
//   as they are, [split][row][n]; they are summed, biased and rectified by
//   whoever reads them: the next layer's activation load, or the final dot
//   product.
//   Up to kHalfKMaxTiles m-tiles (128 rows) the same kernel with eight waves
//   and K over two workgroups, whose K-partials are stored by k-group (see
//   km_index), like all activations from here on.
//   Above that mlp_layer_tile_kernel: a wave per output tile, see there.
//
// The order of every sum is fixed, so results are reproducible.  Same packed
// weights, same MFMA instruction, same fragment layout as above.
constexpr int kSplit = 8;            // K-partials per hidden layer, up to kSplitMaxRows rows
// Rows up to which K is split over workgroups (the partials' traffic grows with
// the rows; beyond this the whole-K shapes are faster).
constexpr int kSplitMaxRows = 20;
// Largest batch that takes this path: 224 m-tiles, 7 steps of the tile kernel on
// 256 compute units, just under what one round of the fused kernel costs
// whatever it holds.  Tuned on 256 compute units.
constexpr int kLayerMaxRows = 7168;
// m-tiles up to which the eight-wave shape splits K over two workgroups (128
// workgroups or fewer per layer would leave half the compute units idle).
constexpr int kHalfKMaxTiles = 4;
// Input features up to which fc1 of a batch stored by k-group is computed with
// plain FMAs (mlp_first_fma_kernel); the reference's networks have 8 to 12.
constexpr int kFirstFmaMaxIn = 16;
constexpr int kFirstFmaSlices = 8;     // workgroups per m-tile (gridDim.y)
constexpr int kFirstFmaMinTiles = 64;  // m-tiles from which that kernel is used (2048 rows)
constexpr size_t kScratchFloats = (size_t)kLayerMaxRows * kWidth;  // each of two buffers (28 MiB)
static_assert((size_t)kSplit * kRows * kWidth <= kScratchFloats, "the K-partials fit the scratch");

struct LayerArgs {
  const float* w_stream;   // packed weights, see above
  int32_t groups_total;    // k-groups per wave stream (all layers)
  int32_t g0;              // first stream group of this layer
  int32_t kg;              // k-groups of this layer (K / 8)
  int32_t splits;          // K-partials this launch writes (gridDim.y)
  const float* p_in;       // m_pad x kWidth activations, or S_IN such blocks of K-partials
  const float* bias_in;    // [kWidth], bias of the previous layer (with partials)
  const float* bias_out;   // [kWidth], bias of this layer (FINAL)
  const double* raw;       // FIRST: [n][in_features], with mu and sigma
  const double* mu;
  const double* sigma;
  int32_t in_features;
  int64_t n;
  int32_t m_pad;           // rows rounded up to 32
  float* p_out;            // m_pad x kWidth activations (FINAL), else `splits` blocks of partials
  const float* w_first_t;  // fc1.weight transposed, [kFirstFmaMaxIn][kWidth] (mlp_first_fma_kernel)
};

// Outside the split-K shape activations are stored by k-group (KM below): element
// (row, n) at [row / 32][n / 8][row % 32][n % 8], so that the fragment a wave
// loads for one m-tile and k-group, 32 rows x 8 values, is 1 KiB of contiguous
// memory (8 cache lines used whole) where row-major storage spreads it over 32
// lines, 32 bytes of each.
__device__ __forceinline__ size_t km_index(int m_tile, int k_group, int m, int c) {
  return (((size_t)m_tile * (kWidth / 8) + k_group) * kRows + m) * 8 + c;
}

// G k-groups of a wave: the weight fragments of the n-tile and what the
// matching activation fragments are made from (the activations themselves, or
// S_IN K-partials and the bias that goes with them).
template <int G, int S_IN, int NT>
struct LayerFrag {
  f32x4 w[G][NT];
  f32x4 x[G][S_IN > 0 ? S_IN : 1];
  f32x4 bias[S_IN > 0 ? G : 1];
};

// One layer for one m-tile (blockIdx.z), NT n-tiles (blockIdx.x) and one
// K-partial (blockIdx.y of a.splits).  The WAVES waves split the partial's
// k-groups (at most G each); fc1 has fewer, so there each group is checked
// against the wave's count (wave-uniform).
//   FIRST: fc1, from the raw fp64 rows, standardised on the spot.
//   S_IN: 0 = the input holds activations; otherwise it holds that many
//     K-partials, to be summed, biased and rectified on the way in.
//   FINAL: the launch covers all of K (a.splits == 1), so the output is
//     biased and rectified here and the next layer reads activations.
//   PADDED_ROWS: rows past the end of the batch are read like the others (the
//     padded m-tile holds them) instead of being masked; masking saves most of
//     the traffic of a handful of rows, not masking keeps the loads of a full
//     tile free of branches.
//   NT: n-tiles per workgroup (blockIdx.x counts groups of NT); an activation
//     fragment then serves NT MFMAs.
//   DEPTH: k-groups whose loads are kept in flight ahead of the MFMAs; 0 leaves
//     the placement to the compiler (each group's loads next to its MFMAs, one
//     trip to memory after the other, which resident workgroups hide from each
//     other).
//   KM: activations (read, unless FIRST, and written) are stored by k-group.
//   S_OUT: K-partials this launch writes (a.splits; 1 with FINAL).
// The instantiations in use: fc1 (FIRST, FINAL, 4 waves) with row-major or
// k-group output; hidden layers with kSplit K-partials in and out (4 waves,
// rows masked); hidden layers with two K-partials in and out (8 waves, DEPTH 2,
// KM).
template <bool FIRST, int S_IN, bool FINAL, int WAVES, bool PADDED_ROWS, int DEPTH, int NT = 1,
          bool KM = false, int S_OUT = (FINAL ? 1 : kSplit)>
__global__ __launch_bounds__(WAVES * 64) void mlp_layer_kernel(const LayerArgs a) {
  static_assert((S_OUT == 1) == FINAL, "one K-partial is the whole sum");
  static_assert(8 % NT == 0, "a workgroup's n-tiles lie in one wave stream of the packed weights");
  static_assert(S_IN == 0 || !FINAL, "K-partials go in and come out together");
  static_assert(WAVES == 4 || WAVES == 8, "the reduction below is written for these");
  constexpr int G = FIRST ? kMaxInPadded / 8 / WAVES : kWidth / 8 / WAVES / S_OUT;
  __shared__ float red[WAVES][NT][16][64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 31, h = lane >> 5;
  const int split = blockIdx.y;
  // rows past the end of the batch: computed (from zeros, or from what the
  // padded m-tile holds) and stored within the padded m-tile, never read out
  const int64_t row = (int64_t)blockIdx.z * kRows + m;
  const bool row_ok = PADDED_ROWS || row < a.n;

  // this wave's k-groups: [first, first + count) of the layer's kg
  const int per_split = a.kg / a.splits;
  const int per_wave = (per_split + WAVES - 1) / WAVES;
  const int first = split * per_split + wave * per_wave;
  int count = per_split - wave * per_wave;
  count = count < 0 ? 0 : (count > per_wave ? per_wave : count);

  // n-tile of the layer -> (stream of the fused kernel's wave, slot in its group)
  const int tile = blockIdx.x * NT;  // the first of the workgroup's NT
  const f32x4* w_lane = reinterpret_cast<const f32x4*>(a.w_stream) +
                        ((size_t)(tile >> 3) * a.groups_total + a.g0) * (8 * 64) +
                        (tile & 7) * 64 + lane;

  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  LayerFrag<G, S_IN, NT> f;
  // Hidden layers fetch weights, activations (or K-partials) and bias through
  // buffer loads: bases in scalar registers, the k-group's offset a scalar, one
  // 32-bit register of lane offset each, no 64-bit address arithmetic.  A lane
  // whose row is past the end of the batch gets an offset beyond the buffer
  // instead of a branch around the load: such a load returns zeros.
  constexpr bool BUFFER = !FIRST;
  __amdgpu_buffer_rsrc_t w_rsrc, x_rsrc, b_rsrc;
  int w_lane_bytes = 0, x_lane_bytes = 0, w_base_bytes = 0;
  const int split_bytes = a.m_pad * (kWidth * 4);  // one K-partial, or the activations
  if (BUFFER) {
    w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.w_stream), 0,
                                               4 * a.groups_total * (8 * 64 * 16), 0x00020000);
    x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.p_in), 0,
                                               (S_IN > 0 ? S_IN : 1) * split_bytes, 0x00020000);
    b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.bias_in), 0, kWidth * 4,
                                               0x00020000);
    w_lane_bytes = ((tile & 7) * 64 + lane) * 16;
    w_base_bytes = ((tile >> 3) * a.groups_total + a.g0) * (8 * 64 * 16);
    if (KM) x_lane_bytes = row_ok ? (int)km_index(blockIdx.z, 0, m, 4 * h) * 4 : 0x7fffff00;
    else x_lane_bytes = row_ok ? (int)row * (kWidth * 4) + 16 * h : 0x7fffff00;
  }
  auto load_group = [&](int j) {
    if (!FIRST || j < count) {
      const int gl = first + j;  // layer-local group
      if (BUFFER) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
          f.w[j][t] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
              w_rsrc, w_lane_bytes + t * 1024, w_base_bytes + gl * (8 * 64 * 16), 0));
#pragma unroll
        for (int s = 0; s < (S_IN > 0 ? S_IN : 1); ++s)
          f.x[j][s] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
              x_rsrc, x_lane_bytes, s * split_bytes + gl * (KM ? kRows * 32 : 32), 0));
        if (S_IN > 0)
          f.bias[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
              b_rsrc, 16 * h, gl * 32, 0));
        return;
      }
      // fc1: a few groups, the raw fp64 features standardised on the spot
#pragma unroll
      for (int t = 0; t < NT; ++t) f.w[j][t] = w_lane[(size_t)gl * (8 * 64) + t * 64];
      const int k = 8 * gl + 4 * h;
      f32x4 v = zero;
      if (row_ok) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (k + e < a.in_features)
            v[e] = (float)((a.raw[row * a.in_features + k + e] - a.mu[k + e]) / a.sigma[k + e]);
      }
      f.x[j][0] = v;
    }
  };

  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  auto mfma_group = [&](int j) {
    if (!FIRST || j < count) {
      f32x4 v = f.x[j][0];
      if (S_IN > 0) {
        // the previous layer's K-partials, in their fixed order, then bias and ReLU
        v = f.bias[j];
#pragma unroll
        for (int s = 0; s < S_IN; ++s) v += f.x[j][s];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = relu(v[e]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.w[j][t][e], v[e], acc[t], 0, 0, 0);
    }
  };

  if (DEPTH == 0) {
    // the compiler places the loads: each group's next to its MFMAs, one trip
    // to memory after the other, which resident workgroups hide from each other
#pragma unroll
    for (int j = 0; j < G; ++j) load_group(j);
#pragma unroll
    for (int j = 0; j < G; ++j) mfma_group(j);
  } else {
    // DEPTH groups in flight ahead of the MFMAs
#pragma unroll
    for (int j = 0; j < (DEPTH < G ? DEPTH : G); ++j) load_group(j);
#pragma unroll
    for (int j = 0; j < G; ++j) {
      if (j + DEPTH < G) load_group(j + DEPTH);
      __builtin_amdgcn_sched_barrier(0);
      mfma_group(j);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) red[wave][t][r][lane] = acc[t][r];
  __syncthreads();
  // thread (wave, lane) adds the waves' registers R*wave .. R*wave+R-1, in wave
  // order: accumulator register 4g + e of lane (m, h) is output n = 8g + 4h + e
  // of row m
  constexpr int R = 16 / WAVES;
  const int r0 = R * wave;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n0 = (tile + t) * 32 + 8 * (r0 >> 2) + 4 * h + (r0 & 3);
    float o[R];
#pragma unroll
    for (int e = 0; e < R; ++e) {
      float sum = red[0][t][r0 + e][lane];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) sum += red[w][t][r0 + e][lane];
      if (FINAL) sum = relu(sum + a.bias_out[n0 + e]);
      o[e] = sum;
    }
    float* dst = a.p_out + ((size_t)split * a.m_pad + (size_t)blockIdx.z * kRows + m) * kWidth + n0;
    if (KM)
      dst = a.p_out + (size_t)split * a.m_pad * kWidth + km_index(blockIdx.z, n0 >> 3, m, n0 & 7);
    if constexpr (R == 4) {
      *reinterpret_cast<f32x4*>(dst) = f32x4{o[0], o[1], o[2], o[3]};
    } else {
      *reinterpret_cast<f32x2*>(dst) = f32x2{o[0], o[1]};
    }
  }
}

// One hidden layer with a wave owning ONE output tile (32 rows x 32 outputs) for
// 1 / KS of K: no loop over tiles, accumulators in place for the wave's whole
// run of k-groups, fragments through a ring of SLOTS register slots (loads
// SLOTS - 1 k-groups ahead of their MFMAs, one 16-byte buffer load per lane and
// fragment, 1 KiB of contiguous memory per wave), no LDS staging.  A workgroup
// is four waves:
//   KS = 1   2 m-tiles x 2 n-tiles, no reduction, no barrier
//   KS = 2   1 m-tile x 2 n-tiles, two halves of K
//   KS = 4   1 m-tile x 1 n-tile, four quarters of K
// With KS > 1 the waves of a tile add their accumulators through LDS in wave
// order, each finishing 16 / KS of the tile's registers.  A tile for the whole
// of K is 13.7 us of one SIMD's matrix core, so a layer takes that times the
// tiles per SIMD, rounded up: KS trades a finer rounding (1024 / KS rows per
// step) against shorter runs per wave.  Activations in and out are stored by
// k-group (km_index); bias and ReLU are applied on the way out.
template <int KS, int SLOTS>
__global__ __launch_bounds__(256) void mlp_layer_tile_kernel(const LayerArgs a) {
  static_assert(KS == 1 || KS == 2 || KS == 4, "four waves per workgroup");
  constexpr int kGroups = kWidth / 8 / KS;  // per wave
  static_assert(kGroups % SLOTS == 0, "the ring turns a whole number of times");
  __shared__ float red[KS > 1 ? 4 : 1][16][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int m = lane & 31, h = lane >> 5;
  const int m_tiles = a.m_pad / kRows;
  // wave -> (part of K, n-tile, m-tile)
  const int k_part = wave % KS;
  const int n_tile = KS == 4 ? (int)blockIdx.x : (int)blockIdx.x * 2 + (KS == 2 ? wave >> 1 : wave & 1);
  const int m_tile = KS == 1 ? (int)blockIdx.y * 2 + (wave >> 1) : (int)blockIdx.y;
  if (m_tile >= m_tiles) return;  // KS = 1 only (no barrier there): an odd number of m-tiles

  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(a.w_stream), 0, 4 * a.groups_total * (8 * 64 * 16), 0x00020000);
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(a.p_in), 0, a.m_pad * (kWidth * 4), 0x00020000);
  const int first = k_part * kGroups;  // the wave's first k-group of the layer
  const int w_lane_bytes = ((n_tile & 7) * 64 + lane) * 16;
  const int w_base_bytes = ((n_tile >> 3) * a.groups_total + a.g0 + first) * (8 * 64 * 16);
  const int x_lane_bytes = m_tile * (kWidth * kRows * 4) + m * 32 + 16 * h;
  const int x_base_bytes = first * (kRows * 32);

  f32x4 w[SLOTS], x[SLOTS];
  auto load = [&](int slot, int group) {
    w[slot] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
        w_rsrc, w_lane_bytes, w_base_bytes + group * (8 * 64 * 16), 0));
    x[slot] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
        x_rsrc, x_lane_bytes, x_base_bytes + group * (kRows * 32), 0));
  };

  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
  for (int s = 0; s < SLOTS - 1; ++s) load(s, s);
  for (int j = 0; j < kGroups; j += SLOTS) {
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      // past the wave's last group the last one is fetched again (unused)
      const int ahead = j + s + SLOTS - 1;
      load((s + SLOTS - 1) % SLOTS, ahead < kGroups ? ahead : kGroups - 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w[s][e], x[s][e], acc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // accumulator register 4g + e of lane (m, h) is output n = 8g + 4h + e of row m
  auto finish = [&](int g, const f32x4 sum) {
    const int n0 = n_tile * 32 + 8 * g + 4 * h;
    const f32x4 bias = *reinterpret_cast<const f32x4*>(a.bias_out + n0);
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = relu(sum[e] + bias[e]);
    *reinterpret_cast<f32x4*>(a.p_out + km_index(m_tile, n0 >> 3, m, 4 * h)) = o;
  };
  if constexpr (KS == 1) {
#pragma unroll
    for (int g = 0; g < 4; ++g) finish(g, f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]});
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) red[wave][r][lane] = acc[r];
    __syncthreads();
    // the KS waves of a tile are wave0 .. wave0 + KS - 1; this one finishes the
    // register groups g0 .. g0 + 4 / KS - 1, adding the parts of K in wave order
    const int wave0 = wave - k_part;
#pragma unroll
    for (int i = 0; i < 4 / KS; ++i) {
      const int g = k_part * (4 / KS) + i;
      f32x4 sum;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = red[wave0][4 * g + e][lane];
#pragma unroll
        for (int p = 1; p < KS; ++p) v += red[wave0 + p][4 * g + e][lane];
        sum[e] = v;
      }
      finish(g, sum);
    }
  }
}

// fc1 for large batches stored by k-group, with at most kFirstFmaMaxIn input
// features: K is a dozen, so the layer is its 4 KiB-per-row write and little
// else, and plain FMAs from LDS do it without the matrix cores.  A workgroup
// takes one m-tile and an eighth of the outputs: it standardises the m-tile's
// raw fp64 rows (the 4-wave MFMA kernel does that once per n-tile, 32 times per
// row, this one 8 times), stages its slice of the transposed weights in LDS,
// and each lane (row m, half h) then produces four consecutive outputs per
// k-group of the next layer, 1 KiB of contiguous memory per wave and store.
// Sum order: bias, then k ascending.  Faster than the MFMA kernel from about
// 2048 rows (kFirstFmaMinTiles), slower below.
__global__ __launch_bounds__(256) void mlp_first_fma_kernel(const LayerArgs a) {
  __shared__ float xs[kRows][kFirstFmaMaxIn + 1];
  __shared__ __attribute__((aligned(16))) float wl[kFirstFmaMaxIn * (kWidth / kFirstFmaSlices)];  // [k][n of the slice]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  const int m_tile = blockIdx.x;
  constexpr int slice_n = kWidth / kFirstFmaSlices;  // outputs of this workgroup
  const int n_base = (int)blockIdx.y * slice_n;
  for (int idx = tid; idx < kRows * kFirstFmaMaxIn; idx += 256) {
    const int r = idx / kFirstFmaMaxIn, k = idx - r * kFirstFmaMaxIn;
    const int64_t row = (int64_t)m_tile * kRows + r;
    float v = 0.f;
    if (k < a.in_features && row < a.n)
      v = (float)((a.raw[row * a.in_features + k] - a.mu[k]) / a.sigma[k]);
    xs[r][k] = v;
  }
  for (int idx = tid; idx < a.in_features * (slice_n / 4); idx += 256) {
    const int k = idx / (slice_n / 4), c = idx - k * (slice_n / 4);
    *reinterpret_cast<f32x4*>(wl + k * slice_n + 4 * c) =
        *reinterpret_cast<const f32x4*>(a.w_first_t + (size_t)k * kWidth + n_base + 4 * c);
  }
  __syncthreads();
  float x[kFirstFmaMaxIn];
#pragma unroll
  for (int k = 0; k < kFirstFmaMaxIn; ++k) x[k] = xs[m][k];
  for (int g = wave; g < slice_n / 8; g += 4) {
    const int local = 8 * g + 4 * h, n0 = n_base + local;
    f32x4 o = *reinterpret_cast<const f32x4*>(a.bias_out + n0);
#pragma unroll
    for (int k = 0; k < kFirstFmaMaxIn; ++k)
      if (k < a.in_features) {
        const f32x4 w = *reinterpret_cast<const f32x4*>(wl + k * slice_n + local);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = fmaf(x[k], w[e], o[e]);
      }
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = relu(o[e]);
    *reinterpret_cast<f32x4*>(a.p_out + km_index(m_tile, n0 >> 3, m, 4 * h)) = o;
  }
}

struct LastArgs {
  const float* p_in;     // m_pad x kWidth activations, or S_IN such blocks of K-partials
  const float* bias_in;  // [kWidth], bias of the last hidden layer (with partials)
  const float* w_last;   // [kWidth]
  float b_last;
  int64_t n;
  int32_t m_pad;
  float* out;            // [n]
  // hbt_mlp_predict_one: once out[0] is written, done_value is stored here
  // (host-visible memory) so that the caller need not wait for the stream
  uint32_t* done_flag;   // nullable
  uint32_t done_value;
};

// Publishes `value` to a waiting host thread after this thread's earlier stores.
__device__ __forceinline__ void publish_done(uint32_t* flag, uint32_t value) {
  __threadfence_system();
  __hip_atomic_store(flag, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// fc2 after the per-layer kernels: one wavefront per row.  S_IN as in mlp_layer_kernel.
template <int S_IN>
__global__ __launch_bounds__(256) void mlp_last_kernel(const LastArgs a) {
  constexpr int P = S_IN > 0 ? S_IN : 1;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.n) return;
  f32x4 part[kWidth / 256][P];
#pragma unroll
  for (int i = 0; i < kWidth / 256; ++i)
#pragma unroll
    for (int s = 0; s < P; ++s)
      part[i][s] = *reinterpret_cast<const f32x4*>(
          a.p_in + ((size_t)s * a.m_pad + row) * kWidth + 256 * i + 4 * lane);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kWidth / 256; ++i) {
    const int k = 256 * i + 4 * lane;
    f32x4 v = part[i][0];
    if (S_IN > 0) {
      v = *reinterpret_cast<const f32x4*>(a.bias_in + k);
#pragma unroll
      for (int s = 0; s < S_IN; ++s) v += part[i][s];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = relu(v[e]);
    }
    const f32x4 wl = *reinterpret_cast<const f32x4*>(a.w_last + k);
#pragma unroll
    for (int e = 0; e < 4; ++e) sum = fmaf(v[e], wl[e], sum);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off);
  if (lane == 0) {
    a.out[row] = sum + a.b_last;
    if (a.done_flag != nullptr && row == 0) publish_done(a.done_flag, a.done_value);
  }
}

// fc2 from activations stored by k-group: one workgroup per m-tile, its four
// waves take a quarter of K each; lane (m, h) reads 16 bytes of its row per
// k-group, so that a wave's load is the k-group's contiguous 1 KiB.
template <int S_IN>
__global__ __launch_bounds__(256) void mlp_last_km_kernel(const LastArgs a) {
  constexpr int kGroupsPerWave = kWidth / 8 / 4;
  __shared__ float part[4][kRows];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = lane & 31, h = lane >> 5;
  const f32x4* x = reinterpret_cast<const f32x4*>(
      a.p_in + km_index(blockIdx.x, wave * kGroupsPerWave, m, 4 * h));
  const f32x4* wl = reinterpret_cast<const f32x4*>(a.w_last + 8 * wave * kGroupsPerWave + 4 * h);
  constexpr int P = S_IN > 0 ? S_IN : 1;
  constexpr int kStep = 8;  // k-groups whose loads are issued together
  float sum = 0.f;
  for (int g0 = 0; g0 < kGroupsPerWave; g0 += kStep) {
    f32x4 v[kStep][P], w[kStep], bias[kStep];
#pragma unroll
    for (int j = 0; j < kStep; ++j) {
#pragma unroll
      for (int s = 0; s < P; ++s)
        v[j][s] = x[(size_t)(g0 + j) * (kRows * 2) + (size_t)s * a.m_pad * (kWidth / 4)];
      w[j] = wl[2 * (g0 + j)];
      if (S_IN > 0)
        bias[j] = *reinterpret_cast<const f32x4*>(
            a.bias_in + 8 * (wave * kGroupsPerWave + g0 + j) + 4 * h);
    }
    __builtin_amdgcn_sched_barrier(0);  // all of the step's loads before its arithmetic
#pragma unroll
    for (int j = 0; j < kStep; ++j) {
      f32x4 act = v[j][0];
      if (S_IN > 0) {
        // K-partials in their fixed order, then bias and ReLU
        act = bias[j];
#pragma unroll
        for (int s = 0; s < S_IN; ++s) act += v[j][s];
#pragma unroll
        for (int e = 0; e < 4; ++e) act[e] = relu(act[e]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) sum = fmaf(act[e], w[j][e], sum);
    }
  }
  sum += __shfl_xor(sum, 32);
  if (h == 0) part[wave][m] = sum;
  __syncthreads();
  const int64_t row = (int64_t)blockIdx.x * kRows + threadIdx.x;
  if (threadIdx.x < kRows && row < a.n)
    a.out[row] = ((part[0][threadIdx.x] + part[1][threadIdx.x]) +
                  (part[2][threadIdx.x] + part[3][threadIdx.x])) + a.b_last;
}

constexpr size_t kOneOutOffset = 512;   // hbt_mlp_predict_one's result within its staging block
constexpr size_t kOneDoneOffset = 768;  // and the call number the last kernel publishes after it
constexpr size_t kOneBytes = 1024;
static_assert(kMaxInPadded * sizeof(double) <= kOneOutOffset, "a raw row fits below the result");

constexpr int kWaves = 4;  // one wave per SIMD: fewer, longer MFMA runs between load bursts than with two
constexpr size_t kLdsBytes =
    (size_t)(kRows * kStride + (kWaves * 64 / 32) * 32 + kWidth) * sizeof(float);

}  // namespace

}  // namespace hbt

struct hbt_mlp {
  int32_t in_features, in_padded, width, hidden;
  int device;
  int compute_units;   // of that device: the fused kernel runs one workgroup on each
  void* blob;          // one device allocation holding everything below
  const double* mu;
  const double* sigma;
  const float* w_stream;
  const float* bias;
  const float* w_last;
  const float* w_first_t;  // fc1.weight transposed [kFirstFmaMaxIn][width]; null above that many inputs
  float b_last;
  float* scratch[2];   // per-layer path: two buffers of kScratchFloats activations or partials
  // hbt_mlp_predict_one: a pinned, device-visible block (one raw row in, one
  // prediction out at kOneOutOffset) and the lock that serialises its callers
  unsigned char* one_host;
  unsigned char* one_device;
  uint32_t one_calls;      // numbers the calls: the value the kernel publishes
  std::mutex one_lock;
};

namespace hbt {
namespace {

// Repack one layer, a row-major [kWidth][k_in] weight matrix (k_in <= k_padded),
// into the per-wave streams: wave w's copy goes to dst + w * wave_stride as
// [k_padded/8][tpw][64 lanes][4].
void pack_layer(const float* W, int k_in, int k_padded, int waves, float* dst, size_t wave_stride) {
  const int tpw = (kWidth / 32) / waves;
  const int kg = k_padded / 8;
  for (int w = 0; w < waves; ++w)
    for (int j = 0; j < kg; ++j)
      for (int t = 0; t < tpw; ++t)
        for (int lane = 0; lane < 64; ++lane)
          for (int e = 0; e < 4; ++e) {
            const int n = (w * tpw + t) * 32 + (lane & 31);
            const int k = 8 * j + 4 * (lane >> 5) + e;
            const float v = (k < k_in) ? W[(size_t)n * k_in + k] : 0.f;
            dst[(size_t)w * wave_stride + (((size_t)j * tpw + t) * 64 + lane) * 4 + e] = v;
          }
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace
}  // namespace hbt

// Scratch memory of hbt_mlp_forward_static: the per-layer path's two buffers
// for up to HBT_MLP_STATIC_MAX_ROWS rows, part of the code object (each GPU the
// library runs on holds its own copy until the process ends).  In host code
// this name is only a handle for hipGetSymbolAddress: kernels and copies get
// the per-device address kept in static_scratch_of().
constexpr int kStaticMaxRows = HBT_MLP_STATIC_MAX_ROWS;
constexpr size_t kStaticFloats = (size_t)kStaticMaxRows * hbt::kWidth;  // each of the two
static_assert((size_t)hbt::kSplit * hbt::kRows * hbt::kWidth <= kStaticFloats &&
                  2 * (size_t)hbt::kHalfKMaxTiles * hbt::kRows * hbt::kWidth <= kStaticFloats &&
                  kStaticMaxRows % hbt::kRows == 0 && kStaticMaxRows <= hbt::kLayerMaxRows,
              "the K-partials of the small shapes and the padded rows fit the static scratch");
static __device__ __align__(256) float scratch[2 * kStaticFloats];

namespace {

// The device address of `scratch` on the current device, looked up once per
// device (nullptr and *rc set when the runtime refuses).
constexpr int kMaxDevices = 64;
float* static_scratch_of(int device, int* rc) {
  static std::mutex lock;
  static float* address[kMaxDevices] = {};
  *rc = HBT_OK;
  if (device < 0 || device >= kMaxDevices) {
    *rc = HBT_ESIZE;
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(lock);
  if (address[device] == nullptr) {
    float* ptr = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess ||
        ptr == nullptr) {
      (void)hipGetLastError();
      *rc = HBT_EHIP;
      return nullptr;
    }
    address[device] = ptr;
  }
  return address[device];
}

// Into how many parts mlp_layer_tile_kernel splits K for a batch of m_tiles
// m-tiles.  A layer is 32 x m_tiles output tiles on 4 x compute_units SIMDs and
// takes ceil(32 m_tiles KS / SIMDs) steps of 1 / KS of a whole-K tile's time:
// the finest split is never worse by that count, but a wave's run gets shorter
// (a run of 32 k-groups is 3.4 us of MFMAs, next to about a microsecond until
// its first fragments arrive) and all workgroups should be resident at once (8
// per compute unit), so the coarsest split among the cheapest is taken: on 256
// compute units KS = 2 up to 4096 rows and KS = 4 up to 2048.
int tile_k_parts(int m_tiles, int compute_units) {
  const int simds = 4 * compute_units;  // 1024 on the GPU the thresholds were measured on
  // steps a layer takes with K in `ks` parts, in quarters of a whole-K step
  auto cost = [&](int ks) { return (32 * m_tiles * ks + simds - 1) / simds * (4 / ks); };
  int best = 1, best_cost = cost(1);
  if (m_tiles <= simds / 8 && cost(2) < best_cost) {
    best = 2;
    best_cost = cost(2);
  }
  if (m_tiles <= simds / 16 && cost(4) < best_cost) best = 4;
  return best;
}

// One launch per layer for n <= kLayerMaxRows rows, through two buffers of
// activations or K-partials (each at least max(n rounded up to 32, kSplit * 32)
// x kWidth floats): the handle's, or the library's static ones.
int forward_layers(hbt_mlp* mlp, const double* raw_features, int64_t n, float* out,
                   float* const buffers[2], hipStream_t stream, uint32_t* done_flag = nullptr,
                   uint32_t done_value = 0) {
  using namespace hbt;
  const int m_tiles = (int)((n + kRows - 1) / kRows);
  const bool split_k = n <= kSplitMaxRows;
  // with a few m-tiles the eight-wave shape splits K in two as well
  const int ks = (!split_k && m_tiles <= kHalfKMaxTiles) ? 2 : 1;
  LayerArgs l{};
  l.w_stream = mlp->w_stream;
  l.groups_total = mlp->in_padded / 8 + mlp->hidden * (kWidth / 8);
  l.raw = raw_features; l.mu = mlp->mu; l.sigma = mlp->sigma;
  l.in_features = mlp->in_features;
  l.n = n;
  l.m_pad = m_tiles * kRows;
  l.w_first_t = mlp->w_first_t;
  bool partials = false;
  const float* p_in = nullptr;
  const int tile_ks = tile_k_parts(m_tiles, mlp->compute_units);
  for (int layer = 0; layer <= mlp->hidden; ++layer) {
    l.g0 = (layer == 0) ? 0 : mlp->in_padded / 8 + (layer - 1) * (kWidth / 8);
    l.kg = (layer == 0) ? mlp->in_padded / 8 : kWidth / 8;
    l.splits = layer == 0 ? 1 : (split_k ? kSplit : ks);
    l.p_in = p_in;
    l.bias_in = (layer == 0) ? nullptr : mlp->bias + (size_t)(layer - 1) * kWidth;
    l.bias_out = mlp->bias + (size_t)layer * kWidth;
    l.p_out = buffers[layer & 1];
    const dim3 grid(kWidth / 32, (unsigned)l.splits, (unsigned)m_tiles);
    if (layer == 0 && split_k)
      hipLaunchKernelGGL((mlp_layer_kernel<true, 0, true, 4, false, 0>), grid, dim3(256), 0,
                         stream, l);
    else if (layer == 0 && mlp->w_first_t != nullptr && m_tiles >= kFirstFmaMinTiles) {
      hipLaunchKernelGGL(mlp_first_fma_kernel, dim3((unsigned)m_tiles, kFirstFmaSlices), dim3(256), 0,
                         stream, l);
    } else if (layer == 0)
      hipLaunchKernelGGL((mlp_layer_kernel<true, 0, true, 4, false, 0, 1, true>), grid, dim3(256),
                         0, stream, l);
    else if (ks == 2 && !partials)
      hipLaunchKernelGGL((mlp_layer_kernel<false, 0, false, 8, true, 2, 1, true, 2>), grid,
                         dim3(512), 0, stream, l);
    else if (ks == 2)
      hipLaunchKernelGGL((mlp_layer_kernel<false, 2, false, 8, true, 2, 1, true, 2>), grid,
                         dim3(512), 0, stream, l);
    else if (!split_k && tile_ks == 1)
      hipLaunchKernelGGL((mlp_layer_tile_kernel<1, 4>),
                         dim3(kWidth / 64, (unsigned)((m_tiles + 1) / 2)), dim3(256), 0, stream, l);
    else if (!split_k && tile_ks == 2)
      hipLaunchKernelGGL((mlp_layer_tile_kernel<2, 4>), dim3(kWidth / 64, (unsigned)m_tiles),
                         dim3(256), 0, stream, l);
    else if (!split_k)
      hipLaunchKernelGGL((mlp_layer_tile_kernel<4, 4>), dim3(kWidth / 32, (unsigned)m_tiles),
                         dim3(256), 0, stream, l);
    else if (partials)
      hipLaunchKernelGGL((mlp_layer_kernel<false, kSplit, false, 4, false, 0>), grid, dim3(256),
                         0, stream, l);
    else
      hipLaunchKernelGGL((mlp_layer_kernel<false, 0, false, 4, false, 0>), grid, dim3(256), 0,
                         stream, l);
    p_in = l.p_out;
    partials = l.splits != 1;
  }
  LastArgs z{};
  z.p_in = p_in;
  z.bias_in = mlp->bias + (size_t)mlp->hidden * kWidth;
  z.w_last = mlp->w_last; z.b_last = mlp->b_last;
  z.n = n; z.m_pad = l.m_pad; z.out = out;
  z.done_flag = split_k ? done_flag : nullptr;  // (only the few-row shape publishes)
  z.done_value = done_value;
  const dim3 rows_grid((unsigned)((n + 3) / 4));
  if (partials && split_k)
    hipLaunchKernelGGL(mlp_last_kernel<kSplit>, rows_grid, dim3(256), 0, stream, z);
  else if (split_k) hipLaunchKernelGGL(mlp_last_kernel<0>, rows_grid, dim3(256), 0, stream, z);
  else if (partials && ks == 2)
    hipLaunchKernelGGL(mlp_last_km_kernel<2>, dim3((unsigned)m_tiles), dim3(256), 0, stream, z);
  else hipLaunchKernelGGL(mlp_last_km_kernel<0>, dim3((unsigned)m_tiles), dim3(256), 0, stream, z);
  return hipGetLastError() == hipSuccess ? HBT_OK : HBT_EHIP;
}

// The fused kernel: one workgroup per 32 rows.
int forward_fused(hbt_mlp* mlp, const double* raw_features, int64_t n, float* out,
                  hipStream_t stream) {
  using namespace hbt;
  const int64_t blocks = (n + kRows - 1) / kRows;
  MlpArgs a{};
  a.raw = raw_features;
  a.out = out;
  a.n = n;
  a.in_features = mlp->in_features;
  a.in_padded = mlp->in_padded;
  a.hidden = mlp->hidden;
  a.mu = mlp->mu;
  a.sigma = mlp->sigma;
  a.w_stream = mlp->w_stream;
  a.bias = mlp->bias;
  a.w_last = mlp->w_last;
  a.b_last = mlp->b_last;
  hipLaunchKernelGGL(mlp_fused_kernel<kWaves>, dim3((unsigned)blocks), dim3(kWaves * 64),
                     kLdsBytes, stream, a);
  return hipGetLastError() == hipSuccess ? HBT_OK : HBT_EHIP;
}

}  // namespace

extern "C" {

hbt_mlp* hbt_mlp_create(int32_t in_features, int32_t width, int32_t hidden_layers,
                        const float* const* W, const float* const* b, const double* mu,
                        const double* sigma, int* err) {
  using namespace hbt;
  int dummy;
  if (err == nullptr) err = &dummy;
  *err = HBT_OK;
  if (W == nullptr || b == nullptr || mu == nullptr || sigma == nullptr || in_features <= 0 ||
      hidden_layers < 0) {
    *err = HBT_EINVAL;
    return nullptr;
  }
  for (int i = 0; i < hidden_layers + 2; ++i)
    if (W[i] == nullptr || b[i] == nullptr) { *err = HBT_EINVAL; return nullptr; }
  const int in_padded = (int)align_up((size_t)in_features, 32);
  if (width != kWidth || in_padded > kMaxInPadded || hidden_layers > 64) {
    *err = HBT_ESIZE;
    return nullptr;
  }
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    *err = HBT_EHIP;
    return nullptr;
  }

  int compute_units = 0;
  if (hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device) !=
          hipSuccess ||
      compute_units <= 0) {
    (void)hipGetLastError();
    *err = HBT_EHIP;
    return nullptr;
  }

  // Host image of the device blob.
  // floats per wave: (fc1 groups + 128 per hidden layer) x tpw x 64 lanes x 4
  const int tpw = (kWidth / 32) / kWaves;
  const size_t group_floats = (size_t)tpw * 64 * 4;
  const size_t wave_stride = ((size_t)in_padded / 8 + (size_t)hidden_layers * (kWidth / 8)) * group_floats;
  const size_t n_stream = wave_stride * kWaves;
  const size_t n_bias = (size_t)(hidden_layers + 1) * kWidth;
  size_t off = 0;
  const size_t off_mu = off; off = align_up(off + sizeof(double) * in_features, 256);
  const size_t off_sigma = off; off = align_up(off + sizeof(double) * in_features, 256);
  const size_t off_stream = off; off = align_up(off + sizeof(float) * n_stream, 256);
  const size_t off_bias = off; off = align_up(off + sizeof(float) * n_bias, 256);
  const size_t off_last = off; off = align_up(off + sizeof(float) * kWidth, 256);
  const bool first_fma = in_features <= kFirstFmaMaxIn;
  const size_t off_first_t = off;
  if (first_fma) off = align_up(off + sizeof(float) * kFirstFmaMaxIn * kWidth, 256);
  const size_t image = off;  // what is copied from the host; scratch follows
  const size_t scratch_bytes = sizeof(float) * kScratchFloats;
  const size_t off_scratch0 = off; off = align_up(off + scratch_bytes, 256);
  const size_t off_scratch1 = off; off = align_up(off + scratch_bytes, 256);
  const size_t total = off;

  std::vector<unsigned char> host;
  try {
    host.resize(image, 0);
  } catch (const std::bad_alloc&) {
    *err = HBT_ENOMEM;
    return nullptr;
  }
  std::memcpy(host.data() + off_mu, mu, sizeof(double) * in_features);
  std::memcpy(host.data() + off_sigma, sigma, sizeof(double) * in_features);
  float* stream = reinterpret_cast<float*>(host.data() + off_stream);
  pack_layer(W[0], in_features, in_padded, kWaves, stream, wave_stride);
  for (int l = 0; l < hidden_layers; ++l)
    pack_layer(W[1 + l], kWidth, kWidth, kWaves,
               stream + ((size_t)in_padded / 8 + (size_t)l * (kWidth / 8)) * group_floats, wave_stride);
  for (int l = 0; l <= hidden_layers; ++l)
    std::memcpy(host.data() + off_bias + sizeof(float) * (size_t)l * kWidth, b[l],
                sizeof(float) * kWidth);
  std::memcpy(host.data() + off_last, W[hidden_layers + 1], sizeof(float) * kWidth);
  if (first_fma) {
    float* t = reinterpret_cast<float*>(host.data() + off_first_t);  // zero beyond in_features
    for (int n = 0; n < kWidth; ++n)
      for (int k = 0; k < in_features; ++k) t[(size_t)k * kWidth + n] = W[0][(size_t)n * in_features + k];
  }

  void* blob = nullptr;
  if (hipMalloc(&blob, total) != hipSuccess) {
    (void)hipGetLastError();
    *err = HBT_ENOMEM;
    return nullptr;
  }
  if (hipMemcpy(blob, host.data(), image, hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(blob);
    *err = HBT_EHIP;
    return nullptr;
  }
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(&mlp_fused_kernel<kWaves>),
                          hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)kLdsBytes) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(blob);
    *err = HBT_EHIP;
    return nullptr;
  }

  void* one_host = nullptr;
  void* one_device = nullptr;
  if (hipHostMalloc(&one_host, kOneBytes, hipHostMallocDefault) != hipSuccess ||
      hipHostGetDevicePointer(&one_device, one_host, 0) != hipSuccess || one_device == nullptr) {
    (void)hipGetLastError();
    if (one_host != nullptr) (void)hipHostFree(one_host);
    (void)hipFree(blob);
    *err = HBT_ENOMEM;
    return nullptr;
  }
  std::memset(one_host, 0, kOneBytes);

  hbt_mlp* m = new (std::nothrow) hbt_mlp();
  if (m == nullptr) {
    (void)hipHostFree(one_host);
    (void)hipFree(blob);
    *err = HBT_ENOMEM;
    return nullptr;
  }
  m->one_host = static_cast<unsigned char*>(one_host);
  m->one_device = static_cast<unsigned char*>(one_device);
  unsigned char* base = static_cast<unsigned char*>(blob);
  m->in_features = in_features;
  m->in_padded = in_padded;
  m->width = width;
  m->hidden = hidden_layers;
  m->device = device;
  m->compute_units = compute_units;
  m->blob = blob;
  m->mu = reinterpret_cast<const double*>(base + off_mu);
  m->sigma = reinterpret_cast<const double*>(base + off_sigma);
  m->w_stream = reinterpret_cast<const float*>(base + off_stream);
  m->bias = reinterpret_cast<const float*>(base + off_bias);
  m->w_last = reinterpret_cast<const float*>(base + off_last);
  m->w_first_t = first_fma ? reinterpret_cast<const float*>(base + off_first_t) : nullptr;
  m->b_last = b[hidden_layers + 1][0];
  m->scratch[0] = reinterpret_cast<float*>(base + off_scratch0);
  m->scratch[1] = reinterpret_cast<float*>(base + off_scratch1);
  return m;
}

int hbt_mlp_forward(hbt_mlp* mlp, const double* raw_features, int64_t n, float* out,
                    void* hip_stream) {
  using namespace hbt;
  if (mlp == nullptr || n < 0) return HBT_EINVAL;
  if (n == 0) return HBT_OK;
  if (raw_features == nullptr || out == nullptr) return HBT_EINVAL;
  if ((reinterpret_cast<uintptr_t>(raw_features) % 8) != 0 ||
      (reinterpret_cast<uintptr_t>(out) % 4) != 0)
    return HBT_EALIGN;
  const int64_t blocks = (n + kRows - 1) / kRows;
  if (blocks > 0x7fffffff) return HBT_ESIZE;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (device != mlp->device) return HBT_EINVAL;

  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  // The fused kernel keeps every compute unit busy for whole rounds of
  // 32 rows x compute units (about 0.94 ms each); what is left over after the
  // last whole round would cost another one.  Up to kLayerMaxRows leftover rows
  // go through the per-layer path instead, which takes less for them.
  const int64_t round_rows = (int64_t)kRows * mlp->compute_units;
  const int64_t leftover = n % round_rows;
  if (leftover == 0 || leftover > kLayerMaxRows)
    return forward_fused(mlp, raw_features, n, out, stream);
  const int64_t done = n - leftover;
  if (done > 0) {
    const int rc = forward_fused(mlp, raw_features, done, out, stream);
    if (rc != HBT_OK) return rc;
  }
  return forward_layers(mlp, raw_features + done * mlp->in_features, leftover, out + done,
                        mlp->scratch, stream);
}

int hbt_mlp_forward_static(hbt_mlp* mlp, const double* raw_features, int64_t n, float* out,
                           void* hip_stream) {
  using namespace hbt;
  if (mlp == nullptr || n < 0) return HBT_EINVAL;
  if (n > kStaticMaxRows) return HBT_ESIZE;
  if (n == 0) return HBT_OK;
  if (raw_features == nullptr || out == nullptr) return HBT_EINVAL;
  if ((reinterpret_cast<uintptr_t>(raw_features) % 8) != 0 ||
      (reinterpret_cast<uintptr_t>(out) % 4) != 0)
    return HBT_EALIGN;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (device != mlp->device) return HBT_EINVAL;
  int rc = HBT_OK;
  float* base = static_scratch_of(device, &rc);
  if (base == nullptr) return rc;
  // Every value a layer reads was written by the layer before it in this call
  // (rows past n within the last 32-row tile included), so nothing needs
  // clearing between calls.
  float* const buffers[2] = {base, base + kStaticFloats};
  return forward_layers(mlp, raw_features, n, out, buffers, static_cast<hipStream_t>(hip_stream));
}

int hbt_mlp_predict_one(hbt_mlp* mlp, const double* raw_row, float* out, void* hip_stream) {
  using namespace hbt;
  if (mlp == nullptr || raw_row == nullptr || out == nullptr) return HBT_EINVAL;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (device != mlp->device) return HBT_EINVAL;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  // the call waits for its stream: a stream under graph capture cannot be used
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  if (capture != hipStreamCaptureStatusNone) return HBT_EINVAL;

  std::lock_guard<std::mutex> guard(mlp->one_lock);
  std::memcpy(mlp->one_host, raw_row, sizeof(double) * (size_t)mlp->in_features);
  const uint32_t call = ++mlp->one_calls;
  const int rc = forward_layers(mlp, reinterpret_cast<const double*>(mlp->one_device), 1,
                                reinterpret_cast<float*>(mlp->one_device + kOneOutOffset),
                                mlp->scratch, stream,
                                reinterpret_cast<uint32_t*>(mlp->one_device + kOneDoneOffset), call);
  if (rc != HBT_OK) return rc;
  // The last kernel publishes the call's number once the prediction is in the
  // block: watching for it takes microseconds less than waiting for the
  // stream's completion signal.  Should it not show up in time, the stream is
  // waited for, which is always right.
  if (!hbt::wait_published(reinterpret_cast<const uint32_t*>(mlp->one_host + kOneDoneOffset), call) &&
      hipStreamSynchronize(stream) != hipSuccess) {
    (void)hipGetLastError();
    return HBT_EHIP;
  }
  std::memcpy(out, mlp->one_host + kOneOutOffset, sizeof(float));
  return HBT_OK;
}

void hbt_mlp_destroy(hbt_mlp* mlp) {
  if (mlp == nullptr) return;
  if (mlp->one_host != nullptr) (void)hipHostFree(mlp->one_host);
  if (mlp->blob != nullptr) (void)hipFree(mlp->blob);
  delete mlp;
}

}  // extern "C"
