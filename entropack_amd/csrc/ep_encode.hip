// The encoders on the device. First the lattice_rans encoder: nearest-E8 quantisation, stream statistics, row-scale refit
// and the tiled 32-way interleaved rANS encode. Every kernel produces, from the same inputs, exactly what the CPU encoder
// (csrc/host_codec.c) produces: the float work is single IEEE operations in the same order (this file is compiled
// without contraction), the rest is integer work. The one exception is the row-scale refit, whose float32 row sums are
// added in this kernel's own fixed order (the CPU lane adds them in torch's).
//
// Counterparts in the reference (entropack/schemes/lattice_rans/): the quantise kernels lattice_rans.cu:224, the refit
// kernels :313, e8_minmax_fields_kernel :334, e8_histogram_kernel :376, e8_rans_encode_vector_kernel :400 and
// e8_compact_kernel :467, launched from cuda.py:115-221 and :520-558. The algorithms followed are the eager lane's
// (eager.py:18-58, rans.py:133-186), with which the reference states its kernels agree bit for bit
// (lattice_rans.cu:3-18).
//
// Then the lossless tile_ans encoder (byte histogram, one rANS or raw stream per byte lane and tile), all integer work
// and bit-identical to hc_tile_ans_encode; counterparts tile_ans.cu:27 (histogram), :67 (encode), :157 (compact),
// launched from entropack/schemes/tile_ans/cuda.py:31-119. Both encoders share the cumulative sum and the gather.
#include <hip/hip_runtime.h>
#include <limits.h>

#include "entropack_hip.h"
#include "ep_common.hpp"

namespace ep {

constexpr int kSummaryMinMax = 2 * kFieldStreams;       // summary[2 k], [2 k + 1]: least and greatest value of field stream k
constexpr int kSummaryOnes = kSummaryMinMax;            // summary[32]: vectors of coset 1
constexpr int kSummaryWords = kSummaryOnes + 1;
static_assert(kSummaryWords == EP_HIP_ENCODE_SUMMARY_WORDS, "header and kernels agree on the summary's size");

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4v __attribute__((ext_vector_type(4)));

__global__ void summary_init_kernel(long long* __restrict__ summary) {
  const int k = threadIdx.x;
  if (k < kSummaryMinMax) summary[k] = (k & 1) ? LLONG_MIN : LLONG_MAX;
  else if (k == kSummaryOnes) summary[k] = 0;
}

// Nearest point of D8 (integer vectors with an even sum): round every coordinate to nearest-even; when the sum is odd,
// move the coordinate that was rounded furthest (the first of equals) one step to its other side (up when its residual
// is zero).
__device__ __forceinline__ void nearest_d8(const float (&y)[8], float (&out)[8]) {
  float total = 0.0f, best = -1.0f, residual_at_best = 0.0f;
  int at = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    out[j] = __builtin_rintf(y[j]);
    const float r = y[j] - out[j];
    total += out[j];                          // small integers: exact
    const float a = __builtin_fabsf(r);
    if (a > best) { best = a; at = j; residual_at_best = r; }
  }
  const float halved = total * 0.5f;          // exact; a whole number exactly when the sum is even
  const bool odd = halved != __builtin_rintf(halved);
  const float step = residual_at_best < 0.0f ? -1.0f : 1.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j) out[j] = (odd && j == at) ? out[j] + step : out[j];
}

// Squared distance in float64, added as ((0+4)+(2+6)) + ((1+5)+(3+7)): the order that decides exact ties between the
// two cosets in the CPU encoder.
__device__ __forceinline__ double distance2(const float (&y)[8], const float (&p)[8]) {
  double s[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const double d = static_cast<double>(y[j]) - static_cast<double>(p[j]);
    s[j] = d * d;
  }
  return ((s[0] + s[4]) + (s[2] + s[6])) + ((s[1] + s[5]) + (s[3] + s[7]));
}

// One thread per vector (grid-stride). y = (x / rms[row]) / scale, nearest E8 point = the nearer of the nearest D8 point
// and the nearest point of D8 + 1/2 (the first on a tie), written as the coset bit and the fields z0..z6, m with
// 2 m + parity(z0..z6) = z7. Every block folds the least and greatest field values it saw, per stream, into `summary`.
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ x, const float* __restrict__ rms, int64_t cols, float scale,
                                                       const int64_t* __restrict__ row_index, int64_t vectors, int64_t vectors_per_row,
                                                       int8_t* __restrict__ coset, int32_t* __restrict__ fields,
                                                       long long* __restrict__ summary) {
  __shared__ int lo_shared[kFieldStreams], hi_shared[kFieldStreams];
  __shared__ unsigned ones_shared;
  if (threadIdx.x < kFieldStreams) { lo_shared[threadIdx.x] = INT_MAX; hi_shared[threadIdx.x] = INT_MIN; }
  if (threadIdx.x == 0) ones_shared = 0;
  __syncthreads();

  int lo[kFieldStreams], hi[kFieldStreams];
#pragma unroll
  for (int k = 0; k < kFieldStreams; ++k) { lo[k] = INT_MAX; hi[k] = INT_MIN; }
  unsigned ones = 0;
  // (picked, v) = (at / vectors_per_row, at % vectors_per_row), carried along instead of divided out for every vector
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t stride_rows = stride / vectors_per_row, stride_rest = stride - stride_rows * vectors_per_row;
  const int64_t start = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t picked = start / vectors_per_row, v = start - picked * vectors_per_row;
  for (int64_t at = start; at < vectors; at += stride, picked += stride_rows, v += stride_rest) {
    if (v >= vectors_per_row) { v -= vectors_per_row; ++picked; }
    const int64_t row = row_index != nullptr ? row_index[picked] : picked;
    const f32x4* source = reinterpret_cast<const f32x4*>(x + row * cols + v * 8);
    const f32x4 first = source[0], second = source[1];
    const float raw[8] = {first.x, first.y, first.z, first.w, second.x, second.y, second.z, second.w};
    const float norm = rms[row];
    float y[8], shifted[8], p0[8], p1[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      y[j] = (raw[j] / norm) / scale;
      shifted[j] = y[j] - 0.5f;
    }
    nearest_d8(y, p0);
    nearest_d8(shifted, p1);
#pragma unroll
    for (int j = 0; j < 8; ++j) p1[j] += 0.5f;
    const int c = !(distance2(y, p0) <= distance2(y, p1));
    int z[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) z[j] = static_cast<int>(__builtin_rintf(c ? p1[j] - 0.5f : p0[j] - 0.0f));
    const int parity = (z[0] + z[1] + z[2] + z[3] + z[4] + z[5] + z[6]) & 1;
    z[7] = (z[7] - parity) >> 1;              // even for a lattice point; floor otherwise
    coset[at] = static_cast<int8_t>(c);
    i32x4v* to = reinterpret_cast<i32x4v*>(fields + at * 8);
    to[0] = i32x4v{z[0], z[1], z[2], z[3]};
    to[1] = i32x4v{z[4], z[5], z[6], z[7]};
    ones += static_cast<unsigned>(c);
#pragma unroll
    for (int f = 0; f < kFields; ++f) {
      const int k0 = 2 * f, k1 = 2 * f + 1;
      lo[k0] = c ? lo[k0] : min(lo[k0], z[f]);
      hi[k0] = c ? hi[k0] : max(hi[k0], z[f]);
      lo[k1] = c ? min(lo[k1], z[f]) : lo[k1];
      hi[k1] = c ? max(hi[k1], z[f]) : hi[k1];
    }
  }
#pragma unroll
  for (int k = 0; k < kFieldStreams; ++k) {
    if (lo[k] != INT_MAX) { atomicMin(&lo_shared[k], lo[k]); atomicMax(&hi_shared[k], hi[k]); }
  }
  if (ones != 0) atomicAdd(&ones_shared, ones);
  __syncthreads();
  // Most blocks have nothing to add to what others already recorded: a look at the current value (it only ever moves
  // one way, so a stale look costs an atomic that changes nothing) spares the device thousands of atomics on 32 words.
  if (threadIdx.x < kFieldStreams && lo_shared[threadIdx.x] != INT_MAX) {
    const volatile long long* seen = summary;
    if (lo_shared[threadIdx.x] < seen[2 * threadIdx.x]) atomicMin(&summary[2 * threadIdx.x], static_cast<long long>(lo_shared[threadIdx.x]));
    if (hi_shared[threadIdx.x] > seen[2 * threadIdx.x + 1]) atomicMax(&summary[2 * threadIdx.x + 1], static_cast<long long>(hi_shared[threadIdx.x]));
  }
  if (threadIdx.x == 0 && ones_shared != 0)
    atomicAdd(reinterpret_cast<unsigned long long*>(&summary[kSummaryOnes]), static_cast<unsigned long long>(ones_shared));
}

// Counts of every symbol of every stream. bin_rel[s] = first bin of stream s - least value of stream s (stream 0 = the
// coset bits, stream 1 + 2 f + c = field f of the vectors of coset c). STAGED: the block counts in LDS and adds what it
// counted to the global bins at its end. A value whose bin lies outside [0, total_bins) is not counted (the caller
// compares the bins' sum with the number of symbols).
template <bool STAGED>
__global__ __launch_bounds__(256) void histogram_kernel(const int8_t* __restrict__ coset, const int32_t* __restrict__ fields, int64_t vectors,
                                                        const int32_t* __restrict__ bin_rel, int total_bins,
                                                        unsigned long long* __restrict__ bins) {
  extern __shared__ unsigned staged[];
  __shared__ int rel[kStreams];
  if (threadIdx.x < kStreams) rel[threadIdx.x] = bin_rel[threadIdx.x];
  if (STAGED)
    for (int b = threadIdx.x; b < total_bins; b += blockDim.x) staged[b] = 0;
  __syncthreads();
  auto count = [&](int bin) {
    if (static_cast<unsigned>(bin) >= static_cast<unsigned>(total_bins)) return;
    if (STAGED) atomicAdd(&staged[bin], 1u);
    else atomicAdd(&bins[bin], 1ull);
  };
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t at = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; at < vectors; at += stride) {
    const int c = coset[at] != 0;
    const i32x4v* from = reinterpret_cast<const i32x4v*>(fields + at * 8);
    const i32x4v a = from[0], b = from[1];
    const int z[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    count(rel[0] + c);
#pragma unroll
    for (int f = 0; f < kFields; ++f) count(rel[1 + 2 * f + c] + z[f]);
  }
  if (STAGED) {
    __syncthreads();
    for (int b = threadIdx.x; b < total_bins; b += blockDim.x)
      if (staged[b] != 0) atomicAdd(&bins[b], static_cast<unsigned long long>(staged[b]));
  }
}

__global__ void zero_words_kernel(unsigned long long* __restrict__ words, int64_t count) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) words[i] = 0;
}

// Least-squares scale of a row against the lattice points chosen for it: sum(x p) / sum(p p) in float32, at least
// 1e-12; scale * rms[row] for a row of zeros. row_sse (optional) = the squared error that scale leaves,
// max(sum(x x) - sum(x p)^2 / sum(p p), 0), or sum(x x) for a row of zeros. One block per row; every thread adds its
// vectors (t, t + 256, ...) in order, coordinate 0 to 7, and the 256 partial sums are added pairwise (t with t + 128,
// then + 64, ...).
__global__ __launch_bounds__(256) void row_scales_kernel(const float* __restrict__ x, const float* __restrict__ rms, int64_t cols, float scale,
                                                         const int8_t* __restrict__ coset, const int32_t* __restrict__ fields,
                                                         float* __restrict__ scales, float* __restrict__ row_sse) {
  __shared__ float numerators[256], denominators[256], energies[256];
  const int64_t row = blockIdx.x, vectors_per_row = cols / 8;
  float numerator = 0.0f, denominator = 0.0f, energy = 0.0f;
  for (int64_t v = threadIdx.x; v < vectors_per_row; v += 256) {
    const int64_t at = row * vectors_per_row + v;
    const f32x4* source = reinterpret_cast<const f32x4*>(x + row * cols + v * 8);
    const f32x4 first = source[0], second = source[1];
    const float raw[8] = {first.x, first.y, first.z, first.w, second.x, second.y, second.z, second.w};
    const i32x4v* from = reinterpret_cast<const i32x4v*>(fields + at * 8);
    const i32x4v a = from[0], b = from[1];
    const int z[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    const float half = coset[at] != 0 ? 0.5f : 0.0f;
    const int parity = (z[0] + z[1] + z[2] + z[3] + z[4] + z[5] + z[6]) & 1;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float level = static_cast<float>(j < 7 ? z[j] : 2 * z[7] + parity) + half;
      numerator += raw[j] * level;
      denominator += level * level;
      energy += raw[j] * raw[j];
    }
  }
  numerators[threadIdx.x] = numerator;
  denominators[threadIdx.x] = denominator;
  energies[threadIdx.x] = energy;
  __syncthreads();
  for (int width = 128; width > 0; width >>= 1) {
    if (threadIdx.x < width) {
      numerators[threadIdx.x] += numerators[threadIdx.x + width];
      denominators[threadIdx.x] += denominators[threadIdx.x + width];
      energies[threadIdx.x] += energies[threadIdx.x + width];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float fitted = numerators[0] / denominators[0];
    scales[row] = denominators[0] > 0.0f ? (fitted > 1.0e-12f ? fitted : 1.0e-12f) : scale * rms[row];
    if (row_sse != nullptr) {
      const float left = energies[0] - numerators[0] * numerators[0] / denominators[0];
      row_sse[row] = denominators[0] > 0.0f ? (left > 0.0f ? left : 0.0f) : energies[0];
    }
  }
}

// One tile per 32-lane half of a wavefront, lane l carrying state l. A group of 32 vectors is one vector per lane; its
// symbols go in last to first (field 7 ... field 0, then the coset bit), and the words the lanes push out in one step
// are appended in lane order, as the sequential encoder appends them. entries[i] = {freq | cdf << 16, min(floor(2^32 /
// freq), 2^32 - 1)} of table position i; table_rel[s] = first position of stream s - least value of stream s. The
// quotient state / freq is the high half of state * floor(2^32 / freq), which is the quotient or one less (the product
// falls short of 2^32 state / freq by less than state <= 2^32), put right by one comparison of the remainder. A symbol
// outside the tables, or one of frequency 0, raises *error and is coded with frequency 1 so that the launch still ends.
// STAGED: the block first copies the table entries into LDS (total_entries * 8 bytes of dynamic LDS) and the nine
// lookups of a vector go there; all nine are made before the first symbol is coded, since none depends on the state.
template <bool STAGED>
__global__ __launch_bounds__(256) void rans_encode_kernel(const int8_t* __restrict__ coset, const int32_t* __restrict__ fields, int64_t vectors,
                                                          int tile_vectors, int64_t tiles, const uint2* __restrict__ entries,
                                                          const int32_t* __restrict__ table_rel, int total_entries, int prob_bits,
                                                          uint32_t* __restrict__ states, uint32_t* __restrict__ tile_words,
                                                          uint16_t* __restrict__ scratch, int* __restrict__ error) {
  extern __shared__ uint2 staged_entries[];
  __shared__ int rel[kStreams];
  if (threadIdx.x < kStreams) rel[threadIdx.x] = table_rel[threadIdx.x];
  if (STAGED)
    for (int i = threadIdx.x; i < total_entries; i += blockDim.x) staged_entries[i] = entries[i];
  __syncthreads();
  const uint2* table = STAGED ? staged_entries : entries;
  const int lane = threadIdx.x & 63, half = lane >> 5, l = lane & 31;
  const int64_t tile = (static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2 + half;
  if (tile >= tiles) return;
  int rel_even[kFields], rel_odd[kFields];               // first table position - least value, of the field's two streams
#pragma unroll
  for (int f = 0; f < kFields; ++f) { rel_even[f] = rel[1 + 2 * f]; rel_odd[f] = rel[2 + 2 * f]; }
  const int rel_coset = rel[0];
  const int64_t begin = tile * tile_vectors;
  const int64_t end = begin + tile_vectors < vectors ? begin + tile_vectors : vectors;
  uint16_t* out = scratch + tile * (static_cast<int64_t>(tile_vectors) * 9);
  const uint32_t below = (1u << l) - 1u;
  const int renorm_shift = 31 - prob_bits;
  uint32_t state = kStateMin, cursor = 0;
  bool bad = false;
  for (int64_t base = begin; base < end; base += kStatesPerTile) {
    const bool valid = base + l < end;
    int c = 0;
    int z[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (valid) {
      c = coset[base + l] != 0;
      const i32x4v* from = reinterpret_cast<const i32x4v*>(fields + (base + l) * 8);
      const i32x4v a = from[0], b = from[1];
      z[0] = a.x; z[1] = a.y; z[2] = a.z; z[3] = a.w; z[4] = b.x; z[5] = b.y; z[6] = b.z; z[7] = b.w;
    }
    uint2 looked_up[9];
#pragma unroll
    for (int step = 0; step < 9; ++step) {
      const int f = 7 - step;
      const int position = step < 8 ? (c ? rel_odd[f] : rel_even[f]) + z[f] : rel_coset + c;
      const bool inside = static_cast<unsigned>(position) < static_cast<unsigned>(total_entries);
      bad = bad || (valid && !inside);
      looked_up[step] = table[inside ? position : 0];
    }
#pragma unroll
    for (int step = 0; step < 9; ++step) {
      uint2 entry = looked_up[step];
      uint32_t freq = entry.x & 0xFFFFu;
      const uint32_t cdf = entry.x >> 16;
      if (freq == 0) { bad = bad || valid; freq = 1; entry.y = 0xFFFFFFFFu; }
      const bool push = valid && state >= (freq << renorm_shift);
      const uint32_t pushing = static_cast<uint32_t>(__ballot(push) >> (32 * half));
      if (push) {
        out[cursor + __popc(pushing & below)] = static_cast<uint16_t>(state & 0xFFFFu);
        state >>= 16;
      }
      cursor += __popc(pushing);
      if (valid) {
        uint32_t quotient = __umulhi(state, entry.y);
        uint32_t rest = state - quotient * freq;
        if (rest >= freq) { rest -= freq; ++quotient; }
        state = (quotient << prob_bits) + rest + cdf;
      }
    }
  }
  states[tile * kStatesPerTile + l] = state;
  if (l == 0) tile_words[tile] = cursor;
  if (bad) *error = 1;
}

// offsets[0] = 0, offsets[t + 1] = words of tiles 0..t (modulo 2^32; *total holds the full sum). One block walks the
// counts 1024 at a time: every thread holds one count (the next chunk's is already on its way), the wavefronts scan
// theirs with shuffles, sixteen wavefront totals meet in LDS, and a 64-bit carry runs from chunk to chunk.
__global__ __launch_bounds__(1024) void offsets_kernel(const uint32_t* __restrict__ tile_words, int64_t tiles, uint32_t* __restrict__ offsets,
                                                       unsigned long long* __restrict__ total) {
  __shared__ unsigned long long wave_totals[16];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  unsigned long long carry = 0;
  uint32_t coming = t < tiles ? tile_words[t] : 0u;
  for (int64_t base = 0; base < tiles; base += 1024) {
    const uint32_t mine = coming;
    const int64_t after = base + 1024 + t;
    coming = after < tiles ? tile_words[after] : 0u;
    unsigned long long upto = mine;                        // inclusive sum over the lanes of this wavefront up to this one
#pragma unroll
    for (int distance = 1; distance < 64; distance <<= 1) {
      const unsigned long long from_below = __shfl_up(upto, distance);
      if (lane >= distance) upto += from_below;
    }
    if (lane == 63) wave_totals[wave] = upto;
    __syncthreads();
    unsigned long long before = 0, chunk = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const unsigned long long one = wave_totals[w];
      before += w < wave ? one : 0ull;
      chunk += one;
    }
    if (base + t < tiles) offsets[base + t + 1] = static_cast<uint32_t>(carry + before + upto);
    carry += chunk;
    __syncthreads();
  }
  if (t == 0) {
    offsets[0] = 0;
    *total = carry;
  }
}

// payload[offsets[t] ..) = the words stream t left at the start of its `stride` words of the scratch.
__global__ __launch_bounds__(256) void gather_kernel(const uint16_t* __restrict__ scratch, const uint32_t* __restrict__ offsets, int64_t tiles,
                                                     int64_t stride, uint16_t* __restrict__ payload) {
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const uint32_t from = offsets[tile];
    uint32_t words = offsets[tile + 1] - from;
    if (words > stride) words = static_cast<uint32_t>(stride);
    const uint16_t* source = scratch + tile * stride;
    uint16_t* to = payload + from;
    // one word to reach a 4-byte boundary of the destination, then two words per thread and store, then the last one
    const uint32_t head = (from & 1u) < words ? (from & 1u) : words;
    if (head != 0 && threadIdx.x == 0) to[0] = source[0];
    const uint32_t pairs = (words - head) / 2;
    uint32_t* to_pairs = reinterpret_cast<uint32_t*>(to + head);
    for (uint32_t i = threadIdx.x; i < pairs; i += blockDim.x)
      to_pairs[i] = static_cast<uint32_t>(source[head + 2 * i]) | static_cast<uint32_t>(source[head + 2 * i + 1]) << 16;
    if (head + 2 * pairs < words && threadIdx.x == 0) to[words - 1] = source[words - 1];
  }
}

// ---- tile_ans ----------------------------------------------------------------------------------------------------------

// counts[b][s] = number of elements whose byte b is s. Every thread takes 16 consecutive bytes at a time (the tensor's
// storage is 16-byte aligned and its byte count a multiple of the element size, so a byte's lane is its index modulo
// num_lanes). The bins are in LDS, in 2048 / (256 num_lanes) copies taken by the low bits of the thread index and one
// word apart in their bank alignment: the bytes of a weight tensor crowd into a few values, and lanes of a wavefront
// that add to one address (or to different addresses of one bank) take turns. Flushed with 64-bit atomics.
constexpr int kByteBins = 2048;
__global__ __launch_bounds__(256) void byte_histogram_kernel(const uint8_t* __restrict__ bytes, int64_t total_bytes, int num_lanes,
                                                             unsigned long long* __restrict__ counts) {
  __shared__ unsigned bins[kByteBins + 8];
  for (int b = threadIdx.x; b < kByteBins + 8; b += blockDim.x) bins[b] = 0;
  __syncthreads();
  const int per_copy = num_lanes * 256, copies = kByteBins / per_copy;
  unsigned* mine = bins + (threadIdx.x & (copies - 1)) * (per_copy + 1);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x * 16;
  const int lane_mask = num_lanes - 1;                   // 1, 2, 4 or 8 byte lanes
  for (int64_t at = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 16; at < total_bytes; at += stride) {
    if (at + 16 <= total_bytes) {
      const uint4 chunk = *reinterpret_cast<const uint4*>(bytes + at);
      const uint32_t words[4] = {chunk.x, chunk.y, chunk.z, chunk.w};
#pragma unroll
      for (int j = 0; j < 16; ++j) atomicAdd(&mine[(j & lane_mask) * 256 + ((words[j >> 2] >> (8 * (j & 3))) & 0xFFu)], 1u);
    } else {
      for (int64_t i = at; i < total_bytes; ++i) atomicAdd(&mine[(static_cast<int>(i) & lane_mask) * 256 + bytes[i]], 1u);
    }
  }
  __syncthreads();
  for (int b = threadIdx.x; b < per_copy; b += blockDim.x) {
    unsigned sum = 0;
    for (int c = 0; c < copies; ++c) sum += bins[c * (per_copy + 1) + b];
    if (sum != 0) atomicAdd(&counts[b], static_cast<unsigned long long>(sum));
  }
}

// One stream (byte lane b, tile t; stream index b * tiles + t) per 32-lane half. A raw lane stores its bytes two per
// word, the even element in the low byte. A coded lane runs 32 interleaved states over its symbols in order, lane l
// taking symbols l, l + 32, ...; the words a group of 32 symbols pushes out are appended in lane order. entries[b][s] =
// {freq | cdf << 16, min(floor(2^32 / freq), 2^32 - 1)}. states: [coded lanes before b * tiles + t][32]. A symbol of
// frequency 0 raises *error and is coded with frequency 1.
//
// The kernel is bound by the number of memory instructions it issues, so STAGED (tiles that start on 16 bytes, an even
// scratch stride) brings the elements in through LDS: a half fetches 256 whole elements with 16-byte loads, every lane
// then picks its bytes out of LDS, and the lane's 256 table entries are read from a copy in LDS as well. The last,
// short chunk of a tile and everything else take one byte per lane and load. (Collecting a coded stream's words in LDS
// too, to store them two per lane, measured slower: 432 against 406 us on the 8192 x 28672 bf16 weight.)
constexpr int kChunkElements = 8 * kStatesPerTile;         // 256 elements = eight groups of symbols
template <bool STAGED>
__global__ __launch_bounds__(256) void tile_ans_encode_kernel(const uint8_t* __restrict__ bytes, int64_t num_elements, int num_lanes,
                                                              int64_t tile_elements, int64_t tiles, int prob_bits, unsigned raw_mask,
                                                              const uint2* __restrict__ entries, uint32_t* __restrict__ states,
                                                              uint32_t* __restrict__ stream_words, uint16_t* __restrict__ scratch,
                                                              int64_t scratch_stride, int* __restrict__ error) {
  __shared__ uint4 staged_elements[STAGED ? 8 : 1][STAGED ? kChunkElements * 8 / 16 : 1];      // per half: 256 elements of up to 8 bytes
  __shared__ uint2 staged_table[STAGED ? 8 : 1][STAGED ? 256 : 1];
  const int lane = threadIdx.x & 63, half = lane >> 5, l = lane & 31;
  const int slot = STAGED ? static_cast<int>(threadIdx.x >> 6) * 2 + half : 0;
  const int64_t stream = (static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 2 + half;
  if (stream >= tiles * num_lanes) return;
  const int byte_lane = static_cast<int>(stream / tiles);
  const int64_t tile = stream - byte_lane * tiles;
  const int64_t begin = tile * tile_elements;
  const int64_t end = begin + tile_elements < num_elements ? begin + tile_elements : num_elements;
  uint16_t* out = scratch + stream * scratch_stride;
  const uint8_t* column = bytes + byte_lane;
  const uint8_t* staged_column = reinterpret_cast<const uint8_t*>(staged_elements[slot]) + byte_lane;
  // Fetches elements [base, base + 256) into this half's part of LDS (every lane of the half calls it).
  auto stage = [&](int64_t base) {
    __builtin_amdgcn_wave_barrier();                       // the reads of the chunk before are issued
    const uint4* source = reinterpret_cast<const uint4*>(bytes + base * num_lanes);
    for (int piece = l; piece < kChunkElements * num_lanes / 16; piece += 32) staged_elements[slot][piece] = source[piece];
    __builtin_amdgcn_wave_barrier();
  };
  if ((raw_mask >> byte_lane) & 1u) {
    const int64_t words = (end - begin + 1) / 2;
    int64_t done = 0;                                      // words written so far
    if (STAGED) {
      uint32_t* out_pairs = reinterpret_cast<uint32_t*>(out);
      for (; begin + 2 * done + kChunkElements <= end; done += kChunkElements / 2) {
        stage(begin + 2 * done);
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const int e = 4 * (l + 32 * k);                  // four elements = two words per lane and store
          const uint32_t pair = staged_column[e * num_lanes] | staged_column[(e + 1) * num_lanes] << 8 |
                                staged_column[(e + 2) * num_lanes] << 16 | staged_column[(e + 3) * num_lanes] << 24;
          out_pairs[done / 2 + l + 32 * k] = pair;
        }
      }
    }
    constexpr int kWordsAhead = 8;                         // 16 byte loads in flight per lane, then 8 stores
    for (int64_t first = done + l; first < words; first += 32 * kWordsAhead) {
      uint32_t low[kWordsAhead], high[kWordsAhead];
#pragma unroll
      for (int u = 0; u < kWordsAhead; ++u) {
        const int64_t e = begin + 2 * (first + 32 * u);
        low[u] = e < end ? column[e * num_lanes] : 0u;
        high[u] = e + 1 < end ? column[(e + 1) * num_lanes] : 0u;
      }
#pragma unroll
      for (int u = 0; u < kWordsAhead; ++u)
        if (first + 32 * u < words) out[first + 32 * u] = static_cast<uint16_t>(low[u] | high[u] << 8);
    }
    if (l == 0) stream_words[stream] = static_cast<uint32_t>(words);
    return;
  }
  const uint2* table = entries + byte_lane * 256;
  if (STAGED) {
    for (int i = l; i < 256; i += 32) staged_table[slot][i] = table[i];
    __builtin_amdgcn_wave_barrier();
  }
  const uint32_t below = (1u << l) - 1u;
  const int renorm_shift = 31 - prob_bits;
  uint32_t state = kStateMin, cursor = 0;
  bool bad = false;
  // The symbols and table entries of eight groups are fetched before the first of them is coded: neither depends on
  // the state, and a step that waited for its own two loads would last as long as two trips to memory.
  constexpr int kAhead = kChunkElements / kStatesPerTile;
  for (int64_t base = begin; base < end; base += kChunkElements) {
    uint32_t symbol[kAhead];
    uint2 entry[kAhead];
    if (STAGED && base + kChunkElements <= end) {
      stage(base);
#pragma unroll
      for (int u = 0; u < kAhead; ++u) symbol[u] = staged_column[(u * kStatesPerTile + l) * num_lanes];
    } else {
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int64_t at = base + u * kStatesPerTile + l;
        symbol[u] = at < end ? column[at * num_lanes] : 0u;
      }
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) entry[u] = STAGED ? staged_table[slot][symbol[u]] : table[symbol[u]];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int64_t group = base + u * kStatesPerTile;
      if (group >= end) break;
      const bool valid = group + l < end;
      uint32_t freq = entry[u].x & 0xFFFFu;
      const uint32_t cdf = entry[u].x >> 16;
      uint32_t reciprocal = entry[u].y;
      if (freq == 0) { bad = bad || valid; freq = 1; reciprocal = 0xFFFFFFFFu; }
      const bool push = valid && state >= (freq << renorm_shift);
      const uint32_t pushing = static_cast<uint32_t>(__ballot(push) >> (32 * half));
      if (push) {
        out[cursor + __popc(pushing & below)] = static_cast<uint16_t>(state & 0xFFFFu);
        state >>= 16;
      }
      cursor += __popc(pushing);
      if (valid) {
        uint32_t quotient = __umulhi(state, reciprocal);
        uint32_t rest = state - quotient * freq;
        if (rest >= freq) { rest -= freq; ++quotient; }
        state = (quotient << prob_bits) + rest + cdf;
      }
    }
  }
  const int coded_before = __popc(~raw_mask & ((1u << byte_lane) - 1u));
  states[(coded_before * tiles + tile) * kStatesPerTile + l] = state;
  if (l == 0) stream_words[stream] = cursor;
  if (bad) *error = 1;
}

static int grid_for(int64_t items, int per_block, int* blocks) {
  int device = 0, cus = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  EP_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  const int64_t wanted = (items + per_block - 1) / per_block, most = static_cast<int64_t>(cus > 0 ? cus : 256) * 8;
  *blocks = static_cast<int>(wanted < 1 ? 1 : (wanted < most ? wanted : most));
  return EP_HIP_OK;
}

}  // namespace ep

extern "C" int ep_hip_encode_quantize(const float* x_dev, const float* rms_dev, int64_t cols, float scale, const int64_t* row_index_dev,
                                      int64_t rows, int8_t* coset_dev, int32_t* fields_dev, int64_t* summary_dev, void* stream) {
  if (x_dev == nullptr || rms_dev == nullptr || coset_dev == nullptr || fields_dev == nullptr || summary_dev == nullptr) return EP_HIP_EINVAL;
  if (rows <= 0 || cols <= 0 || cols % 8 != 0 || !(scale > 0.0f)) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(x_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(fields_dev) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(summary_dev) % 8 != 0)
    return EP_HIP_EINVAL;
  const int64_t vectors_per_row = cols / 8, vectors = rows * vectors_per_row;
  int blocks = 0;
  const int status = ep::grid_for(vectors, 256, &blocks);
  if (status != EP_HIP_OK) return status;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(ep::summary_init_kernel, dim3(1), dim3(64), 0, s, reinterpret_cast<long long*>(summary_dev));
  hipLaunchKernelGGL(ep::quantize_kernel, dim3(blocks), dim3(256), 0, s, x_dev, rms_dev, cols, scale, row_index_dev, vectors, vectors_per_row,
                     coset_dev, fields_dev, reinterpret_cast<long long*>(summary_dev));
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

extern "C" int ep_hip_encode_histogram(const int8_t* coset_dev, const int32_t* fields_dev, int64_t vectors, const int32_t* bin_rel_dev,
                                       int32_t total_bins, uint64_t* bins_dev, void* stream) {
  if (coset_dev == nullptr || fields_dev == nullptr || bin_rel_dev == nullptr || bins_dev == nullptr) return EP_HIP_EINVAL;
  if (vectors <= 0 || total_bins <= 0 || reinterpret_cast<uintptr_t>(fields_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(bins_dev) % 8 != 0)
    return EP_HIP_EINVAL;
  int blocks = 0;
  const int status = ep::grid_for(vectors, 256 * 8, &blocks);
  if (status != EP_HIP_OK) return status;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(ep::zero_words_kernel, dim3((total_bins + 255) / 256), dim3(256), 0, s, reinterpret_cast<unsigned long long*>(bins_dev),
                     static_cast<int64_t>(total_bins));
  constexpr int kMostStagedBins = 15360;      // 60 KiB of LDS
  if (total_bins <= kMostStagedBins)
    hipLaunchKernelGGL(ep::histogram_kernel<true>, dim3(blocks), dim3(256), static_cast<size_t>(total_bins) * 4, s, coset_dev, fields_dev, vectors,
                       bin_rel_dev, total_bins, reinterpret_cast<unsigned long long*>(bins_dev));
  else
    hipLaunchKernelGGL(ep::histogram_kernel<false>, dim3(blocks), dim3(256), 0, s, coset_dev, fields_dev, vectors, bin_rel_dev, total_bins,
                       reinterpret_cast<unsigned long long*>(bins_dev));
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

extern "C" int ep_hip_encode_row_scales(const float* x_dev, const float* rms_dev, int64_t cols, float scale, int64_t rows,
                                        const int8_t* coset_dev, const int32_t* fields_dev, float* scales_dev, float* row_sse_dev,
                                        void* stream) {
  if (x_dev == nullptr || rms_dev == nullptr || coset_dev == nullptr || fields_dev == nullptr || scales_dev == nullptr) return EP_HIP_EINVAL;
  if (rows <= 0 || cols <= 0 || cols % 8 != 0) return EP_HIP_EINVAL;
  if (rows > 0x7FFFFFFF) return EP_HIP_EUNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(x_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(fields_dev) % 16 != 0) return EP_HIP_EINVAL;
  hipLaunchKernelGGL(ep::row_scales_kernel, dim3(static_cast<unsigned>(rows)), dim3(256), 0, static_cast<hipStream_t>(stream), x_dev, rms_dev,
                     cols, scale, coset_dev, fields_dev, scales_dev, row_sse_dev);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

extern "C" int ep_hip_encode_rans(const int8_t* coset_dev, const int32_t* fields_dev, int64_t vectors, const uint64_t* entries_dev,
                                  const int32_t* table_rel_dev, int32_t total_entries, int prob_bits, int tile_vectors,
                                  uint32_t* states_dev, uint32_t* tile_words_dev, uint16_t* scratch_dev, int32_t* error_dev, void* stream) {
  if (coset_dev == nullptr || fields_dev == nullptr || entries_dev == nullptr || table_rel_dev == nullptr || states_dev == nullptr ||
      tile_words_dev == nullptr || scratch_dev == nullptr || error_dev == nullptr)
    return EP_HIP_EINVAL;
  if (vectors <= 0 || total_entries <= 0 || prob_bits < 1 || prob_bits > 15 || tile_vectors < ep::kStatesPerTile) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(fields_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(entries_dev) % 8 != 0) return EP_HIP_EINVAL;
  const int64_t tiles = (vectors + tile_vectors - 1) / tile_vectors;
  const int64_t blocks = (tiles + 7) / 8;                 // 4 wavefronts of two tiles each
  if (blocks > 0x7FFFFFFF) return EP_HIP_EUNSUPPORTED;
  constexpr int kMostStagedEntries = 6144;                // 48 KiB of LDS
  if (total_entries <= kMostStagedEntries)
    hipLaunchKernelGGL(ep::rans_encode_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(256), static_cast<size_t>(total_entries) * 8,
                       static_cast<hipStream_t>(stream), coset_dev, fields_dev, vectors, tile_vectors, tiles,
                       reinterpret_cast<const uint2*>(entries_dev), table_rel_dev, total_entries, prob_bits, states_dev, tile_words_dev,
                       scratch_dev, error_dev);
  else
    hipLaunchKernelGGL(ep::rans_encode_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       coset_dev, fields_dev, vectors, tile_vectors, tiles, reinterpret_cast<const uint2*>(entries_dev), table_rel_dev,
                       total_entries, prob_bits, states_dev, tile_words_dev, scratch_dev, error_dev);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

extern "C" int ep_hip_encode_offsets(const uint32_t* tile_words_dev, int64_t tiles, uint32_t* offsets_dev, uint64_t* total_words_dev,
                                     void* stream) {
  if (tile_words_dev == nullptr || offsets_dev == nullptr || total_words_dev == nullptr || tiles <= 0) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(total_words_dev) % 8 != 0) return EP_HIP_EINVAL;
  hipLaunchKernelGGL(ep::offsets_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream), tile_words_dev, tiles, offsets_dev,
                     reinterpret_cast<unsigned long long*>(total_words_dev));
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

extern "C" int ep_hip_encode_gather(const uint16_t* scratch_dev, const uint32_t* offsets_dev, int64_t tiles, int64_t stride_words,
                                    uint16_t* payload_dev, void* stream) {
  if (scratch_dev == nullptr || offsets_dev == nullptr || payload_dev == nullptr || tiles <= 0 || stride_words <= 0) return EP_HIP_EINVAL;
  // The kernel stores pairs of words: the payload must start on four bytes.
  if (reinterpret_cast<uintptr_t>(payload_dev) % 4 != 0) return EP_HIP_EINVAL;
  int blocks = 0;
  const int status = ep::grid_for(tiles, 1, &blocks);
  if (status != EP_HIP_OK) return status;
  hipLaunchKernelGGL(ep::gather_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), scratch_dev, offsets_dev, tiles,
                     stride_words, payload_dev);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

extern "C" int ep_hip_tile_ans_histogram(const uint8_t* bytes_dev, int64_t num_elements, int num_lanes, uint64_t* counts_dev, void* stream) {
  if (bytes_dev == nullptr || counts_dev == nullptr || num_elements <= 0) return EP_HIP_EINVAL;
  if (num_lanes != 1 && num_lanes != 2 && num_lanes != 4 && num_lanes != 8) return EP_HIP_EUNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(bytes_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(counts_dev) % 8 != 0) return EP_HIP_EINVAL;
  const int64_t total_bytes = num_elements * num_lanes;
  int blocks = 0;
  const int status = ep::grid_for(total_bytes, 256 * 16 * 8, &blocks);
  if (status != EP_HIP_OK) return status;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(ep::zero_words_kernel, dim3(num_lanes), dim3(256), 0, s, reinterpret_cast<unsigned long long*>(counts_dev),
                     static_cast<int64_t>(num_lanes) * 256);
  hipLaunchKernelGGL(ep::byte_histogram_kernel, dim3(blocks), dim3(256), 0, s, bytes_dev, total_bytes, num_lanes,
                     reinterpret_cast<unsigned long long*>(counts_dev));
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

extern "C" int ep_hip_tile_ans_encode(const uint8_t* bytes_dev, int64_t num_elements, int num_lanes, int64_t tile_elements, int prob_bits,
                                      const uint64_t* entries_dev, const uint8_t* lane_raw_host, uint32_t* states_dev,
                                      uint32_t* stream_words_dev, uint16_t* scratch_dev, int64_t scratch_stride_words, int32_t* error_dev,
                                      void* stream) {
  if (bytes_dev == nullptr || entries_dev == nullptr || lane_raw_host == nullptr || stream_words_dev == nullptr || scratch_dev == nullptr ||
      error_dev == nullptr)
    return EP_HIP_EINVAL;
  if (num_elements <= 0 || tile_elements <= 0 || prob_bits < 1 || prob_bits > 15 || scratch_stride_words < tile_elements) return EP_HIP_EINVAL;
  if (num_lanes != 1 && num_lanes != 2 && num_lanes != 4 && num_lanes != 8) return EP_HIP_EUNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(entries_dev) % 8 != 0) return EP_HIP_EINVAL;
  unsigned raw_mask = 0;
  for (int b = 0; b < num_lanes; ++b) raw_mask |= (lane_raw_host[b] != 0 ? 1u : 0u) << b;
  if (raw_mask != (1u << num_lanes) - 1u && states_dev == nullptr) return EP_HIP_EINVAL;
  const int64_t tiles = (num_elements + tile_elements - 1) / tile_elements;
  const int64_t blocks = (tiles * num_lanes + 7) / 8;
  if (blocks > 0x7FFFFFFF) return EP_HIP_EUNSUPPORTED;
  const bool staged = (tile_elements * num_lanes) % 16 == 0 && reinterpret_cast<uintptr_t>(bytes_dev) % 16 == 0 &&
                      scratch_stride_words % 2 == 0 && reinterpret_cast<uintptr_t>(scratch_dev) % 4 == 0;
  if (staged)
    hipLaunchKernelGGL(ep::tile_ans_encode_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       bytes_dev, num_elements, num_lanes, tile_elements, tiles, prob_bits, raw_mask,
                       reinterpret_cast<const uint2*>(entries_dev), states_dev, stream_words_dev, scratch_dev, scratch_stride_words, error_dev);
  else
    hipLaunchKernelGGL(ep::tile_ans_encode_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       bytes_dev, num_elements, num_lanes, tile_elements, tiles, prob_bits, raw_mask,
                       reinterpret_cast<const uint2*>(entries_dev), states_dev, stream_words_dev, scratch_dev, scratch_stride_words, error_dev);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}
