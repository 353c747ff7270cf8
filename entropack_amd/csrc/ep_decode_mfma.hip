// Decode-to-GEMM in one kernel: y = x W^T with W a lattice_rans container, the decoded weight handed from the rANS
// lanes to the matrix cores through LDS and never written to memory (gfx950, wave64).
//
// The difficulty is that a tile is a serial chain (32 vectors per group of nine dependent steps, top of the tile
// first) and tiles are not aligned with weight rows, so at any moment the tiles of a container sit at unrelated
// k positions, while a matrix-core operand needs many weight rows at the SAME k. Two tiles whose first vectors lie at
// the same position inside a weight row (t * tile_vectors equal modulo vectors_per_row) stay aligned for their whole
// chain. The host therefore sorts the tiles by that position and hands each workgroup a batch of up to 32 tiles whose
// positions differ by at most 31 vectors (ep_hip_fused_plan): tile s of a batch, shifted by its `delta`, produces at
// chain step g the vectors with aligned index a in [32 g + delta, 32 g + delta + 32), and aligned index a means in-row
// vector position (base + a) mod vectors_per_row for every tile of the batch.
//
// Workgroup = 16 waves = 32 tiles (one per 32-lane half) x one block of 32 F activation rows. Per step:
//   1. every lane decodes one vector (the two-level tables and inline-assembly steps of the decode kernels), scales it,
//      rounds it to bf16 exactly as the store of the decode kernel would, and writes its 16 bytes into its tile's row of
//      an LDS ring of 128 vectors at position a mod 128 (lanes without a vector write zeros);
//   2. one workgroup barrier;
//   3. the window of 32 aligned positions that every tile has completed (one group behind the producers) is multiplied:
//      wave w < 2 F owns 32 activation rows (w mod F) and every second 16-wide k step (w / F); its A fragments are x
//      itself, requested straight into registers before the chain started; its B fragment is one ds_read_b128 per lane
//      of the ring (lane l: tile l mod 32, vector l / 32 of the step), i.e. 32 weight rows x 16 k per instruction
//      (v_mfma_f32_32x32x16_bf16). The accumulator column of tile s belongs to one weight row until the window crosses a
//      row boundary (all tiles of a batch cross it at the same aligned index); then the wave stores its 32 x 32 sums as
//      one of the row's partial-sum planes (no atomics: every tile of a row and both wave parities have their own plane)
//      and starts the next row.
// A ring row is written by its own half-wave only; the barrier orders the writes of step g before the reads of step g,
// and the ring depth (writers are at most 96 positions below the oldest reader) makes a second barrier unnecessary.
// A second kernel adds a row's planes and the bias and rounds once (finish_fused_planes_kernel).
#include "ep_decode_lds.hpp"

#include <algorithm>
#include <exception>
#include <vector>

namespace ep {

constexpr int kFusedRingDepth = 128;                                  // vectors per tile kept in LDS
// A ring row: 128 vectors of 16 bytes (bf16) or 8 bytes (int8 codes) + 16 bytes of padding, so that 16 tiles read at one
// position cover all banks.
constexpr uint32_t fused_row_bytes(bool int8) { return kFusedRingDepth * (int8 ? 8u : 16u) + 16u; }
constexpr int kFusedWaves = 16;

typedef __bf16 fused_bf16x8 __attribute__((ext_vector_type(8)));
typedef float fused_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t fused_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t fused_u32x2 __attribute__((ext_vector_type(2)));
typedef int fused_i32x4 __attribute__((ext_vector_type(4)));
typedef int fused_i32x16 __attribute__((ext_vector_type(16)));

inline int fused_lds_bytes(int prob_bits, bool int8) {
  return sym_table_bytes(prob_bits) + kFusedWaves * 2 * kRingBytes + EP_HIP_FUSED_SLOTS * static_cast<int>(fused_row_bytes(int8));
}

// The weights of the vector a lane just decoded with the two-level tables: (z + c / 2) * scale with one rounding,
// the same operations as the decode kernels' (their `weights_of` for these tables).
__device__ __forceinline__ void sym_weights(const Pair& s, float scale, float (&w)[8]) {
  const uint32_t folded = xor3(xor3(s.e[0], s.e[1], s.e[2]), xor3(s.e[3], s.e[4], s.e[5]), s.e[6]);
  const bool ordinary = __float_as_uint(scale) - 0x0DA24260u <= 0x7149F2CAu - 0x0DA24260u;      // 1e-30 <= scale <= 1e30
  if (__builtin_expect(ordinary, 1)) {
#pragma unroll
    for (int f = 0; f < 7; ++f) w[f] = mul_high_half(s.ey[f], scale);
    w[7] = __fmul_rn(twice_high_half_plus(s.ey[7], folded), scale);
  } else {
#pragma unroll
    for (int f = 0; f < 7; ++f) {
      const float z = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(s.ey[f] >> 16)));
      w[f] = __fmul_rn(__fadd_rn(z, 0.0f), scale);
    }
    w[7] = __fmul_rn(__fadd_rn(twice_high_half_plus(s.ey[7], folded), 0.0f), scale);
    if (__builtin_fabsf(scale) > 1.0e30f) {
#pragma unroll
      for (int f = 0; f < 8; ++f) w[f] = clamp_bf16(w[f]);
    }
  }
}

template <int PB, bool MASKED>
__device__ __forceinline__ void fused_chain(Pair& s, const StepConsts& k, bool valid_lane, uint64_t valid) {
  chain_priority();
  coset_step_single<PB, kModeSym, MASKED>(s, k, valid);
#pragma unroll
  for (int f = 0; f < kFields; ++f) {
    sym_step<PB, MASKED>(s, f, k, valid_lane);
    if ((f & 1) == 0 || f == kFields - 1) slide_window(s);
  }
  emit_priority();
}

// INT8: the container decodes to int8 codes (the int8 store's rounding and clamp), the activations are int8, the products
// are v_mfma_i32_32x32x32_i8 (a step is 32 k = four vectors, a wave takes four of a window's eight) and the planes hold
// exact int32 sums.
template <int PB, int F, bool INT8>
__global__ __launch_bounds__(1024) void decode_mfma_kernel(DecodeArgs a, const ep_hip_fused_batch* __restrict__ batches) {
  extern __shared__ __align__(16) uint8_t smem[];
  typedef __attribute__((address_space(3))) uint8_t* lds_ptr;
  typedef __attribute__((address_space(3))) fused_u32x4* lds_u4;
  typedef __attribute__((address_space(3))) fused_u32x2* lds_u2;
  constexpr uint32_t kTables = static_cast<uint32_t>(sym_table_bytes(PB));
  constexpr uint32_t kTable = 1u << PB;
  constexpr uint32_t kVectorBytes = INT8 ? 8u : 16u;
  constexpr uint32_t kRowBytes = fused_row_bytes(INT8);
  constexpr int kStepVectors = INT8 ? 4 : 2;           // vectors one matrix-core instruction multiplies (32 or 16 k)
  constexpr int kWaveSteps = INT8 ? 4 : 8;             // steps of a window one wave takes (every second one)
  static_assert(F == 1 || F == 2 || F == 4 || F == 8, "32 F activation rows per workgroup, two waves per 32");

  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr)smem));
  if (lds0 != 0) {          // the steps address the tables from LDS offset 0
    if (threadIdx.x == 0) flag_error(a.error, EP_DECODE_BAD_OFFSETS);
    return;
  }
  const uint32_t windows0 = kTables;
  const uint32_t ring0 = windows0 + kFusedWaves * 2 * kRingBytes;

  const ep_hip_fused_batch& batch = batches[blockIdx.x];
  const int vpr = a.vecs_per_row;
  const int tv = a.tile_vectors;
  const int groups = (tv + 31) >> 5;
  const int rows_total = static_cast<int>(a.num_vectors / vpr);
  // In-row vector position of the window's first aligned index; windows go down by 32 per step. Checked before anything
  // is in flight into LDS: a workgroup must not end with loads on their way into memory that is no longer its own.
  int q0 = __builtin_amdgcn_readfirstlane(static_cast<int>((static_cast<int64_t>(batch.base) + 32 * groups) % vpr));
  if (q0 < 0 || (q0 & (kStepVectors - 1)) != 0) {        // a batch table that is not ep_hip_fused_plan's: nothing below may index with it
    if (threadIdx.x == 0) flag_error(a.error, EP_DECODE_BAD_OFFSETS);
    return;
  }

  // Tables: memory -> LDS without registers in between, left in flight during the set-up below.
  for (uint32_t kib = static_cast<uint32_t>(wave); kib < kTables / 1024u; kib += kFusedWaves) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.sym_tables + kib * 1024u + static_cast<uint32_t>(lane) * 16u),
                                     (__attribute__((address_space(3))) void*)(smem + kib * 1024u), 16, 0, 0);
  }

  StepConsts k;
  k.f0s = uniform(a.plan[kHdrCosetFreq0]);
  k.f0v = k.f0s;
  k.f1v = kTable - k.f0s;
  k.ktab = static_cast<uint32_t>(kSymFbStreamBytes);
  k.shv = half ? 16u : 0u;
  asm volatile("" : "+v"(k.f0v), "+v"(k.f1v), "+v"(k.ktab), "+v"(k.shv));

  // ---- this half's tile ------------------------------------------------------------------------------------------
  const int slot = 2 * wave + half;
  const int tile = batch.tile[slot];
  const int delta = batch.delta[slot];
  Pair s;
  s.count = 0;
  s.x = kStateMin;
  s.vector0 = 0;
  s.coset_base = 0;
  s.coset_mask = 0;
  uint32_t word_begin = 0, word_end = 0;
  if (tile >= 0 && tile < a.num_tiles) {
    word_begin = a.offsets[tile];
    word_end = a.offsets[tile + 1];
    const int64_t v0 = static_cast<int64_t>(tile) * tv;
    const int64_t left = a.num_vectors - v0;
    s.vector0 = static_cast<uint32_t>(v0);
    s.count = static_cast<int>(left < tv ? left : tv);
    if (word_begin > word_end || word_end > a.payload_words) {
      flag_error(a.error, EP_DECODE_BAD_OFFSETS);
      s.count = 0;
      word_begin = word_end = 0;
    } else {
      s.x = a.states[static_cast<int64_t>(tile) * kStatesPerTile + l32];
    }
  }
  open_window(s, windows0 + static_cast<uint32_t>(slot) * kRingBytes, word_begin, word_end, s.count > 0, a.payload, a.payload_words, a.offsets, l32);
  const uint32_t my_row = ring0 + static_cast<uint32_t>(slot) * kRowBytes;
  auto ring_store = [&](int aligned, fused_u32x4 value) {       // int8: the first two words
    if (aligned >= 0) {
      const uint32_t at = my_row + (static_cast<uint32_t>(aligned) & (kFusedRingDepth - 1)) * kVectorBytes;
      if constexpr (INT8) *reinterpret_cast<lds_u2>(static_cast<uintptr_t>(at)) = fused_u32x2{value[0], value[1]};
      else *reinterpret_cast<lds_u4>(static_cast<uintptr_t>(at)) = value;
    }
  };

  // ---- this wave's share of the products ----------------------------------------------------------------------------
  const bool multiplies = wave < 2 * F;
  const int fragment = wave % F, parity = wave / F;        // 32 activation rows, and which of every two k steps
  const int m_first = static_cast<int>(blockIdx.y) * 32 * F + 32 * fragment;
  // a.x = the activations repacked by pack_activations_kernel: [k step][activation row][32 bytes] (16 bf16 or 32 int8
  // values), so that the 32 rows of a fragment are 1 KiB of consecutive memory (a.ldx = rows per k step, a multiple of 32 F).
  const uint8_t* x_row = reinterpret_cast<const uint8_t*>(a.x) + static_cast<int64_t>(m_first + l32) * 32 + half * 16;
  const int64_t x_block_bytes = a.ldx * 32;
  const uint32_t read_row = ring0 + static_cast<uint32_t>(l32) * kRowBytes;
  // The accumulator column l32 holds tile `l32` of the batch. row_now = the weight row that column is summing: that of
  // the position just above the first window, lowered by one at every row boundary the windows cross.
  const int column_tile = batch.tile[l32];
  const bool column_live = column_tile >= 0 && column_tile < a.num_tiles;
  int row_now = -1;
  if (column_live) {
    row_now = static_cast<int>((static_cast<int64_t>(column_tile) * tv - batch.delta[l32] + 32 * groups + 32) / vpr);
  }
  using Acc = typename std::conditional<INT8, fused_i32x16, fused_f32x16>::type;
  Acc acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0;
  // A column's sums for one weight row are one of several partial sums of that row: a row touches up to `planes` tiles,
  // and two waves share a fragment's k steps. Every (tile of the row, wave parity) has its own plane of the workspace,
  // laid out [plane][weight row][activation row]: a lane's four consecutive activation rows are 16 contiguous bytes, a
  // column's 32 rows one 128-byte line, written with plain stores; the finishing kernel adds the planes.
  auto flush = [&]() {
    if (column_live && row_now >= 0 && row_now < rows_total) {
      const int64_t row_first = static_cast<int64_t>(row_now) * vpr;
      const int64_t tile_first = static_cast<int64_t>(column_tile) * tv;
      const int64_t tile_end = tile_first + tv < a.num_vectors ? tile_first + tv : a.num_vectors;
      if (tile_first < row_first + vpr && tile_end > row_first) {        // the tile holds vectors of this row
        const int plane = 2 * (column_tile - static_cast<int>(row_first / tv)) + parity;
        float* at = a.y32 + (static_cast<int64_t>(plane) * rows_total + row_now) * a.ldy32 + m_first + 4 * half;
#pragma unroll
        for (int q = 0; q < 4; ++q) {          // int8: the same cells hold int32 sums
          typedef typename std::conditional<INT8, fused_i32x4, float __attribute__((ext_vector_type(4)))>::type Cell4;
          *reinterpret_cast<Cell4*>(at + 8 * q) = Cell4{acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0;
    row_now -= 1;
  };

  // Positions above the tile's top group (read by the first window) start as zeros.
  ring_store(32 * groups + l32 + delta, fused_u32x4{0, 0, 0, 0});
  __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): this wave's part of the tables has landed
  __syncthreads();

#pragma unroll 1
  for (int g = groups - 1; g >= -1; --g) {
    // The activations of the window this step completes, aligned indices [32 (g + 1), 32 (g + 2)): 16 bytes per lane and
    // k step, requested now and used after the chain.
    fused_u32x4 xa[kWaveSteps];
    if (multiplies) {
#pragma unroll
      for (int j = 0; j < kWaveSteps; ++j) {
        int q = q0 + kStepVectors * (2 * j + parity);
        q = q >= vpr ? q - vpr : q;
        xa[j] = *reinterpret_cast<const fused_u32x4*>(x_row + static_cast<int64_t>(q / kStepVectors) * x_block_bytes);
      }
    }

    const int first = 32 * g;
    const bool valid_lane = g >= 0 && first + l32 < s.count;
    const uint64_t valid = __builtin_amdgcn_ballot_w64(valid_lane);
    fused_u32x4 packed = {0, 0, 0, 0};
    if (valid != 0) {
      const uint32_t vector = s.vector0 + static_cast<uint32_t>(valid_lane ? first + l32 : 0);
      const float scale = valid_lane ? a.scales[row_of(a, vector)] : 0.0f;
      if (valid == ~0ull) fused_chain<PB, false>(s, k, true, valid);
      else fused_chain<PB, true>(s, k, valid_lane, valid);
      float w[8];
      sym_weights(s, scale, w);
      if constexpr (INT8) {
        uint32_t low, high;
        codes_i8(w, low, high);
        packed[0] = valid_lane ? low : 0u;
        packed[1] = valid_lane ? high : 0u;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          typedef float float2v __attribute__((ext_vector_type(2)));
          typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
          const float2v two = {w[2 * i], w[2 * i + 1]};
          packed[i] = valid_lane ? __builtin_bit_cast(uint32_t, __builtin_convertvector(two, bf16x2)) : 0u;
        }
      }
    }
    ring_store(first + l32 + delta, packed);
    __syncthreads();

    if (multiplies) {
      const uint32_t window = static_cast<uint32_t>(32 * (g + 1));
      const bool crossing = q0 + 32 >= vpr;                 // a row ends inside this window, or exactly at its top
      const int boundary = crossing ? vpr - q0 : 64;        // window-relative index of the upper row's first vector
      auto multiply = [&](int j) {       // a lane's 16 bytes: one bf16 vector, or two consecutive vectors of int8 codes
        const uint32_t at = (window + static_cast<uint32_t>(kStepVectors * (2 * j + parity) + (kStepVectors / 2) * half)) & (kFusedRingDepth - 1);
        const fused_u32x4 b = *reinterpret_cast<lds_u4>(static_cast<uintptr_t>(read_row + at * kVectorBytes));
        if constexpr (INT8) {
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(fused_i32x4, xa[j]), __builtin_bit_cast(fused_i32x4, b), acc, 0, 0, 0);
        } else {
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(fused_bf16x8, xa[j]), __builtin_bit_cast(fused_bf16x8, b), acc, 0, 0, 0);
        }
      };
      if (!crossing) {
#pragma unroll
        for (int j = 0; j < kWaveSteps; ++j) multiply(j);
      } else {
#pragma unroll
        for (int j = 0; j < kWaveSteps; ++j) {
          if (kStepVectors * (2 * j + parity) >= boundary) multiply(j);
        }
        flush();
#pragma unroll
        for (int j = 0; j < kWaveSteps; ++j) {
          if (kStepVectors * (2 * j + parity) < boundary) multiply(j);
        }
      }
    }
    q0 -= 32;
    q0 = q0 < 0 ? q0 + vpr : q0;
  }
  if (multiplies) flush();

  // A valid tile ends with every word consumed and every lane back at the encoder's initial state.
  const uint64_t stale = __builtin_amdgcn_ballot_w64(s.count > 0 && s.x != kStateMin);
  const uint64_t live = __builtin_amdgcn_ballot_w64(s.count > 0);
  const bool liveA = (live & 1u) != 0, liveB = ((live >> 32) & 1u) != 0;
  const int ptrA = window_pointer_a(s), ptrB = window_pointer_b(s);
  const bool badA = liveA && (ptrA != s.beginA || static_cast<uint32_t>(stale) != 0);
  const bool badB = liveB && (ptrB != s.beginB || static_cast<uint32_t>(stale >> 32) != 0);
  if ((badA || badB) && lane == 0) {
    const bool over = (liveA && ptrA < s.beginA) || (liveB && ptrB < s.beginB);
    flag_error(a.error, over ? EP_DECODE_OVERREAD : EP_DECODE_NOT_CONSUMED);
  }
}

// x[m][32-byte steps of a row] (row stride in bytes) -> packed[step][m][32 bytes], rows m_rows .. m_padded - 1 zero: 16
// bf16 or 32 int8 activations per step. One thread per 32 bytes.
__global__ __launch_bounds__(256) void pack_activations_kernel(const uint8_t* __restrict__ x, int64_t row_bytes, int m_rows, int64_t m_padded,
                                                               int k_steps, uint8_t* __restrict__ packed) {
  const int64_t index = blockIdx.x * int64_t{256} + threadIdx.x;
  if (index >= m_padded * k_steps) return;
  const int64_t m = index % m_padded, step = index / m_padded;
  uint4 low = make_uint4(0, 0, 0, 0), high = low;
  if (m < m_rows) {
    const uint4* from = reinterpret_cast<const uint4*>(x + m * row_bytes + step * 32);
    low = from[0];
    high = from[1];
  }
  uint4* to = reinterpret_cast<uint4*>(packed + index * 32);
  to[0] = low;
  to[1] = high;
}

// Tiles a weight row of `vpr` vectors can touch when tiles hold `tv` vectors.
inline int fused_planes_per_row(int64_t vpr, int tv) { return 1 + static_cast<int>((vpr - 1 + tv - 1) / tv); }

// y[m][n] = cast(sum of the partial-sum planes of weight row n + bias[n]). Workspace layout [plane][n][m_padded]; row n
// was written by tiles first_tile(n) .. last_tile(n), two planes (wave parities) each. A block transposes a 32 x 32 patch
// through LDS so that both the reads (along m) and the writes (along n) are contiguous. INT8: the planes hold int32 sums,
// added exactly, then f32(sum) * scale_a[m] * scale_b[n] + bias[n] as three single-rounded operations (the epilogue of the
// int8 GEMM kernels, entropack/linear/quant_kernels.py:15-54 of the reference).
template <bool INT8>
__global__ __launch_bounds__(256) void finish_fused_planes_kernel(const float* __restrict__ y32, const float* __restrict__ scale_a,
                                                                  const float* __restrict__ scale_b, const void* __restrict__ bias,
                                                                  void* __restrict__ y, int m_rows, int64_t m_padded, int outer, int vpr, int tv,
                                                                  int64_t ldy, int out_kind) {
  __shared__ float patch[32][33];
  const int n0 = static_cast<int>(blockIdx.x) * 32, m0 = static_cast<int>(blockIdx.y) * 32;
  const int lane_m = threadIdx.x & 31, group = threadIdx.x >> 5;          // 8 groups of 32 threads
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = n0 + group * 4 + i;
    float sum = 0.0f;
    if (n < outer && m0 + lane_m < m_padded) {
      const int64_t row_first = static_cast<int64_t>(n) * vpr;
      const int tiles = static_cast<int>((row_first + vpr - 1) / tv) - static_cast<int>(row_first / tv) + 1;
      if constexpr (INT8) {
        int total = 0;
        for (int plane = 0; plane < 2 * tiles; ++plane) {
          total += reinterpret_cast<const int*>(y32)[(static_cast<int64_t>(plane) * outer + n) * m_padded + m0 + lane_m];
        }
        sum = static_cast<float>(total);
      } else {
        for (int plane = 0; plane < 2 * tiles; ++plane) sum += y32[(static_cast<int64_t>(plane) * outer + n) * m_padded + m0 + lane_m];
      }
    }
    patch[group * 4 + i][lane_m] = sum;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + group * 4 + i, n = n0 + lane_m;
    if (m >= m_rows || n >= outer) continue;
    float v = patch[lane_m][group * 4 + i];
    if constexpr (INT8) v = __fmul_rn(__fmul_rn(v, scale_a[m]), scale_b[n]);
    if (bias != nullptr) {
      float add;
      if (out_kind == EP_FLOAT_BF16) add = __uint_as_float(static_cast<uint32_t>(static_cast<const uint16_t*>(bias)[n]) << 16);
      else if (out_kind == EP_FLOAT_F16) add = static_cast<float>(static_cast<const _Float16*>(bias)[n]);
      else add = static_cast<const float*>(bias)[n];
      v = __fadd_rn(v, add);
    }
    if (out_kind == EP_FLOAT_BF16) static_cast<uint16_t*>(y)[m * ldy + n] = static_cast<uint16_t>(bf16_bits_rne(v));
    else if (out_kind == EP_FLOAT_F16) static_cast<_Float16*>(y)[m * ldy + n] = static_cast<_Float16>(v);
    else static_cast<float*>(y)[m * ldy + n] = v;
  }
}

template <int PB, int F, bool INT8>
static int launch_fused_one(const DecodeArgs& args, const ep_hip_fused_batch* batches, int n_batches, int m_blocks, hipStream_t stream) {
  static thread_local int configured_for = -1;
  const int status = allow_full_lds(reinterpret_cast<const void*>(decode_mfma_kernel<PB, F, INT8>), configured_for);
  if (status != EP_HIP_OK) return status;
  hipLaunchKernelGGL((decode_mfma_kernel<PB, F, INT8>), dim3(static_cast<unsigned>(n_batches), static_cast<unsigned>(m_blocks)), dim3(1024),
                     static_cast<size_t>(fused_lds_bytes(PB, INT8)), stream, args, batches);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

int fused_rows_per_block(int64_t m_rows) { return m_rows <= 32 ? 32 : (m_rows <= 64 ? 64 : (m_rows <= 128 ? 128 : 256)); }

static int64_t fused_padded_rows(int64_t m_rows) {
  const int per_block = fused_rows_per_block(m_rows);
  return (m_rows + per_block - 1) / per_block * per_block;
}
static size_t fused_plane_bytes(int64_t rows, int64_t cols_padded, int tile_elements, int64_t m_rows) {
  const size_t bytes = static_cast<size_t>(2 * fused_planes_per_row(cols_padded / 8, tile_vectors_of(tile_elements))) * static_cast<size_t>(rows) *
                       static_cast<size_t>(fused_padded_rows(m_rows)) * 4;
  return (bytes + 255) / 256 * 256;
}
// The partial-sum planes, then the repacked activations (`element_bytes` each: 2 for bf16, 1 for int8).
size_t fused_workspace_bytes(int64_t rows, int64_t cols_padded, int tile_elements, int64_t m_rows, int element_bytes) {
  return fused_plane_bytes(rows, cols_padded, tile_elements, m_rows) +
         static_cast<size_t>(fused_padded_rows(m_rows)) * static_cast<size_t>(cols_padded) * static_cast<size_t>(element_bytes);
}

template <bool INT8>
static int launch_fused_kind(DecodeArgs args, const ep_hip_fused_batch* batches, int n_batches, const float* scale_a, const float* scale_b,
                             const void* bias, void* y, int64_t ldy, int out_kind, hipStream_t stream) {
  const int m = args.m_rows;
  const int per_block = fused_rows_per_block(m);
  const int m_blocks = (m + per_block - 1) / per_block;
  if (m_blocks > 65535) return EP_HIP_EUNSUPPORTED;
  args.ldy32 = static_cast<int64_t>(m_blocks) * per_block;          // activation rows per workspace row
  const int64_t cols_padded = static_cast<int64_t>(args.vecs_per_row) * 8;
  const int outer = static_cast<int>(args.num_vectors / args.vecs_per_row);
  uint8_t* packed = reinterpret_cast<uint8_t*>(args.y32) + fused_plane_bytes(outer, cols_padded, args.tile_vectors * 9, m);
  {
    const int element_bytes = INT8 ? 1 : 2;
    const int k_steps = static_cast<int>(cols_padded * element_bytes / 32);
    const int64_t threads = args.ldy32 * k_steps;
    hipLaunchKernelGGL(pack_activations_kernel, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const uint8_t*>(args.x), args.ldx * element_bytes, m, args.ldy32, k_steps, packed);
    EP_HIP_TRY(hipGetLastError());
    args.x = reinterpret_cast<const uint16_t*>(packed);
    args.ldx = args.ldy32;
  }
  int status;
  switch (per_block / 32) {
    case 1: status = launch_fused_one<11, 1, INT8>(args, batches, n_batches, m_blocks, stream); break;
    case 2: status = launch_fused_one<11, 2, INT8>(args, batches, n_batches, m_blocks, stream); break;
    case 4: status = launch_fused_one<11, 4, INT8>(args, batches, n_batches, m_blocks, stream); break;
    default: status = launch_fused_one<11, 8, INT8>(args, batches, n_batches, m_blocks, stream); break;
  }
  if (status != EP_HIP_OK) return status;
  const dim3 grid(static_cast<unsigned>((outer + 31) / 32), static_cast<unsigned>((m + 31) / 32));
  hipLaunchKernelGGL(finish_fused_planes_kernel<INT8>, grid, dim3(256), 0, stream, args.y32, scale_a, scale_b, bias, y, m, args.ldy32, outer,
                     args.vecs_per_row, args.tile_vectors, ldy, out_kind);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

// args.x / args.ldx: the activations as the caller holds them (bf16, or int8 codes with scale_a / scale_b given).
int launch_fused_mfma(const DecodeArgs& args, const ep_hip_plan_desc& desc, const ep_hip_fused_batch* batches, int n_batches, bool int8,
                      const float* scale_a, const float* scale_b, const void* bias, void* y, int64_t ldy, int out_kind, hipStream_t stream) {
  if (desc.prob_bits != 11 || args.sym_tables == nullptr) return EP_HIP_EUNSUPPORTED;       // the two-level tables of prob_bits 11 plans
  if (args.vecs_per_row < 32 || args.vecs_per_row % 4 != 0 || n_batches <= 0 || args.m_rows <= 0) return EP_HIP_EUNSUPPORTED;
  if (int8) return launch_fused_kind<true>(args, batches, n_batches, scale_a, scale_b, bias, y, ldy, out_kind, stream);
  return launch_fused_kind<false>(args, batches, n_batches, nullptr, nullptr, bias, y, ldy, out_kind, stream);
}

}  // namespace ep

extern "C" int ep_hip_fused_plan(int64_t rows, int64_t cols_padded, int tile_elements, ep_hip_fused_batch* batches_host, int capacity,
                                 int* n_batches) {
  using namespace ep;
  if (rows <= 0 || cols_padded <= 0 || cols_padded % 8 != 0 || tile_elements <= 0 || n_batches == nullptr || capacity < 0) return EP_HIP_EINVAL;
  const int64_t vpr = cols_padded / 8;
  const int tv = tile_vectors_of(tile_elements);
  const int64_t vectors = rows * vpr;
  const int64_t tiles = (vectors + tv - 1) / tv;
  if (vpr < 32 || vpr % 4 != 0 || vpr > 0x7FFFFFFF || vectors >= (int64_t{1} << 31) || tiles >= (int64_t{1} << 30)) return EP_HIP_EUNSUPPORTED;
  std::vector<std::pair<int32_t, int32_t>> order;      // (position of the tile's first vector in its row, tile)
  try {
    order.resize(static_cast<size_t>(tiles));
  } catch (const std::exception&) {                   // no exception leaves the C ABI
    return EP_HIP_EINVAL;
  }
  for (int64_t t = 0; t < tiles; ++t) order[static_cast<size_t>(t)] = {static_cast<int32_t>((t * tv) % vpr), static_cast<int32_t>(t)};
  std::sort(order.begin(), order.end());
  int count = 0;
  size_t at = 0;
  while (at < order.size()) {
    const int32_t base = order[at].first & ~3;        // a multiple of 4: a k step (two vectors of bf16, four of int8 codes) never straddles a row boundary
    size_t end = at;
    while (end < order.size() && end - at < EP_HIP_FUSED_SLOTS && order[end].first - base <= EP_HIP_FUSED_MAX_SKEW) ++end;
    if (batches_host != nullptr) {
      if (count >= capacity) return EP_HIP_EINVAL;
      ep_hip_fused_batch& b = batches_host[count];
      b.base = base;
      b.reserved[0] = b.reserved[1] = b.reserved[2] = 0;
      for (int slot = 0; slot < EP_HIP_FUSED_SLOTS; ++slot) {
        const bool used = at + static_cast<size_t>(slot) < end;
        b.tile[slot] = used ? order[at + static_cast<size_t>(slot)].second : -1;
        b.delta[slot] = used ? order[at + static_cast<size_t>(slot)].first - base : 0;
      }
    }
    ++count;
    at = end;
  }
  *n_batches = count;
  return EP_HIP_OK;
}
