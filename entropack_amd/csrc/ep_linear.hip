// The consumers of decoded weights: MFMA GEMMs for gfx950 and the activation row quantiser.
//
//   gemm_bf16_nt_kernel   y[M,N] = x[M,K] . w[N,K]^T (+ bias[N]), bf16 operands, f32 accumulation in
//                         v_mfma_f32_32x32x16_bf16, one bf16 rounding at the end (what F.linear does in the
//                         reference's forward, entropack/linear/linear.py:163-165).
//   gemm_i8_nt_kernel     y[M,N] = (a[M,K] . b[N,K]^T)_i32 -> f32 * sa[m] * sb[n] (+ bias[n]) -> out dtype, with
//                         v_mfma_i32_32x32x32_i8 (semantics of the reference's Triton kernel,
//                         entropack/linear/quant_kernels.py:15-54).
//   quantize_rows_kernel  per row: scale = max(absmax / 127, eps_f32), code = clamp(rint(x / scale), +-127)
//                         (entropack/linear/quant_kernels.py:56-79).
//
// Both GEMMs are "NT": each operand row is contiguous in K, which is exactly the MFMA fragment shape (a lane holds
// 8 bf16 / 16 int8 consecutive in K of one row), so tiles go global -> LDS -> fragment with 16-byte accesses only.
// Block tile 128 x 128 x 64 (bf16) or 128 x 128 x 128 (int8), 4 waves in a 2 x 2 arrangement, each wave 64 x 64 as
// 2 x 2 MFMA tiles; the next K tile is fetched into registers while the current one is multiplied.
#include <type_traits>

#include "ep_common.hpp"

namespace ep {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

constexpr int kBlockM = 128, kBlockN = 128;
constexpr int kTileBytesK = 128;                 // bytes of K per tile row: 64 bf16 or 128 int8
constexpr int kRowStride = kTileBytesK + 16;     // padded LDS row: 16-byte reads of 32 consecutive rows spread over banks
constexpr int kChunksPerRow = kTileBytesK / 16;

enum : int { kOutBF16 = 0, kOutF16 = 1, kOutF32 = 2 };

__device__ __forceinline__ uint32_t bf16_bits_of(float v) {
  typedef float float2v __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const float2v two = {v, 0.0f};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(two, bf16x2)) & 0xFFFFu;
}

__device__ __forceinline__ void store_out(void* y, int kind, int64_t at, float v) {
  if (kind == kOutBF16) reinterpret_cast<uint16_t*>(y)[at] = static_cast<uint16_t>(bf16_bits_of(v));
  else if (kind == kOutF16) reinterpret_cast<_Float16*>(y)[at] = static_cast<_Float16>(v);
  else reinterpret_cast<float*>(y)[at] = v;
}

__device__ __forceinline__ float load_bias(const void* bias, int kind, int n) {
  if (kind == kOutBF16) return __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(bias)[n]) << 16);
  if (kind == kOutF16) return static_cast<float>(reinterpret_cast<const _Float16*>(bias)[n]);
  return reinterpret_cast<const float*>(bias)[n];
}

// Shared skeleton. ELEM = bytes per operand element (2 = bf16, 1 = int8). Operand rows are `ld*` elements apart.
template <int ELEM>
struct TileLoader {
  // Each of the 256 threads moves 4 chunks of 16 bytes per operand tile: chunk c covers row c / 8, bytes 16 (c % 8).
  uint4 reg[4];

  __device__ __forceinline__ void fetch(const uint8_t* base, int64_t ld_bytes, int row0, int rows, int64_t k_byte0,
                                        int64_t k_bytes, int tid) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int chunk = tid + 256 * i;
      const int r = chunk / kChunksPerRow;
      const int64_t kb = k_byte0 + 16 * (chunk % kChunksPerRow);
      uint4 v = make_uint4(0, 0, 0, 0);
      if (row0 + r < rows && kb < k_bytes) v = *reinterpret_cast<const uint4*>(base + (row0 + r) * ld_bytes + kb);
      reg[i] = v;
    }
  }

  __device__ __forceinline__ void stash(uint8_t* tile, int tid) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int chunk = tid + 256 * i;
      *reinterpret_cast<uint4*>(tile + (chunk / kChunksPerRow) * kRowStride + 16 * (chunk % kChunksPerRow)) = reg[i];
    }
  }
};

__global__ __launch_bounds__(256) void gemm_bf16_nt_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                           const void* __restrict__ bias, void* __restrict__ y, int M,
                                                           int N, int K, int64_t ldx, int64_t ldw, int64_t ldy,
                                                           int out_kind) {
  __shared__ __align__(16) uint8_t tile_a[kBlockM * kRowStride];
  __shared__ __align__(16) uint8_t tile_b[kBlockN * kRowStride];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;
  const int m0 = blockIdx.y * kBlockM, n0 = blockIdx.x * kBlockN;
  const uint8_t* xa = reinterpret_cast<const uint8_t*>(x);
  const uint8_t* wb = reinterpret_cast<const uint8_t*>(w);
  const int64_t k_bytes = static_cast<int64_t>(K) * 2;

  f32x16 acc[2][2] = {};
  TileLoader<2> la, lb;
  la.fetch(xa, ldx * 2, m0, M, 0, k_bytes, tid);
  lb.fetch(wb, ldw * 2, n0, N, 0, k_bytes, tid);
  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 16;             // byte offset of this lane's 8 bf16 inside a 16-element K step

  for (int64_t kb = 0; kb < k_bytes; kb += kTileBytesK) {
    __syncthreads();                                // everyone is done reading the previous tile
    la.stash(tile_a, tid);
    lb.stash(tile_b, tid);
    __syncthreads();
    if (kb + kTileBytesK < k_bytes) {               // fetch the next tile while this one is multiplied
      la.fetch(xa, ldx * 2, m0, M, kb + kTileBytesK, k_bytes, tid);
      lb.fetch(wb, ldw * 2, n0, N, kb + kTileBytesK, k_bytes, tid);
    }
#pragma unroll
    for (int kk = 0; kk < kTileBytesK / 32; ++kk) {
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        fa[t] = *reinterpret_cast<const bf16x8*>(tile_a + (wave_m * 64 + t * 32 + frag_row) * kRowStride + kk * 32 + frag_k);
        fb[t] = *reinterpret_cast<const bf16x8*>(tile_b + (wave_n * 64 + t * 32 + frag_row) * kRowStride + kk * 32 + frag_k);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  }

  // Accumulator layout of a 32 x 32 tile: register r of lane l holds row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32.
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wave_n * 64 + j * 32 + (lane & 31);
      if (n >= N) continue;
      const float b = bias != nullptr ? load_bias(bias, out_kind, n) : 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wave_m * 64 + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        if (m < M) store_out(y, out_kind, static_cast<int64_t>(m) * ldy + n, acc[i][j][r] + b);
      }
    }
  }
}

__global__ __launch_bounds__(256) void gemm_i8_nt_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ b,
                                                         const float* __restrict__ scale_a, const float* __restrict__ scale_b,
                                                         const void* __restrict__ bias, void* __restrict__ y, int M, int N,
                                                         int K, int64_t lda, int64_t ldb, int64_t ldy, int out_kind) {
  __shared__ __align__(16) uint8_t tile_a[kBlockM * kRowStride];
  __shared__ __align__(16) uint8_t tile_b[kBlockN * kRowStride];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;
  const int m0 = blockIdx.y * kBlockM, n0 = blockIdx.x * kBlockN;
  const uint8_t* pa = reinterpret_cast<const uint8_t*>(a);
  const uint8_t* pb = reinterpret_cast<const uint8_t*>(b);
  const int64_t k_bytes = K;

  i32x16 acc[2][2] = {};
  TileLoader<1> la, lb;
  la.fetch(pa, lda, m0, M, 0, k_bytes, tid);
  lb.fetch(pb, ldb, n0, N, 0, k_bytes, tid);
  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 16;             // this lane's 16 int8 inside a 32-element K step

  for (int64_t kb = 0; kb < k_bytes; kb += kTileBytesK) {
    __syncthreads();
    la.stash(tile_a, tid);
    lb.stash(tile_b, tid);
    __syncthreads();
    if (kb + kTileBytesK < k_bytes) {
      la.fetch(pa, lda, m0, M, kb + kTileBytesK, k_bytes, tid);
      lb.fetch(pb, ldb, n0, N, kb + kTileBytesK, k_bytes, tid);
    }
#pragma unroll
    for (int kk = 0; kk < kTileBytesK / 32; ++kk) {
      i32x4 fa[2], fb[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        fa[t] = *reinterpret_cast<const i32x4*>(tile_a + (wave_m * 64 + t * 32 + frag_row) * kRowStride + kk * 32 + frag_k);
        fb[t] = *reinterpret_cast<const i32x4*>(tile_b + (wave_n * 64 + t * 32 + frag_row) * kRowStride + kk * 32 + frag_k);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  }

#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wave_n * 64 + j * 32 + (lane & 31);
      if (n >= N) continue;
      const float sb = scale_b[n];
      const bool has_bias = bias != nullptr;
      const float bv = has_bias ? load_bias(bias, out_kind, n) : 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wave_m * 64 + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        if (m < M) {
          // int32 -> f32, times the activation row scale, times the weight row scale, plus bias: in that order,
          // each a single rounded float operation.
          float v = __fmul_rn(__fmul_rn(static_cast<float>(acc[i][j][r]), scale_a[m]), sb);
          if (has_bias) v = __fadd_rn(v, bv);
          store_out(y, out_kind, static_cast<int64_t>(m) * ldy + n, v);
        }
      }
    }
  }
}

// One block per row. in_kind: kOutBF16 / kOutF16 / kOutF32 naming the activation dtype.
__global__ __launch_bounds__(256) void quantize_rows_kernel(const void* __restrict__ x, int in_kind, int64_t ldx, int K,
                                                            int8_t* __restrict__ codes, float* __restrict__ scales) {
  __shared__ float partial[4];
  const int64_t row = blockIdx.x;
  auto value = [&](int k) -> float {
    if (in_kind == kOutBF16) return __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(x)[row * ldx + k]) << 16);
    if (in_kind == kOutF16) return static_cast<float>(reinterpret_cast<const _Float16*>(x)[row * ldx + k]);
    return reinterpret_cast<const float*>(x)[row * ldx + k];
  };
  float top = 0.0f;
  for (int k = threadIdx.x; k < K; k += blockDim.x) top = __builtin_fmaxf(top, __builtin_fabsf(value(k)));
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) top = __builtin_fmaxf(top, __shfl_xor(top, offset));
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = top;
  __syncthreads();
  top = __builtin_fmaxf(__builtin_fmaxf(partial[0], partial[1]), __builtin_fmaxf(partial[2], partial[3]));
  const float scale = __builtin_fmaxf(top / 127.0f, 1.1920928955078125e-07f);
  for (int k = threadIdx.x; k < K; k += blockDim.x) {
    const float q = __builtin_fminf(__builtin_fmaxf(__builtin_rintf(value(k) / scale), -127.0f), 127.0f);
    codes[row * K + k] = static_cast<int8_t>(q);
  }
  if (threadIdx.x == 0) scales[row] = scale;
}

// Plain quantisation of two-byte activations, one wave per row (four rows per block): no LDS, no barrier, the row read
// once with fully coalesced 16-byte loads (chunk c of lane l holds elements 8 (64 c + l) .. + 8) and kept packed in
// registers between the absmax and the codes. The codes are rint(v / scale) with IEEE division by definition; dividing
// 12 M activations costs more vector instructions than everything else in this kernel together, so a chunk first forms
// t = v * (1 / scale), which lies within 127.5 * 2^-23 of the true quotient, as does the correctly rounded quotient itself:
// unless t is closer than 2^-14 to a half-integer the two round to the same integer. Chunks in which some lane's value is
// that close (about one in sixteen) are redone with the division; the result is the definition's, bit for bit, either way.
template <int IN_KIND, int CHUNKS>
__global__ __launch_bounds__(256) void quantize_rows_wave_kernel(const uint16_t* __restrict__ x, int64_t ldx, int K, int rows,
                                                                 int8_t* __restrict__ codes, float* __restrict__ scales) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
  const int lane = threadIdx.x & 63;
  const int64_t row = blockIdx.x * int64_t{4} + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint16_t* from = x + row * ldx;
  auto value_of_bits = [](uint32_t bits) -> float {       // bits: a two-byte pattern in the low half
    if constexpr (IN_KIND == kOutBF16) return __uint_as_float(bits << 16);
    else return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits)));
  };
  auto value = [&](uint32_t word, int high) -> float {
    if constexpr (IN_KIND == kOutBF16) return __uint_as_float(high ? word & 0xFFFF0000u : word << 16);
    else return value_of_bits(high ? word >> 16 : word & 0xFFFFu);
  };
  // The row's largest magnitude, found on the bit patterns: without its sign bit a bf16 or f16 pattern grows with the
  // magnitude it stands for (a NaN counts as larger than every number), two elements per instruction.
  u32x4 held[CHUNKS];
  u16x2 top2 = {0, 0};
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int k = 8 * (64 * c + lane);
    held[c] = u32x4{0u, 0u, 0u, 0u};
    if (k < K) held[c] = *reinterpret_cast<const u32x4*>(from + k);
#pragma unroll
    for (int i = 0; i < 4; ++i) top2 = __builtin_elementwise_max(top2, __builtin_bit_cast(u16x2, held[c][i] & 0x7FFF7FFFu));
  }
  uint32_t top_bits = top2[0] > top2[1] ? top2[0] : top2[1];
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    const uint32_t other = static_cast<uint32_t>(__shfl_xor(static_cast<int>(top_bits), offset));
    top_bits = other > top_bits ? other : top_bits;
  }
  const float top = value_of_bits(top_bits);
  const float scale = __builtin_fmaxf(top / 127.0f, 1.1920928955078125e-07f);
  const float inverse = 1.0f / scale;
  // code = rint(x / scale), |code| <= 127. Adding 1.5 * 2^23 rounds to the nearest integer, ties to even, as rint does, and
  // leaves the code as the low byte of the sum's bit pattern. t = x * (1 / scale) is within 2^-14 of the quotient; where it
  // is no closer than that to a half-integer both round alike, and a chunk with a lane that is closer takes the division.
  constexpr float kMagic = 12582912.0f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int k = 8 * (64 * c + lane);
    float shifted[8];
    float nearest_half = 0.0f;               // the largest |t - rint(t)| of the chunk: 0.5 at a half-integer
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float t = __fmul_rn(value(held[c][i >> 1], i & 1), inverse);
      shifted[i] = __fadd_rn(t, kMagic);
      nearest_half = __builtin_fmaxf(nearest_half, __builtin_fabsf(__fsub_rn(t, __fsub_rn(shifted[i], kMagic))));
    }
    if (__builtin_amdgcn_ballot_w64(nearest_half > 0.5f - 0.00006103515625f) != 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) shifted[i] = __fadd_rn(__fdiv_rn(value(held[c][i >> 1], i & 1), scale), kMagic);
    }
    u32x2 packed;
#pragma unroll
    for (int h = 0; h < 2; ++h) {            // the low bytes of four sums into one word
      const uint32_t low = __builtin_amdgcn_perm(__float_as_uint(shifted[4 * h + 1]), __float_as_uint(shifted[4 * h]), 0x0C0C0400u);
      const uint32_t high = __builtin_amdgcn_perm(__float_as_uint(shifted[4 * h + 3]), __float_as_uint(shifted[4 * h + 2]), 0x04000C0Cu);
      packed[h] = low | high;
    }
    if (k < K) *reinterpret_cast<u32x2*>(codes + row * K + k) = packed;
  }
  if (lane == 0) scales[row] = scale;
}

// The same with an optional block rotation in front (entropack/linear/convrot.py:34-53 of the reference: activations
// are multiplied, group by group, with the Kronecker power of the 4 x 4 matrix 1 - 2 * antidiagonal, divided by
// sqrt(group), the product rounded to the activation dtype, and then quantised). The matrix is symmetric and every
// radix-4 stage is y_a = (x_0 + x_1 + x_2 + x_3) - 2 * x_(3 - a), so a group of 4^stages elements takes `stages`
// butterfly stages instead of a product. A lane holds 16 consecutive elements, so the first two stages stay in its
// registers and a group of 256 is one 16-lane row: the third stage runs inside quads and the fourth across the four
// quads of a row, both with data-parallel-primitive lane moves (no LDS traffic). The division is a power of two,
// applied once at the end. One block of four waves per row; the rotated row stays in registers between the absmax
// and the codes (CHUNKS x 4096 elements), so x is read once. stages = 0 is plain quantisation.
template <int CTRL, int BANKS>
__device__ __forceinline__ float dpp(float old, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v), CTRL, 0xF, BANKS, false));
}

__device__ __forceinline__ void butterfly4(float& a, float& b, float& c, float& d) {
  const float sum = (a + b) + (c + d);
  const float ya = sum - 2.0f * d, yb = sum - 2.0f * c, yc = sum - 2.0f * b, yd = sum - 2.0f * a;
  a = ya, b = yb, c = yc, d = yd;
}

template <int IN_KIND, int CHUNKS>
__global__ __launch_bounds__(256) void rotate_quantize_rows_kernel(const void* __restrict__ x, int64_t ldx, int K, int stages,
                                                                   int8_t* __restrict__ codes, float* __restrict__ scales) {
  __shared__ float partial[4];
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  constexpr int kQuadSwap1 = 0xB1, kQuadSwap2 = 0x4E, kQuadReverse = 0x1B;      // quad_perm [1,0,3,2], [2,3,0,1], [3,2,1,0]
  constexpr int kRowRor4 = 0x124, kRowRor8 = 0x128, kRowRor12 = 0x12C;          // lane l takes lane (l - n) mod 16 of its row
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const float shrink = __builtin_ldexpf(1.0f, -stages);

  float v[CHUNKS][16];
  float top = 0.0f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int k0 = (c * 4 + wave) * 1024 + lane * 16;
    if constexpr (IN_KIND == kOutF32) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float* w = &v[c][4 * q];
        w[0] = w[1] = w[2] = w[3] = 0.0f;
        if (k0 + 4 * q < K) {
          const f32x4 in = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(x) + row * ldx + k0 + 4 * q);
#pragma unroll
          for (int i = 0; i < 4; ++i) w[i] = in[i];
        }
      }
    } else {
      // Two-byte elements: eight per 16-byte load (K is a multiple of four: a load is all inside the row or, at the
      // row's end, split into its two halves).
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        u32x4 in = {0u, 0u, 0u, 0u};
        const uint16_t* from = reinterpret_cast<const uint16_t*>(x) + row * ldx + k0 + 8 * h;
        if (k0 + 8 * h + 8 <= K) {
          in = *reinterpret_cast<const u32x4*>(from);
        } else if (k0 + 8 * h < K) {
          const u32x2 low = *reinterpret_cast<const u32x2*>(from);
          in[0] = low[0];
          in[1] = low[1];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t bits = (in[i >> 1] >> (16 * (i & 1))) & 0xFFFFu;
          if constexpr (IN_KIND == kOutBF16) v[c][8 * h + i] = __uint_as_float(bits << 16);
          else v[c][8 * h + i] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits)));
        }
      }
    }
    if (stages >= 1) {
#pragma unroll
      for (int q = 0; q < 4; ++q) butterfly4(v[c][4 * q], v[c][4 * q + 1], v[c][4 * q + 2], v[c][4 * q + 3]);
    }
    if (stages >= 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) butterfly4(v[c][r], v[c][4 + r], v[c][8 + r], v[c][12 + r]);
    }
    if (stages >= 3) {        // digit = lane & 3
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float value = v[c][i];
        const float pair = value + dpp<kQuadSwap1, 0xF>(0.0f, value);
        const float sum = pair + dpp<kQuadSwap2, 0xF>(0.0f, pair);
        v[c][i] = sum - 2.0f * dpp<kQuadReverse, 0xF>(0.0f, value);
      }
    }
    if (stages >= 4) {        // digit = (lane >> 2) & 3; its complement sits 4 lanes down for even digits, 4 up for odd ones
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float value = v[c][i];
        const float pair = value + dpp<kRowRor8, 0xF>(0.0f, value);
        const float sum = pair + dpp<kRowRor4, 0xF>(0.0f, pair);
        float other = dpp<kRowRor4, 0x5>(0.0f, value);
        other = dpp<kRowRor12, 0xA>(other, value);
        v[c][i] = sum - 2.0f * other;
      }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float scaled = v[c][i] * shrink;
      if constexpr (IN_KIND == kOutBF16) v[c][i] = __uint_as_float(bf16_bits_of(scaled) << 16);
      else if constexpr (IN_KIND == kOutF16) v[c][i] = static_cast<float>(static_cast<_Float16>(scaled));
      else v[c][i] = scaled;
      top = __builtin_fmaxf(top, __builtin_fabsf(v[c][i]));
    }
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) top = __builtin_fmaxf(top, __shfl_xor(top, offset));
  if (threadIdx.x < 4) partial[threadIdx.x] = 0.0f;        // a short row runs fewer than four waves
  __syncthreads();
  if (lane == 0) partial[wave] = top;
  __syncthreads();
  top = __builtin_fmaxf(__builtin_fmaxf(partial[0], partial[1]), __builtin_fmaxf(partial[2], partial[3]));
  const float scale = __builtin_fmaxf(top / 127.0f, 1.1920928955078125e-07f);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int k0 = (c * 4 + wave) * 1024 + lane * 16;
    u32x4 packed;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t word = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float code = __builtin_fminf(__builtin_fmaxf(__builtin_rintf(v[c][4 * q + i] / scale), -127.0f), 127.0f);
        word |= (static_cast<uint32_t>(static_cast<int>(code)) & 0xFFu) << (8 * i);
      }
      packed[q] = word;
    }
    int8_t* to = codes + row * K + k0;
    if (k0 + 16 <= K && (K & 15) == 0) {
      *reinterpret_cast<u32x4*>(to) = packed;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (k0 + 4 * q < K) *reinterpret_cast<uint32_t*>(to + 4 * q) = packed[q];
      }
    }
  }
  if (threadIdx.x == 0) scales[row] = scale;
}


// Writes one wave's 64 x 32 NJ accumulator tile: acc[i][j] is the 32 x 32 tile at rows 32 i, columns 32 j of it.
// Accumulator layout of a 32 x 32 tile: register r of lane l holds row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32.
// One lane therefore owns single elements of many rows. Written out as they lie that is 16 NJ two-byte stores per
// lane and half tile, each instruction touching two 64-byte row pieces, and the stores then cost more than a fifth of
// a 4096 x 3072 x 3072 product. When the output allows 16-byte stores, the wave instead passes each half tile (32 rows
// x 32 NJ columns, as f32 after scales and bias) through `slab`, LDS private to it that the tiles no longer need, and
// stores whole row pieces, 16 bytes per lane. In the slab, rows with bit 2 set keep their columns rotated by 32: the
// two lane halves of an accumulator register (rows 4 apart) then write to different banks. The arithmetic and the
// rounding are those of the element-wise path, which ragged products and outputs with unaligned rows take.
template <bool INT8, bool GUARD, int NJ, typename Acc, bool EDGE = false, int NI = 2>    // EDGE: whole row pieces, but the tile may overhang M and N; NI: 32-row tiles of the wave (from the argument)
__device__ __forceinline__ void store_wave_tile(Acc (&acc)[NI][NJ], float* slab, const float* __restrict__ scale_a,
                                                const float* __restrict__ scale_b, const void* __restrict__ bias,
                                                void* __restrict__ y, int M, int N, int64_t ldy, int out_kind, int row0, int col0,
                                                int lane) {
  constexpr int WN = 32 * NJ;
  auto slab_at = [](int row, int col) { const int c = col + ((row & 4) << 3); return row * WN + (c >= WN ? c - WN : c); };
  const int out_bytes = out_kind == kOutF32 ? 4 : 2;
  const bool wide_rows = !GUARD && ((reinterpret_cast<uintptr_t>(y) | static_cast<uintptr_t>(ldy * out_bytes)) & 15u) == 0 &&
                         (!EDGE || N % (16 / out_bytes) == 0);      // a 16-byte piece is then all inside the row or all outside
  if (wide_rows) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        int n = col0 + j * 32 + (lane & 31);
        if (EDGE && n >= N) n = N - 1;                        // overhanging columns are computed and dropped below
        const bool has_bias = bias != nullptr;
        const float bv = has_bias ? load_bias(bias, out_kind, n) : 0.0f;
        float sb = 1.0f;
        if constexpr (INT8) sb = scale_b[n];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
          float v;
          if constexpr (INT8) {
            v = __fmul_rn(__fmul_rn(static_cast<float>(acc[i][j][r]), scale_a[EDGE && row0 + i * 32 + row >= M ? M - 1 : row0 + i * 32 + row]), sb);
            if (has_bias) v = __fadd_rn(v, bv);
          } else {
            v = acc[i][j][r] + bv;
          }
          slab[slab_at(row, j * 32 + (lane & 31))] = v;
        }
      }
      const int64_t first = static_cast<int64_t>(row0 + i * 32) * ldy + col0;
      if (out_kind == kOutF32) {
        constexpr int kPieces = WN / 4;                     // 16-byte pieces per row
        float* out = reinterpret_cast<float*>(y) + first;
#pragma unroll
        for (int at = 0; at < 32 * kPieces; at += 64) {
          const int row = (at + lane) / kPieces, piece = (at + lane) % kPieces;
          if (EDGE && (row0 + i * 32 + row >= M || col0 + 4 * piece >= N)) continue;
          *reinterpret_cast<uint4*>(out + row * ldy + 4 * piece) =
              *reinterpret_cast<const uint4*>(slab + slab_at(row, 4 * piece));
        }
      } else {
        constexpr int kPieces = WN / 8;
        uint16_t* out = reinterpret_cast<uint16_t*>(y) + first;
#pragma unroll
        for (int at = 0; at < 32 * kPieces; at += 64) {
          const int row = (at + lane) / kPieces, piece = (at + lane) % kPieces;
          if (EDGE && (row0 + i * 32 + row >= M || col0 + 8 * piece >= N)) continue;
          const float* from = slab + slab_at(row, 8 * piece);
          const float4 lo = *reinterpret_cast<const float4*>(from);
          const float4 hi = *reinterpret_cast<const float4*>(from + 4);
          uint4 packed;
          if (out_kind == kOutBF16) {
            packed.x = bf16_bits_of(lo.x) | bf16_bits_of(lo.y) << 16;
            packed.y = bf16_bits_of(lo.z) | bf16_bits_of(lo.w) << 16;
            packed.z = bf16_bits_of(hi.x) | bf16_bits_of(hi.y) << 16;
            packed.w = bf16_bits_of(hi.z) | bf16_bits_of(hi.w) << 16;
          } else {
            auto half_bits = [](float v) { return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<_Float16>(v))); };
            packed.x = half_bits(lo.x) | half_bits(lo.y) << 16;
            packed.y = half_bits(lo.z) | half_bits(lo.w) << 16;
            packed.z = half_bits(hi.x) | half_bits(hi.y) << 16;
            packed.w = half_bits(hi.z) | half_bits(hi.w) << 16;
          }
          *reinterpret_cast<uint4*>(out + row * ldy + 8 * piece) = packed;
        }
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int n = col0 + j * 32 + (lane & 31);
      if (n >= N) continue;
      const bool has_bias = bias != nullptr;
      const float bv = has_bias ? load_bias(bias, out_kind, n) : 0.0f;
      float sb = 1.0f;
      if constexpr (INT8) sb = scale_b[n];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = row0 + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        if (m >= M) continue;
        float v;
        if constexpr (INT8) {
          // int32 -> f32, times the activation row scale, times the weight row scale, plus bias: each one rounded operation.
          v = __fmul_rn(__fmul_rn(static_cast<float>(acc[i][j][r]), scale_a[m]), sb);
          if (has_bias) v = __fadd_rn(v, bv);
        } else {
          v = acc[i][j][r] + bv;
        }
        store_out(y, out_kind, static_cast<int64_t>(m) * ldy + n, v);
      }
    }
  }
}

// ---- large products: 256 x 256 block tiles ----------------------------------------------------------------------------------
//
// With 64 x 64 per wave (above) every matrix-core instruction needs one 16-byte LDS read per lane and the LDS port, not
// the matrix cores, sets the pace. Here eight waves share a 256 x 256 block tile, 64 x 128 each: 8 matrix-core
// instructions per 6 fragment reads, accumulators in 128 registers, two waves per SIMD so that one wave's reads hide
// behind the other's multiplies. Two LDS stages alternate, so a K step costs one barrier: the tile for step k + 1 is
// written while step k is multiplied, and the global loads for step k + 2 are already in flight in registers.
constexpr int kBigM = 256, kBigThreads = 512;

// BN = 256 or 192 output columns per block tile (wave tiles 64 x 128 or 64 x 96): the narrower one gives products such
// as 4096 x 3072 one tile per CU (16 x 16) where the square one leaves a quarter of the CUs idle (16 x 12).
template <bool INT8, bool GUARD, int BN>      // GUARD = false: M, N multiples of the tile and K of one tile step, no bounds checks on loads
__global__ __launch_bounds__(512, 2) void gemm_big_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                          const float* __restrict__ scale_a, const float* __restrict__ scale_b,
                                                          const void* __restrict__ bias, void* __restrict__ y, int M, int N,
                                                          int64_t k_bytes, int64_t lda_bytes, int64_t ldb_bytes, int64_t ldy,
                                                          int out_kind) {
  extern __shared__ __align__(16) uint8_t big_smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  constexpr int WN = BN / 2, NJ = WN / 32;                  // columns and 32-wide matrix-core tiles per wave
  constexpr int B_CHUNKS = BN * 8 / kBigThreads;            // 16-byte pieces of the B tile each thread moves
  constexpr int kStageBytes = (kBigM + BN) * kRowStride;
  const int wave_m = wave >> 1, wave_n = wave & 1;          // 4 x 2 waves of 64 x WN
  const int m0 = blockIdx.y * kBigM, n0 = blockIdx.x * BN;
  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 16;

  // Per operand tile: rows of 8 pieces of 16 bytes; thread t moves pieces t, t + 512, ...: 4 of A, then B_CHUNKS of B.
  constexpr int kMoves = 4 + B_CHUNKS;
  uint4 staged[kMoves];
  auto fetch_one = [&](int64_t kb, int c) {
    const bool of_a = c < 4;
    const int chunk = tid + kBigThreads * (of_a ? c : c - 4);
    const int r = (of_a ? m0 : n0) + (chunk >> 3);
    const int64_t at = kb + 16 * (chunk & 7);
    const uint8_t* from = of_a ? a + r * lda_bytes + at : b + r * ldb_bytes + at;
    staged[c] = make_uint4(0, 0, 0, 0);
    if (!GUARD || (r < (of_a ? M : N) && at < k_bytes)) staged[c] = *reinterpret_cast<const uint4*>(from);
  };
  auto stash_one = [&](int stage, int c) {
    const bool of_a = c < 4;
    const int chunk = tid + kBigThreads * (of_a ? c : c - 4);
    uint8_t* tile = big_smem + stage * kStageBytes + (of_a ? 0 : kBigM * kRowStride);
    *reinterpret_cast<uint4*>(tile + (chunk >> 3) * kRowStride + 16 * (chunk & 7)) = staged[c];
  };

  using Acc = typename std::conditional<INT8, i32x16, f32x16>::type;
  using Frag = typename std::conditional<INT8, i32x4, bf16x8>::type;
  Acc acc[2][NJ] = {};
  // Fragments of one 32-byte slice of K, held twice: while the matrix cores work through one set, the LDS reads of the
  // next slice are under way, across the barrier between two K steps as well.
  constexpr int kReads = 2 + NJ, kMultiplies = 2 * NJ;
  Frag frag[2][kReads];
  const uint32_t frag_a_at = static_cast<uint32_t>((wave_m * 64 + frag_row) * kRowStride + frag_k);
  const uint32_t frag_b_at = static_cast<uint32_t>((kBigM + wave_n * WN + frag_row) * kRowStride + frag_k);
  auto read_one = [&](int set, int stage, int kk, int t) {
    const uint32_t at = stage * kStageBytes + kk * 32 + (t < 2 ? frag_a_at + t * 32 * kRowStride : frag_b_at + (t - 2) * 32 * kRowStride);
    frag[set][t] = *reinterpret_cast<const Frag*>(big_smem + at);
  };
  auto multiply_one = [&](int set, int m) {
    const int i = m / NJ, j = m % NJ;
    if constexpr (INT8) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[set][i], frag[set][2 + j], acc[i][j], 0, 0, 0);
    else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag[set][i], frag[set][2 + j], acc[i][j], 0, 0, 0);
  };

  const int64_t steps = (k_bytes + kTileBytesK - 1) / kTileBytesK;
#pragma unroll
  for (int c = 0; c < kMoves; ++c) fetch_one(0, c);
#pragma unroll
  for (int c = 0; c < kMoves; ++c) stash_one(0, c);
  __syncthreads();
  // Same order as in the loop (the pieces beyond one per multiply first): the stores there wait for the loads one by one.
#pragma unroll
  for (int c = kMultiplies; c < kMoves; ++c) fetch_one(steps > 1 ? kTileBytesK : 0, c);
#pragma unroll
  for (int c = 0; c < kMoves && c < kMultiplies; ++c) fetch_one(steps > 1 ? kTileBytesK : 0, c);
#pragma unroll
  for (int t = 0; t < kReads; ++t) read_one(0, 0, 0, t);
  // One K step = four slices. Every multiply is followed by at most two memory operations and the order is pinned, so
  // that the LDS port and the matrix cores work at the same time instead of taking turns: during slice 0 the tile held
  // in registers goes to the other LDS stage, during slice 1 the loads of the tile after it are issued, and each slice
  // reads the fragments of the next one. Past the last tile the stores and loads repeat work that nobody reads (the
  // idle stage, the last tile again), which keeps the loop body one straight line.
  for (int64_t step = 0; step < steps; ++step) {
    const int stage = static_cast<int>(step & 1);
    const int64_t ahead = (step + 2 < steps ? step + 2 : steps - 1) * kTileBytesK;
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(0, m);
      if (kMultiplies + m < kMoves) stash_one(stage ^ 1, kMultiplies + m);
      if (m < kMoves) stash_one(stage ^ 1, m);
      if (m < kReads) read_one(1, stage, 1, m);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(1, m);
      if (kMultiplies + m < kMoves) fetch_one(ahead, kMultiplies + m);
      if (m < kMoves) fetch_one(ahead, m);
      if (m < kReads) read_one(0, stage, 2, m);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(0, m);
      if (m < kReads) read_one(1, stage, 3, m);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(1, m);
      if (m < kReads) read_one(0, stage ^ 1, 0, m);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  static_assert(8 * 32 * WN * 4 <= 2 * kStageBytes, "the eight slabs fit into the two tile stages");
  store_wave_tile<INT8, GUARD, NJ>(acc, reinterpret_cast<float*>(big_smem) + wave * (32 * WN), scale_a, scale_b, bias, y, M, N, ldy, out_kind,
                                   m0 + wave_m * 64, n0 + wave_n * WN, lane);
}

// ---- the same block tile with the operand tiles loaded straight into LDS ----------------------------------------------------
//
// For K a multiple of one tile step (M and N may overhang the tiles with RAGGED). The kernel above moves every tile byte
// memory -> registers -> LDS, and that round trip (seven 16-byte loads and seven LDS stores per wave and K step) is what
// keeps it a third above the matrix cores' own time. Here `global_load_lds_dwordx4` writes the loaded bytes into LDS
// itself: one instruction fills 1 KiB of consecutive LDS (lane l the 16 bytes at 16 l), i.e. eight tile rows of 128
// bytes. Rows therefore cannot be padded; instead row r keeps its eight 16-byte pieces permuted, piece c at place
// c ^ ((r >> 1) & 7), which each lane arranges by choosing the global address it loads from. Sixteen consecutive rows
// read at the same logical piece then cover all 64 banks once. The two stages are two separate arrays and the K loop
// is written out for both parities, so that every LDS access names its array: the compiler then waits for loads in
// flight only where an access may touch the array they fill (before the barrier that publishes it), not before the
// fragment reads of the other stage. (Requesting all pieces right after the barrier, a whole step ahead, measured the
// same: the loads' latency is covered either way.)
// RAGGED: M and N need not be multiples of the tile (K must be of a tile step): rows past the end load the last row
// again and are dropped by the epilogue.
template <bool INT8, int BM, int BN, int WAVES_M, int WAVES_N, bool RAGGED>   // wave tiles of 64 x (BN / WAVES_N); 256 x 192|256 with 4 x 2 waves, 128 x 128 with 2 x 2
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, 2) void gemm_direct_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                             const float* __restrict__ scale_a, const float* __restrict__ scale_b,
                                                             const void* __restrict__ bias, void* __restrict__ y, int M, int N,
                                                             int64_t k_bytes, int64_t lda_bytes, int64_t ldb_bytes, int64_t ldy,
                                                             int out_kind) {
  constexpr int kWaves = WAVES_M * WAVES_N;
  static_assert(BM == 64 * WAVES_M && BN % (32 * WAVES_N) == 0 && BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "tile shapes");
  constexpr int kRowBytes = kTileBytesK;                    // 128, unpadded
  constexpr int kStage = (BM + BN) * kRowBytes;
  __shared__ __align__(1024) uint8_t stage0[kStage];
  __shared__ __align__(1024) uint8_t stage1[kStage];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int WN = BN / WAVES_N, NJ = WN / 32;
  constexpr int kLoadsA = BM / (8 * kWaves), kLoadsB = BN / (8 * kWaves), kLoads = kLoadsA + kLoadsB;   // 1 KiB pieces per wave and tile
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  // Workgroups go to the eight XCDs round-robin in launch order, and each XCD has its own L2. When the whole grid is
  // resident at once (one 256-row tile per CU at most), handing XCD i one compact part of the tile grid instead of every
  // eighth tile lets the 32 CUs of an XCD share operand tiles in that L2: on a 16 x 16 grid of 256 x 192 tiles an XCD
  // then fills 2.5 K tile rows per K step instead of 4.5 K (4096 x 3072 x 3072 with a weight not yet in any cache:
  // 69 -> 67 us). Grids of several rounds keep the launch order, whose window of resident tiles is compact already
  // (8192^3 measured 4 % slower remapped), and so do the small tiles (no gain, warm operands slower).
  int tile_x = blockIdx.x, tile_y = blockIdx.y;
  if (BM == 256 && gridDim.x * gridDim.y <= 256) {
    const int gx = gridDim.x, gy = gridDim.y;
    int parts_x = 0;
    if (gx % 2 == 0 && gy % 4 == 0) parts_x = 2;
    else if (gx % 4 == 0 && gy % 2 == 0) parts_x = 4;
    else if (gy % 8 == 0) parts_x = 1;
    else if (gx % 8 == 0) parts_x = 8;
    if (parts_x != 0) {
      const int parts_y = 8 / parts_x, wx = gx / parts_x;
      const int linear = tile_y * gx + tile_x, xcd = linear & 7, at = linear >> 3;
      tile_x = (xcd % parts_x) * wx + at % wx;
      tile_y = (xcd / parts_x) * (gy / parts_y) + at / wx;
    }
  }
  const int m0 = tile_y * BM, n0 = tile_x * BN;

  // Load c of this wave fills tile rows 8 (wave + kWaves c') .. + 8 of A (c < kLoadsA, c' = c) or of B (c' = c - kLoadsA).
  const uint8_t* source[kLoads];
#pragma unroll
  for (int c = 0; c < kLoads; ++c) {
    const bool of_a = c < kLoadsA;
    const int row = 8 * (wave + kWaves * (of_a ? c : c - kLoadsA)) + (lane >> 3);
    const int piece = (lane & 7) ^ ((row >> 1) & 7);
    int from_row = (of_a ? m0 : n0) + row;
    if (RAGGED && from_row >= (of_a ? M : N)) from_row = (of_a ? M : N) - 1;
    source[c] = of_a ? a + from_row * lda_bytes + 16 * piece : b + from_row * ldb_bytes + 16 * piece;
  }
  auto load_one = [&](uint8_t* stage, int64_t kb, int c) {
    const bool of_a = c < kLoadsA;
    const int first_row = (of_a ? 0 : BM) + 8 * (wave + kWaves * (of_a ? c : c - kLoadsA));
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(source[c] + kb),
                                     (__attribute__((address_space(3))) void*)(stage + first_row * kRowBytes), 16, 0, 0);
  };

  using Acc = typename std::conditional<INT8, i32x16, f32x16>::type;
  using Frag = typename std::conditional<INT8, i32x4, bf16x8>::type;
  Acc acc[2][NJ] = {};
  constexpr int kReads = 2 + NJ, kMultiplies = 2 * NJ;
  Frag frag[2][kReads];
  const int frag_row = lane & 31;
  const int turn = (frag_row >> 1) & 7;                      // the same for rows 32 apart
  const uint32_t frag_a_at = static_cast<uint32_t>((wave_m * 64 + frag_row) * kRowBytes);
  const uint32_t frag_b_at = static_cast<uint32_t>((BM + wave_n * WN + frag_row) * kRowBytes);
  auto read_one = [&](int set, const uint8_t* stage, int kk, int t) {
    const uint32_t place = static_cast<uint32_t>(((2 * kk + (lane >> 5)) ^ turn) * 16);
    const uint32_t at = place + (t < 2 ? frag_a_at + t * 32 * kRowBytes : frag_b_at + (t - 2) * 32 * kRowBytes);
    frag[set][t] = *reinterpret_cast<const Frag*>(stage + at);
  };
  auto multiply_one = [&](int set, int m) {
    const int i = m / NJ, j = m % NJ;
    if constexpr (INT8) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[set][i], frag[set][2 + j], acc[i][j], 0, 0, 0);
    else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag[set][i], frag[set][2 + j], acc[i][j], 0, 0, 0);
  };

  const int64_t steps = k_bytes / kTileBytesK;
  auto tile_at = [&](int64_t t) { return (t < steps ? t : steps - 1) * kTileBytesK; };
  // One K step on the stage `here` while `there` is filled. The A pieces of a tile are requested right after the barrier
  // that frees their stage (the last slice of the step before), the B pieces during the first slice of this step, so
  // every load has most of a step to land before the barrier that publishes the stage. Past the last tile the loads
  // repeat the last one, which nobody reads.
  auto k_step = [&](uint8_t* here, uint8_t* there, int64_t step) {
    const int64_t next = tile_at(step + 1), second = tile_at(step + 2);
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(0, m);
      if (m < kLoadsB) load_one(there, next, kLoadsA + m);
      if (m < kReads) read_one(1, here, 1, m);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(1, m);
      if (m < kReads) read_one(0, here, 2, m);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(0, m);
      if (m < kReads) read_one(1, here, 3, m);
      __builtin_amdgcn_sched_barrier(0);
    }
    // The barrier publishes `there`, which every wave has filled a part of: each waits for its own loads first. (Left
    // to itself the compiler waits for them where this wave next reads that array, which may be after the barrier.)
    __builtin_amdgcn_s_waitcnt(0x0F70);                     // vmcnt(0)
    __syncthreads();
#pragma unroll
    for (int m = 0; m < kMultiplies; ++m) {
      multiply_one(1, m);
      if (m < kLoadsA) load_one(here, second, m);
      if (m < kReads) read_one(0, there, 0, m);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
#pragma unroll
  for (int c = 0; c < kLoads; ++c) load_one(stage0, 0, c);
#pragma unroll
  for (int c = 0; c < kLoadsA; ++c) load_one(stage1, tile_at(1), c);
  __builtin_amdgcn_s_waitcnt(0x0F70);                       // vmcnt(0), as before the barrier in k_step
  __syncthreads();
#pragma unroll
  for (int t = 0; t < kReads; ++t) read_one(0, stage0, 0, t);
  for (int64_t step = 0; step < steps; step += 2) {
    k_step(stage0, stage1, step);
    if (step + 1 < steps) k_step(stage1, stage0, step + 1);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();     // every load has landed and every fragment is read before the slabs below reuse the stages

  static_assert(4 * 32 * WN * 4 <= kStage && kWaves <= 8, "four slabs fit into one stage");
  float* slab = reinterpret_cast<float*>(wave < 4 ? stage0 : stage1) + (wave & 3) * (32 * WN);
  store_wave_tile<INT8, false, NJ, Acc, RAGGED>(acc, slab, scale_a, scale_b, bias, y, M, N, ldy, out_kind, m0 + wave_m * 64, n0 + wave_n * WN, lane);
}

// ---- 128 x 128 tiles with four stages: products of few blocks whose operands come from memory ---------------------------
//
// The two-stage 128 x 128 kernel above keeps one K step of loads (32 KB) in flight per block, which covers the L2's latency
// but not memory's. When a product has at most one such block per CU there is no second block for the LDS anyway, so this
// variant spends it on depth: four stages of 32 KB, the tile three steps ahead requested while a step is multiplied (96 KB
// in flight per block). The wait before the barrier that publishes a stage is counted: the 16 loads issued after that
// stage's own may still be in flight. The barrier is a bare s_barrier, and the loop body has no branch: after the fence of
// __syncthreads(), and after any join of two paths, the compiler's wait-count pass waits for every load into LDS, which
// empties the pipeline (visible as `s_waitcnt vmcnt(0)` at each step in the code it emits). Everything else (piece
// permutation, fragment reads a slice ahead, slab epilogue) is the two-stage kernel's.
// Measured on N = K = 3072 bf16, weight in the last-level cache / weight from memory: M = 256 (48 blocks) 21.6 / 43.0 us
// with two stages, 18.9 / 31.7 us with four; M = 1024 (192 blocks) 32.0 / 43.1 -> 23.2 / 31.5 us (vendor library 18.8 /
// 19.2 and 25.6 / 28.7 us). What remains from memory is not depth: a fifth wave that touched the weight rows two groups of
// steps ahead in 512-byte runs changed nothing, nor did starting each column of blocks at its own K offset. It is the rate at
// which one CU takes operand bytes, 1.5 MB per block here whatever M is (see the K split below).
// SPLIT: the grid's z blocks share a tile, each taking gridDim.z-th of K; the sums go, as they are (f32, or int32 for int8), to
// slab blockIdx.z of `y` ([slice][M][N]) for the kernel that adds the slices, and scales, bias and out_kind are not used.
// TILE = 64: blocks of 64 x 64 (four waves of 32 x 32, four stages of 16 KB) for products whose 128 x 128 tiles would leave most
// CUs idle. TILE = 96: blocks of 128 x 96 (four waves of 32 x 96 one above the other, four stages of 28 KB) for products whose
// 128 x 128 tiles leave some CUs idle: a block then takes 224 instead of 256 operand rows.
template <bool INT8, bool RAGGED, bool SPLIT, int TILE = 128>
__global__ __launch_bounds__(256, 1) void gemm_deep_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                          const float* __restrict__ scale_a, const float* __restrict__ scale_b,
                                                          const void* __restrict__ bias, void* __restrict__ y, int M, int N, int64_t k_bytes,
                                                          int64_t lda_bytes, int64_t ldb_bytes, int64_t ldy, int out_kind) {
  static_assert(TILE == 128 || TILE == 64 || TILE == 96, "2 x 2 waves of 64 x 64 or 32 x 32, or 4 x 1 waves of 32 x 96");
  constexpr int BM = TILE == 64 ? 64 : 128, BN = TILE, kWaves = 4, kWavesN = TILE == 96 ? 1 : 2, kWavesM = kWaves / kWavesN;
  constexpr int WN = BN / kWavesN, NJ = WN / 32, NI = BM / (32 * kWavesM);
  constexpr int kRowBytes = kTileBytesK;
  constexpr int kStage = (BM + BN) * kRowBytes;              // 32 KB (16 KB, 28 KB)
  __shared__ __align__(1024) uint8_t stage0[kStage];
  __shared__ __align__(1024) uint8_t stage1[kStage];
  __shared__ __align__(1024) uint8_t stage2[kStage];
  __shared__ __align__(1024) uint8_t stage3[kStage];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int kLoadsA = BM / (8 * kWaves), kLoadsB = BN / (8 * kWaves), kLoads = kLoadsA + kLoadsB;      // 4 + 4 (2 + 2) pieces of 1 KiB per wave and tile
  const int wave_m = wave / kWavesN, wave_n = wave % kWavesN;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int64_t steps = k_bytes / kTileBytesK / (SPLIT ? gridDim.z : 1);           // this block's
  const int64_t k_first = SPLIT ? blockIdx.z * steps * kTileBytesK : 0;

  const uint8_t* source[kLoads];
#pragma unroll
  for (int c = 0; c < kLoads; ++c) {
    const bool of_a = c < kLoadsA;
    const int row = 8 * (wave + kWaves * (of_a ? c : c - kLoadsA)) + (lane >> 3);
    const int piece = (lane & 7) ^ ((row >> 1) & 7);
    int from_row = (of_a ? m0 : n0) + row;
    if (RAGGED && from_row >= (of_a ? M : N)) from_row = (of_a ? M : N) - 1;
    source[c] = (of_a ? a + from_row * lda_bytes + 16 * piece : b + from_row * ldb_bytes + 16 * piece) + k_first;
  }
  auto load_one = [&](uint8_t* stage, int64_t kb, int c) {
    const bool of_a = c < kLoadsA;
    const int first_row = (of_a ? 0 : BM) + 8 * (wave + kWaves * (of_a ? c : c - kLoadsA));
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(source[c] + kb),
                                     (__attribute__((address_space(3))) void*)(stage + first_row * kRowBytes), 16, 0, 0);
  };

  using Acc = typename std::conditional<INT8, i32x16, f32x16>::type;
  using Frag = typename std::conditional<INT8, i32x4, bf16x8>::type;
  Acc acc[NI][NJ] = {};
  constexpr int kReads = NI + NJ, kMultiplies = NI * NJ;
  Frag frag[2][kReads];
  const int frag_row = lane & 31;
  const int turn = (frag_row >> 1) & 7;
  const uint32_t frag_a_at = static_cast<uint32_t>((wave_m * 32 * NI + frag_row) * kRowBytes);
  const uint32_t frag_b_at = static_cast<uint32_t>((BM + wave_n * WN + frag_row) * kRowBytes);
  auto read_one = [&](int set, const uint8_t* stage, int kk, int t) {
    const uint32_t place = static_cast<uint32_t>(((2 * kk + (lane >> 5)) ^ turn) * 16);
    const uint32_t at = place + (t < NI ? frag_a_at + t * 32 * kRowBytes : frag_b_at + (t - NI) * 32 * kRowBytes);
    frag[set][t] = *reinterpret_cast<const Frag*>(stage + at);
  };
  auto multiply_one = [&](int set, int m) {
    const int i = m / NJ, j = m % NJ;
    if constexpr (INT8) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[set][i], frag[set][NI + j], acc[i][j], 0, 0, 0);
    else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag[set][i], frag[set][NI + j], acc[i][j], 0, 0, 0);
  };

  auto tile_at = [&](int64_t t) { return (t < steps ? t : steps - 1) * kTileBytesK; };
  // One K step on `here`; `there` is read next; `fill` (read in the step before this one) takes the tile three steps ahead,
  // three, three and two of its eight pieces per slice. Past the last tile the loads repeat the last one, which nobody reads.
  auto k_step = [&](uint8_t* here, uint8_t* there, uint8_t* fill, int64_t step) {
    const int64_t ahead = tile_at(step + 3);
    constexpr int kPerSlice = (kLoads + 2) / 3;             // loads a slice issues: 3, 3, 2 of eight; 2, 2, 0 of four
    constexpr int kSlots = kMultiplies > kReads ? (kMultiplies > kPerSlice ? kMultiplies : kPerSlice) : (kReads > kPerSlice ? kReads : kPerSlice);
#pragma unroll
    for (int slice = 0; slice < 3; ++slice) {
#pragma unroll
      for (int m = 0; m < kSlots; ++m) {
        if (m < kMultiplies) multiply_one(slice & 1, m);
        const int piece = kPerSlice * slice + m;
        if (m < kPerSlice && piece < kLoads) load_one(fill, ahead, piece);
        if (m < kReads) read_one((slice & 1) ^ 1, here, slice + 1, m);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // `there` holds the tile of the next step, requested two steps ago: the 16 loads issued since may still be in flight.
    // A bare barrier: the fence of __syncthreads() makes the compiler wait for every load into LDS, which would empty the
    // pipeline at each step. This wave's fragment reads of `here` are complete (lgkmcnt 0) before it arrives, so no wave
    // can overwrite a stage that another still reads.
    constexpr int kInFlight = 2 * kLoads;                   // s_waitcnt: vmcnt in bits 0-3 and 14-15, expcnt (not waited for) 4-6, lgkmcnt 8-11
    __builtin_amdgcn_s_waitcnt((kInFlight & 15) | ((kInFlight >> 4) << 14) | 0x0070);      // vmcnt(2 kLoads), lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int m = 0; m < (kMultiplies > kReads ? kMultiplies : kReads); ++m) {
      if (m < kMultiplies) multiply_one(1, m);
      if (m < kReads) read_one(0, there, 0, m);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
#pragma unroll
  for (int c = 0; c < kLoads; ++c) load_one(stage0, 0, c);
#pragma unroll
  for (int c = 0; c < kLoads; ++c) load_one(stage1, tile_at(1), c);
#pragma unroll
  for (int c = 0; c < kLoads; ++c) load_one(stage2, tile_at(2), c);
  __builtin_amdgcn_s_waitcnt(((2 * kLoads) & 15) | (((2 * kLoads) >> 4) << 14) | 0x0F70);       // vmcnt(2 kLoads): the first tile has landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int t = 0; t < kReads; ++t) read_one(0, stage0, 0, t);
  for (int64_t step = 0; step < steps; step += 4) {
    k_step(stage0, stage1, stage3, step);            // the launcher takes only K of a whole number of four steps: a branch
    k_step(stage1, stage2, stage0, step + 1);        // between the steps would make the compiler's wait-count pass forget which
    k_step(stage2, stage3, stage1, step + 2);        // stage each load in flight fills, and wait for all of them
    k_step(stage3, stage0, stage2, step + 3);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();     // every load has landed and every fragment is read before the slabs below reuse a stage

  if constexpr (SPLIT) {
    // Register r of lane l holds row 8 (r / 4) + 4 (l / 32) + r % 4 and column l % 32 of its 32 x 32 tile.
    using Cell = typename std::conditional<INT8, int32_t, float>::type;
    Cell* out = static_cast<Cell*>(y) + static_cast<int64_t>(blockIdx.z) * M * N;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int n = n0 + wave_n * WN + j * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wave_m * 32 * NI + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
          if (!RAGGED || (m < M && n < N)) out[static_cast<int64_t>(m) * N + n] = acc[i][j][r];
        }
      }
    }
  } else {
    static_assert(TILE == 96 ? 32 * WN * 4 <= kStage : 4 * 32 * WN * 4 <= kStage, "the waves' slabs fit into one stage, or one stage each");
    float* slab = TILE == 96 ? reinterpret_cast<float*>(wave == 0 ? stage0 : (wave == 1 ? stage1 : (wave == 2 ? stage2 : stage3)))
                             : reinterpret_cast<float*>(stage0) + wave * (32 * WN);
    store_wave_tile<INT8, false, NJ, Acc, RAGGED>(acc, slab, scale_a, scale_b, bias, y, M, N, ldy, out_kind, m0 + wave_m * 32 * NI, n0 + wave_n * WN, lane);
  }
}

template <bool INT8, bool GUARD, int BN>
static int launch_big_variant(const void* a, const void* b, const float* scale_a, const float* scale_b, const void* bias, void* y, int64_t M,
                      int64_t N, int64_t k_bytes, int64_t lda_bytes, int64_t ldb_bytes, int64_t ldy, int out_kind, hipStream_t stream) {
  static thread_local int configured_for = -1;
  constexpr int kLdsBytes = 2 * (kBigM + BN) * kRowStride;
  int device = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  if (configured_for != device) {
    EP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_big_kernel<INT8, GUARD, BN>), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
    configured_for = device;
  }
  const dim3 grid(static_cast<unsigned>((N + BN - 1) / BN), static_cast<unsigned>((M + kBigM - 1) / kBigM));
  if (grid.y > 65535) return EP_HIP_EUNSUPPORTED;
  hipLaunchKernelGGL((gemm_big_kernel<INT8, GUARD, BN>), grid, dim3(kBigThreads), kLdsBytes, stream, static_cast<const uint8_t*>(a),
                     static_cast<const uint8_t*>(b), scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes,
                     lda_bytes, ldb_bytes, ldy, out_kind);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

template <bool INT8, int BN>
static int launch_big(const void* a, const void* b, const float* scale_a, const float* scale_b, const void* bias, void* y, int64_t M,
                      int64_t N, int64_t k_bytes, int64_t lda_bytes, int64_t ldb_bytes, int64_t ldy, int out_kind, hipStream_t stream) {
  const bool interior = M % kBigM == 0 && N % BN == 0 && k_bytes % kTileBytesK == 0;
  if (k_bytes % kTileBytesK == 0) {
    const dim3 grid(static_cast<unsigned>((N + BN - 1) / BN), static_cast<unsigned>((M + kBigM - 1) / kBigM));
    if (grid.y > 65535) return EP_HIP_EUNSUPPORTED;
    if (interior)
      hipLaunchKernelGGL((gemm_direct_kernel<INT8, kBigM, BN, 4, 2, false>), grid, dim3(kBigThreads), 0, stream, static_cast<const uint8_t*>(a),
                         static_cast<const uint8_t*>(b), scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes,
                         lda_bytes, ldb_bytes, ldy, out_kind);
    else
      hipLaunchKernelGGL((gemm_direct_kernel<INT8, kBigM, BN, 4, 2, true>), grid, dim3(kBigThreads), 0, stream, static_cast<const uint8_t*>(a),
                         static_cast<const uint8_t*>(b), scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes,
                         lda_bytes, ldb_bytes, ldy, out_kind);
    EP_HIP_TRY(hipGetLastError());
    return EP_HIP_OK;
  }
  return interior ? launch_big_variant<INT8, false, BN>(a, b, scale_a, scale_b, bias, y, M, N, k_bytes, lda_bytes, ldb_bytes, ldy, out_kind, stream)
                  : launch_big_variant<INT8, true, BN>(a, b, scale_a, scale_b, bias, y, M, N, k_bytes, lda_bytes, ldb_bytes, ldy, out_kind, stream);
}

// Products of whole 128 x 128 tiles: the direct-load kernels with four waves per block. The two-stage kernel runs two blocks
// per CU (64 KB of LDS each): 2560 x 3072 x 3072 bf16, 480 blocks in one round, 51 us (256 x 192 tiles 57 us); with more
// blocks than two per CU a second round starts and the 256-row tiles win: 3072 x 3072 x 3072 80 us against 62 us
// (whole_k_tiling below weighs the rounds). Products of at most one block per CU take the four-stage kernels.
template <bool INT8>
static bool small_whole_tiles(int64_t M, int64_t N, int64_t k_bytes) {       // whole in K; M and N may overhang
  return k_bytes % kTileBytesK == 0 && (M + 127) / 128 <= 65535;
}

// Products whose 128 x 128 tiles would occupy at most half the CUs while 64 x 64 tiles still fit them in one round: what
// bounds such a product is the rate at which one CU takes operand bytes (see the K split further down), and a 64 x 64 block
// takes half of a 128 x 128 block's. 256 x 3072 x 3072 bf16, weight cached / from memory: 48 blocks of 128 x 128 18.9 / 31.7 us,
// the same split four ways over K 20.1 / 20.6 us (two kernels), 192 blocks of 64 x 64 16.7 / 16.9 us (the vendor library 19.0 / 19.4).
static int current_compute_units() {
  int device = 0, cus = 0;
  if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) cus = 0;
  return cus;
}

static bool few_tiles_take_small_blocks(int64_t M, int64_t N, int64_t k_bytes, int cus) {
  const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128), tiles64 = ((M + 63) / 64) * ((N + 63) / 64);
  return 2 * tiles128 <= cus && tiles64 <= cus && k_bytes % (4 * kTileBytesK) == 0 && k_bytes >= 8 * kTileBytesK;
}

template <bool INT8>
static int launch_direct_small(const void* a, const void* b, const float* scale_a, const float* scale_b, const void* bias, void* y, int64_t M,
                               int64_t N, int64_t k_bytes, int64_t lda_bytes, int64_t ldb_bytes, int64_t ldy, int out_kind, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((N + 127) / 128), static_cast<unsigned>((M + 127) / 128));
  // At most one block per CU (the deep kernel holds 128 KB of LDS) and K a whole number of four steps, which is what its loop runs.
  const int cus = current_compute_units();
  if (few_tiles_take_small_blocks(M, N, k_bytes, cus)) {
    const dim3 small(static_cast<unsigned>((N + 63) / 64), static_cast<unsigned>((M + 63) / 64));
    if (M % 64 == 0 && N % 64 == 0)
      hipLaunchKernelGGL((gemm_deep_kernel<INT8, false, false, 64>), small, dim3(256), 0, stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                         scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes, lda_bytes, ldb_bytes, ldy, out_kind);
    else
      hipLaunchKernelGGL((gemm_deep_kernel<INT8, true, false, 64>), small, dim3(256), 0, stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                         scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes, lda_bytes, ldb_bytes, ldy, out_kind);
    EP_HIP_TRY(hipGetLastError());
    return EP_HIP_OK;
  }
  // One round of blocks either way: 128 x 96 blocks are more, and each takes fewer operand bytes (1024 x 3072 x 3072 bf16, weight
  // cached / from memory: 23.4 / 31.8 us with 192 blocks of 128 x 128, 23.1 / 28.4 us with 256 of 128 x 96; vendor 26.2 / 29.5).
  if (static_cast<int64_t>(grid.x) * grid.y <= cus && ((N + 95) / 96) * static_cast<int64_t>(grid.y) <= cus && k_bytes % (4 * kTileBytesK) == 0) {
    const dim3 narrow(static_cast<unsigned>((N + 95) / 96), grid.y);
    if (M % 128 == 0 && N % 96 == 0)
      hipLaunchKernelGGL((gemm_deep_kernel<INT8, false, false, 96>), narrow, dim3(256), 0, stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                         scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes, lda_bytes, ldb_bytes, ldy, out_kind);
    else
      hipLaunchKernelGGL((gemm_deep_kernel<INT8, true, false, 96>), narrow, dim3(256), 0, stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                         scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes, lda_bytes, ldb_bytes, ldy, out_kind);
    EP_HIP_TRY(hipGetLastError());
    return EP_HIP_OK;
  }
  if (static_cast<int64_t>(grid.x) * grid.y <= cus && k_bytes % (4 * kTileBytesK) == 0) {
    if (M % 128 == 0 && N % 128 == 0)
      hipLaunchKernelGGL((gemm_deep_kernel<INT8, false, false>), grid, dim3(256), 0, stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                         scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes, lda_bytes, ldb_bytes, ldy, out_kind);
    else
      hipLaunchKernelGGL((gemm_deep_kernel<INT8, true, false>), grid, dim3(256), 0, stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                         scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes, lda_bytes, ldb_bytes, ldy, out_kind);
    EP_HIP_TRY(hipGetLastError());
    return EP_HIP_OK;
  }
  if (M % 128 == 0 && N % 128 == 0)
    hipLaunchKernelGGL((gemm_direct_kernel<INT8, 128, 128, 2, 2, false>), grid, dim3(256), 0, stream, static_cast<const uint8_t*>(a),
                       static_cast<const uint8_t*>(b), scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes,
                       lda_bytes, ldb_bytes, ldy, out_kind);
  else
    hipLaunchKernelGGL((gemm_direct_kernel<INT8, 128, 128, 2, 2, true>), grid, dim3(256), 0, stream, static_cast<const uint8_t*>(a),
                       static_cast<const uint8_t*>(b), scale_a, scale_b, bias, y, static_cast<int>(M), static_cast<int>(N), k_bytes,
                       lda_bytes, ldb_bytes, ldy, out_kind);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

// Which block tile a product with K of whole tile steps takes: the family whose rounds of blocks add up to the least time.
// A round is one set of blocks resident together (one 256-row block per CU, two two-stage 128 x 128 blocks, one four-stage
// block), and a round costs a fixed part plus a time per K step that was measured once per kernel on an MI355X (bf16,
// N = K = 3072 and 8192; the int8 kernels move the same bytes per step and keep the ratios): 256 x 256 1.55 us, 256 x 192
// 1.16 us, two-stage 128 x 128 0.83 us for its two blocks, the four-stage kernels 0.42 us. What the count of rounds decides
// is the tail: 1536 x 8192 x 8192 is 258 blocks of 256 x 192, two rounds for the sake of two blocks (262 us), and one round of
// 192 blocks of 256 x 256. Returns 256 or 192 for the 256-row tiles, 0 for the 128-row family (launch_direct_small).
static int whole_k_tiling(int64_t M, int64_t N, int64_t k_bytes, int cus) {
  if (cus <= 0) cus = 256;
  const double steps = static_cast<double>(k_bytes / kTileBytesK);
  constexpr double kRoundFixed = 4.0;
  auto rounds = [&](int64_t bm, int64_t bn, int64_t slots) { return static_cast<double>((((M + bm - 1) / bm) * ((N + bn - 1) / bn) + slots - 1) / slots); };
  const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
  const double small = tiles128 <= cus ? kRoundFixed + 0.42 * steps : rounds(128, 128, 2 * static_cast<int64_t>(cus)) * (kRoundFixed + 0.83 * steps);
  const double wide = (M + 255) / 256 <= 65535 ? rounds(256, 192, cus) * (kRoundFixed + 1.16 * steps) : 1e30;
  const double square = (M + 255) / 256 <= 65535 ? rounds(256, 256, cus) * (kRoundFixed + 1.55 * steps) : 1e30;
  if (small <= wide && small <= square) return 0;
  return square < wide ? 256 : 192;
}

// The same choice for products whose K is not of whole tile steps (the register-staged 256-row kernel or the single-stage
// 128 x 128 kernel): 256 x 256 once there is one for every CU (256 on MI355X); else 256 x 192 from 150 tiles on (3072 x 3000
// x 3072: 84 us against 102 us, but 512 x 3000 x 3072: 72 us against 55 us). Returns the tile's column count, 0 for the
// 128 x 128 kernel.
static int big_tile_columns(int64_t M, int64_t N, int64_t k_bytes) {
  if (M < kBigM) return 0;
  const int64_t rows = (M + kBigM - 1) / kBigM;
  if (N >= 256 && rows * ((N + 255) / 256) >= 256) return 256;
  (void)k_bytes;
  if (N >= 192 && rows * ((N + 191) / 192) >= 150) return 192;
  return 0;
}

// ---- few activation rows (M <= 128): the weight stream bounds the product ---------------------------------------------------
//
// y = x W^T reads every weight exactly once, so the kernel is built around that stream: a block owns 128 weight rows
// and one slice of K and moves 128 x 64 weight tiles from memory to LDS with fully coalesced 16-byte loads (eight
// lanes per 128-byte row segment), the next tile always in flight in registers. Its four waves each multiply 32 of
// the rows with all activation rows (at most four 32-row tiles, also staged in LDS). Small tiles keep many blocks
// resident per CU, which is what keeps enough bytes in flight; K is split across blocks so that every CU streams.
// The partial sums land in f32 slabs [slice][M][N] and a second kernel adds them, the bias, and rounds once.
constexpr int kSkinnyBlockN = 128;
constexpr int kSkinnyChunkBytes = 128;                        // bytes of K per row and step: 64 bf16 or 128 int8

template <int MT, bool INT8>     // MT = number of 32-row activation tiles, 1..4
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const uint8_t* __restrict__ x, const uint8_t* __restrict__ w,
                                                          void* __restrict__ partial, int M, int N, int64_t k_bytes,
                                                          int64_t ldx_bytes, int64_t ldw_bytes, int chunks_per_slice) {
  __shared__ __align__(16) uint8_t tile_w[kSkinnyBlockN * kRowStride];
  __shared__ __align__(16) uint8_t tile_x[MT * 32 * kRowStride];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 16;             // byte offset of this lane's 16 bytes inside a 32-byte K step
  const int n0 = blockIdx.x * kSkinnyBlockN;
  const int64_t k_begin = static_cast<int64_t>(blockIdx.y) * chunks_per_slice * kSkinnyChunkBytes;
  const int64_t k_stop = k_begin + static_cast<int64_t>(chunks_per_slice) * kSkinnyChunkBytes;
  const int64_t k_end = k_stop < k_bytes ? k_stop : k_bytes;

  // Tiles are rows of 8 chunks of 16 bytes; thread t moves chunks t, t + 256, ... (chunk c: row c / 8, bytes 16 (c % 8)).
  uint4 w_next[4], x_next[MT];
  auto fetch = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int chunk = tid + 256 * i;
      const int n = n0 + (chunk >> 3);
      const int64_t k = k0 + 16 * (chunk & 7);
      w_next[i] = make_uint4(0, 0, 0, 0);
      if (n < N && k < k_end) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(w + n * ldw_bytes + k));   // read once
        w_next[i] = make_uint4(v.x, v.y, v.z, v.w);
      }
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int chunk = tid + 256 * i;
      const int m = chunk >> 3;
      const int64_t k = k0 + 16 * (chunk & 7);
      x_next[i] = make_uint4(0, 0, 0, 0);
      if (m < M && k < k_end) x_next[i] = *reinterpret_cast<const uint4*>(x + m * ldx_bytes + k);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int chunk = tid + 256 * i;
      *reinterpret_cast<uint4*>(tile_w + (chunk >> 3) * kRowStride + 16 * (chunk & 7)) = w_next[i];
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int chunk = tid + 256 * i;
      *reinterpret_cast<uint4*>(tile_x + (chunk >> 3) * kRowStride + 16 * (chunk & 7)) = x_next[i];
    }
  };

  using Acc = typename std::conditional<INT8, i32x16, f32x16>::type;
  Acc acc[MT] = {};
  fetch(k_begin);
  for (int64_t k0 = k_begin; k0 < k_end; k0 += kSkinnyChunkBytes) {
    __syncthreads();                                 // every wave is done with the previous tiles
    stash();
    __syncthreads();
    if (k0 + kSkinnyChunkBytes < k_end) fetch(k0 + kSkinnyChunkBytes);
#pragma unroll
    for (int kk = 0; kk < kSkinnyChunkBytes / 32; ++kk) {
      const uint8_t* at_w = tile_w + (wave * 32 + frag_row) * kRowStride + kk * 32 + frag_k;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const uint8_t* at_x = tile_x + (t * 32 + frag_row) * kRowStride + kk * 32 + frag_k;
        if constexpr (INT8) {
          acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const i32x4*>(at_x), *reinterpret_cast<const i32x4*>(at_w), acc[t], 0, 0, 0);
        } else {
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(at_x), *reinterpret_cast<const bf16x8*>(at_w), acc[t], 0, 0, 0);
        }
      }
    }
  }

  // Register r of lane l holds activation row 8 (r / 4) + 4 (l / 32) + r % 4 of its tile, weight row l % 32.
  const int n = n0 + wave * 32 + frag_row;
  if (n >= N) return;
  using Cell = typename std::conditional<INT8, int32_t, float>::type;
  Cell* slab = static_cast<Cell*>(partial) + static_cast<int64_t>(blockIdx.y) * M * N;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = t * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
      if (m < M) slab[static_cast<int64_t>(m) * N + n] = acc[t][r];
    }
  }
}

// Adds the K slices. bf16 product: f32 sums + bias, one rounding. int8 product: int32 sums are exact, then
// f32(sum) * sa[m] * sb[n] + bias as single rounded operations (the same epilogue as the tiled kernels).
template <bool INT8>
__global__ __launch_bounds__(256) void gemm_skinny_finish_kernel(const void* __restrict__ partial, int slices, const float* __restrict__ scale_a,
                                                                 const float* __restrict__ scale_b, const void* __restrict__ bias,
                                                                 void* __restrict__ y, int M, int N, int64_t ldy, int out_kind) {
  const int64_t cell = blockIdx.x * int64_t{256} + threadIdx.x;
  if (cell >= static_cast<int64_t>(M) * N) return;
  const int m = static_cast<int>(cell / N), n = static_cast<int>(cell % N);
  float v;
  if constexpr (INT8) {
    int32_t sum = 0;
    for (int s = 0; s < slices; ++s) sum += static_cast<const int32_t*>(partial)[static_cast<int64_t>(s) * M * N + cell];
    v = __fmul_rn(__fmul_rn(static_cast<float>(sum), scale_a[m]), scale_b[n]);
    if (bias != nullptr) v = __fadd_rn(v, load_bias(bias, out_kind, n));
  } else {
    v = 0.0f;
    for (int s = 0; s < slices; ++s) v += static_cast<const float*>(partial)[static_cast<int64_t>(s) * M * N + cell];
    if (bias != nullptr) v += load_bias(bias, out_kind, n);
  }
  store_out(y, out_kind, static_cast<int64_t>(m) * ldy + n, v);
}

// The same sums and roundings, four consecutive cells of a row per thread (16-byte loads of the slabs, one store of the
// four results): for N and ldy multiples of 4 and y aligned to four outputs.
template <bool INT8>
__global__ __launch_bounds__(256) void gemm_finish_quads_kernel(const void* __restrict__ partial, int slices, const float* __restrict__ scale_a,
                                                                const float* __restrict__ scale_b, const void* __restrict__ bias,
                                                                void* __restrict__ y, int M, int N, int64_t ldy, int out_kind) {
  const int64_t cell = 4 * (blockIdx.x * int64_t{256} + threadIdx.x);
  const int64_t cells = static_cast<int64_t>(M) * N;
  if (cell >= cells) return;
  const int m = static_cast<int>(cell / N), n = static_cast<int>(cell % N);
  float v[4];
  if constexpr (INT8) {
    int4 sum = make_int4(0, 0, 0, 0);
    for (int s = 0; s < slices; ++s) {
      const int4 p = *reinterpret_cast<const int4*>(static_cast<const int32_t*>(partial) + static_cast<int64_t>(s) * cells + cell);
      sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
    }
    const int32_t sums[4] = {sum.x, sum.y, sum.z, sum.w};
    const float sa = scale_a[m];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = __fmul_rn(__fmul_rn(static_cast<float>(sums[i]), sa), scale_b[n + i]);
      if (bias != nullptr) v[i] = __fadd_rn(v[i], load_bias(bias, out_kind, n + i));
    }
  } else {
    float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int s = 0; s < slices; ++s) {
      const float4 p = *reinterpret_cast<const float4*>(static_cast<const float*>(partial) + static_cast<int64_t>(s) * cells + cell);
      sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
    }
    v[0] = sum.x; v[1] = sum.y; v[2] = sum.z; v[3] = sum.w;
    if (bias != nullptr) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += load_bias(bias, out_kind, n + i);
    }
  }
  const int64_t at = static_cast<int64_t>(m) * ldy + n;
  if (out_kind == kOutF32) {
    *reinterpret_cast<float4*>(static_cast<float*>(y) + at) = make_float4(v[0], v[1], v[2], v[3]);
  } else if (out_kind == kOutBF16) {
    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(y) + at) =
        make_uint2(bf16_bits_of(v[0]) | bf16_bits_of(v[1]) << 16, bf16_bits_of(v[2]) | bf16_bits_of(v[3]) << 16);
  } else {
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
    half4 h = {static_cast<_Float16>(v[0]), static_cast<_Float16>(v[1]), static_cast<_Float16>(v[2]), static_cast<_Float16>(v[3])};
    *reinterpret_cast<half4*>(static_cast<_Float16*>(y) + at) = h;
  }
}

template <bool INT8>
static void launch_finish(const void* partial, int slices, const float* scale_a, const float* scale_b, const void* bias, void* y, int M, int N,
                          int64_t ldy, int out_kind, hipStream_t s) {
  const int64_t cells = static_cast<int64_t>(M) * N;
  const uintptr_t four_outputs = out_kind == kOutF32 ? 16 : 8;
  if (N % 4 == 0 && ldy % 4 == 0 && reinterpret_cast<uintptr_t>(y) % four_outputs == 0 && reinterpret_cast<uintptr_t>(partial) % 16 == 0)
    hipLaunchKernelGGL(gemm_finish_quads_kernel<INT8>, dim3(static_cast<unsigned>((cells / 4 + 255) / 256)), dim3(256), 0, s, partial, slices,
                       scale_a, scale_b, bias, y, M, N, ldy, out_kind);
  else
    hipLaunchKernelGGL(gemm_skinny_finish_kernel<INT8>, dim3(static_cast<unsigned>((cells + 255) / 256)), dim3(256), 0, s, partial, slices,
                       scale_a, scale_b, bias, y, M, N, ldy, out_kind);
}

// K slices for an M x N product with `k_bytes` bytes per row on `cus` compute units: enough blocks for about four
// per CU, at least one chunk each.
static int skinny_slices(int64_t N, int64_t k_bytes, int cus) {
  const int64_t n_blocks = (N + kSkinnyBlockN - 1) / kSkinnyBlockN;
  const int64_t chunks = (k_bytes + kSkinnyChunkBytes - 1) / kSkinnyChunkBytes;
  int64_t slices = (4 * static_cast<int64_t>(cus) + n_blocks - 1) / n_blocks;
  slices = slices < 1 ? 1 : (slices > chunks ? chunks : slices);
  slices = slices > 64 ? 64 : slices;
  const int64_t per = (chunks + slices - 1) / slices;
  return static_cast<int>((chunks + per - 1) / per);
}

template <bool INT8>
static int launch_skinny(const void* x, const void* w, const float* scale_a, const float* scale_b, const void* bias, void* y, int64_t M,
                         int64_t N, int64_t k_bytes, int64_t ldx_bytes, int64_t ldw_bytes, int64_t ldy, int out_kind, int cus,
                         void* workspace, size_t workspace_bytes, hipStream_t s) {
  const int slices = skinny_slices(N, k_bytes, cus);
  if (workspace_bytes < static_cast<size_t>(slices) * static_cast<size_t>(M) * static_cast<size_t>(N) * 4) return EP_HIP_EINVAL;
  const int chunks = static_cast<int>((k_bytes + kSkinnyChunkBytes - 1) / kSkinnyChunkBytes);
  const int per = (chunks + slices - 1) / slices;
  const dim3 grid(static_cast<unsigned>((N + kSkinnyBlockN - 1) / kSkinnyBlockN), static_cast<unsigned>(slices));
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  const int m = static_cast<int>(M), n = static_cast<int>(N);
  if (M <= 32) hipLaunchKernelGGL((gemm_skinny_kernel<1, INT8>), grid, dim3(256), 0, s, xb, wb, workspace, m, n, k_bytes, ldx_bytes, ldw_bytes, per);
  else if (M <= 64) hipLaunchKernelGGL((gemm_skinny_kernel<2, INT8>), grid, dim3(256), 0, s, xb, wb, workspace, m, n, k_bytes, ldx_bytes, ldw_bytes, per);
  else if (M <= 96) hipLaunchKernelGGL((gemm_skinny_kernel<3, INT8>), grid, dim3(256), 0, s, xb, wb, workspace, m, n, k_bytes, ldx_bytes, ldw_bytes, per);
  else hipLaunchKernelGGL((gemm_skinny_kernel<4, INT8>), grid, dim3(256), 0, s, xb, wb, workspace, m, n, k_bytes, ldx_bytes, ldw_bytes, per);
  EP_HIP_TRY(hipGetLastError());
  launch_finish<INT8>(workspace, slices, scale_a, scale_b, bias, y, m, n, ldy, out_kind, s);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

// ---- a few hundred activation rows: 128 x 128 tiles with K split over blocks ----------------------------------------------
//
// A CU moves operand bytes into its LDS at a bounded rate (about 80 GB/s when they come from the last-level cache and 55-60
// GB/s from memory on an MI355X: a bounded number of requests in flight, over the latency). A 128 x 128 tile of a product
// with K = 3072 takes 1.5 MB of operands, 19 us at the first rate and 27-32 us at the second, whatever the pipeline's
// depth, and a product of 48 such tiles leaves four CUs in five idle meanwhile. So when the tiles are at most half as many
// as the CUs, K is divided over `slices` blocks per tile (the four-stage kernel above with SPLIT), each CU moves 1 / slices
// of the bytes, and the kernel that adds the skinny product's slices adds these.
static int split_slices(int64_t M, int64_t N, int64_t k_bytes, int cus) {
  if (M <= 128 || k_bytes % kTileBytesK != 0) return 0;
  if (few_tiles_take_small_blocks(M, N, k_bytes, cus)) return 0;       // one kernel of 64 x 64 blocks does better than two
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  const int64_t steps = k_bytes / kTileBytesK;
  int64_t most = cus / tiles;
  most = most > 8 ? 8 : most;
  for (int64_t slices = most; slices >= 2; --slices)
    if (steps % (4 * slices) == 0 && steps / slices >= 8) return static_cast<int>(slices);   // whole rounds of the kernel's four-step loop
  return 0;
}

template <bool INT8>
static int launch_split(const void* x, const void* w, const float* scale_a, const float* scale_b, const void* bias, void* y, int64_t M,
                        int64_t N, int64_t k_bytes, int64_t ldx_bytes, int64_t ldw_bytes, int64_t ldy, int out_kind, int slices,
                        void* workspace, size_t workspace_bytes, hipStream_t s) {
  if (workspace_bytes < static_cast<size_t>(slices) * static_cast<size_t>(M) * static_cast<size_t>(N) * 4) return EP_HIP_EINVAL;
  const dim3 grid(static_cast<unsigned>((N + 127) / 128), static_cast<unsigned>((M + 127) / 128), static_cast<unsigned>(slices));
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  const int m = static_cast<int>(M), n = static_cast<int>(N);
  if (M % 128 == 0 && N % 128 == 0)
    hipLaunchKernelGGL((gemm_deep_kernel<INT8, false, true>), grid, dim3(256), 0, s, xb, wb, nullptr, nullptr, nullptr, workspace, m, n, k_bytes,
                       ldx_bytes, ldw_bytes, int64_t{0}, 0);
  else
    hipLaunchKernelGGL((gemm_deep_kernel<INT8, true, true>), grid, dim3(256), 0, s, xb, wb, nullptr, nullptr, nullptr, workspace, m, n, k_bytes,
                       ldx_bytes, ldw_bytes, int64_t{0}, 0);
  EP_HIP_TRY(hipGetLastError());
  launch_finish<INT8>(workspace, slices, scale_a, scale_b, bias, y, m, n, ldy, out_kind, s);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

static int out_kind_valid(int kind) { return kind == kOutBF16 || kind == kOutF16 || kind == kOutF32; }

}  // namespace ep

namespace ep {

// Four consecutive elements as one 8- or 16-byte load, four codes as one 4-byte store, a whole row in the registers of
// one workgroup.
constexpr int64_t kQuantiseRegisterColumns = 32768;
static bool rows_take_wide_loads(const void* x, int in_kind, int64_t K, int64_t ldx, const void* codes) {
  const uintptr_t element = in_kind == kOutF32 ? 4 : 2;
  return K % 4 == 0 && K <= kQuantiseRegisterColumns && ldx % 4 == 0 && reinterpret_cast<uintptr_t>(x) % (4 * element) == 0 && reinterpret_cast<uintptr_t>(codes) % 4 == 0;
}

template <int IN_KIND>
static void launch_rotate_quantize_of(const void* x, int64_t rows, int64_t K, int64_t ldx, int stages, int8_t* codes, float* scales,
                                      hipStream_t s) {
  const dim3 grid(static_cast<unsigned>(rows)), block(256);
  const int k = static_cast<int>(K);
  // A wave holds 1024 elements: rows of 2049..3072 run three waves instead of four with one idle (measured 12 % faster;
  // shorter rows measured no better with smaller blocks).
  if (K <= 4096) hipLaunchKernelGGL((rotate_quantize_rows_kernel<IN_KIND, 1>), grid, dim3(K > 2048 && K <= 3072 ? 192 : 256), 0, s, x, ldx, k, stages, codes, scales);
  else if (K <= 8192) hipLaunchKernelGGL((rotate_quantize_rows_kernel<IN_KIND, 2>), grid, block, 0, s, x, ldx, k, stages, codes, scales);
  else if (K <= 16384) hipLaunchKernelGGL((rotate_quantize_rows_kernel<IN_KIND, 4>), grid, block, 0, s, x, ldx, k, stages, codes, scales);
  else hipLaunchKernelGGL((rotate_quantize_rows_kernel<IN_KIND, 8>), grid, block, 0, s, x, ldx, k, stages, codes, scales);
}

static int launch_rotate_quantize(const void* x, int in_kind, int64_t rows, int64_t K, int64_t ldx, int stages, int8_t* codes,
                                  float* scales, void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_kind == kOutBF16) launch_rotate_quantize_of<kOutBF16>(x, rows, K, ldx, stages, codes, scales, s);
  else if (in_kind == kOutF16) launch_rotate_quantize_of<kOutF16>(x, rows, K, ldx, stages, codes, scales, s);
  else launch_rotate_quantize_of<kOutF32>(x, rows, K, ldx, stages, codes, scales, s);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

}  // namespace ep

extern "C" {

int ep_hip_gemm_bf16(const void* x_dev, const void* w_dev, const void* bias_dev, void* y_dev, int64_t M, int64_t N,
                     int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int out_kind, void* stream) {
  using namespace ep;
  if (x_dev == nullptr || w_dev == nullptr || y_dev == nullptr) return EP_HIP_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF) return EP_HIP_EINVAL;
  if (K % 8 != 0 || ldx % 8 != 0 || ldw % 8 != 0 || ldx < K || ldw < K || ldy < N) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(x_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(w_dev) % 16 != 0) return EP_HIP_EINVAL;
  if (!out_kind_valid(out_kind)) return EP_HIP_EINVAL;
  const int columns = small_whole_tiles<false>(M, N, K * 2) ? whole_k_tiling(M, N, K * 2, current_compute_units()) : big_tile_columns(M, N, K * 2);
  if (columns != 0) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    return columns == 256 ? launch_big<false, 256>(x_dev, w_dev, nullptr, nullptr, bias_dev, y_dev, M, N, K * 2, ldx * 2, ldw * 2, ldy, out_kind, s)
                          : launch_big<false, 192>(x_dev, w_dev, nullptr, nullptr, bias_dev, y_dev, M, N, K * 2, ldx * 2, ldw * 2, ldy, out_kind, s);
  }
  if (small_whole_tiles<false>(M, N, K * 2))
    return launch_direct_small<false>(x_dev, w_dev, nullptr, nullptr, bias_dev, y_dev, M, N, K * 2, ldx * 2, ldw * 2, ldy, out_kind, static_cast<hipStream_t>(stream));
  const dim3 grid(static_cast<unsigned>((N + kBlockN - 1) / kBlockN), static_cast<unsigned>((M + kBlockM - 1) / kBlockM));
  if (grid.y > 65535) return EP_HIP_EUNSUPPORTED;
  hipLaunchKernelGGL(gemm_bf16_nt_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(x_dev), static_cast<const uint16_t*>(w_dev), bias_dev, y_dev,
                     static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), ldx, ldw, ldy, out_kind);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

int ep_hip_gemm_takes_small_blocks(int64_t M, int64_t N, int64_t k_bytes, int compute_units) {
  if (M <= 0 || N <= 0 || k_bytes <= 0 || compute_units <= 0) return 0;
  return ep::small_whole_tiles<false>(M, N, k_bytes) && ep::few_tiles_take_small_blocks(M, N, k_bytes, compute_units) ? 1 : 0;
}

size_t ep_hip_gemm_skinny_workspace(int64_t M, int64_t N, int64_t k_bytes, int compute_units) {
  using namespace ep;
  if (M <= 0 || N <= 0 || k_bytes <= 0 || compute_units <= 0) return 0;
  const int slices = M <= 128 ? skinny_slices(N, k_bytes, compute_units) : split_slices(M, N, k_bytes, compute_units);
  return static_cast<size_t>(slices) * static_cast<size_t>(M) * static_cast<size_t>(N) * 4;
}

int ep_hip_gemm_bf16_skinny(const void* x_dev, const void* w_dev, const void* bias_dev, void* y_dev, int64_t M, int64_t N,
                            int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int out_kind, int compute_units,
                            void* workspace_dev, size_t workspace_bytes, void* stream) {
  using namespace ep;
  if (x_dev == nullptr || w_dev == nullptr || y_dev == nullptr || workspace_dev == nullptr) return EP_HIP_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x3FFFFFFF || compute_units <= 0) return EP_HIP_EINVAL;
  if (K % 8 != 0 || ldx % 8 != 0 || ldw % 8 != 0 || ldx < K || ldw < K || ldy < N) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(x_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(w_dev) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(workspace_dev) % 16 != 0) return EP_HIP_EINVAL;
  if (!out_kind_valid(out_kind)) return EP_HIP_EINVAL;
  if (M > 128) {
    const int slices = split_slices(M, N, K * 2, compute_units);
    if (slices == 0) return EP_HIP_EUNSUPPORTED;
    return launch_split<false>(x_dev, w_dev, nullptr, nullptr, bias_dev, y_dev, M, N, K * 2, ldx * 2, ldw * 2, ldy, out_kind, slices,
                               workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
  }
  return launch_skinny<false>(x_dev, w_dev, nullptr, nullptr, bias_dev, y_dev, M, N, K * 2, ldx * 2, ldw * 2, ldy, out_kind, compute_units,
                              workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
}

int ep_hip_gemm_i8_skinny(const int8_t* a_dev, const int8_t* b_dev, const float* scale_a_dev, const float* scale_b_dev,
                          const void* bias_dev, void* y_dev, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                          int64_t ldy, int out_kind, int compute_units, void* workspace_dev, size_t workspace_bytes, void* stream) {
  using namespace ep;
  if (a_dev == nullptr || b_dev == nullptr || scale_a_dev == nullptr || scale_b_dev == nullptr || y_dev == nullptr ||
      workspace_dev == nullptr) return EP_HIP_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF || compute_units <= 0) return EP_HIP_EINVAL;
  if (K % 16 != 0 || lda % 16 != 0 || ldb % 16 != 0 || lda < K || ldb < K || ldy < N) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(a_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(b_dev) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(workspace_dev) % 16 != 0) return EP_HIP_EINVAL;
  if (!out_kind_valid(out_kind)) return EP_HIP_EINVAL;
  if (M > 128) {
    const int slices = split_slices(M, N, K, compute_units);
    if (slices == 0) return EP_HIP_EUNSUPPORTED;
    return launch_split<true>(a_dev, b_dev, scale_a_dev, scale_b_dev, bias_dev, y_dev, M, N, K, lda, ldb, ldy, out_kind, slices,
                              workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
  }
  return launch_skinny<true>(a_dev, b_dev, scale_a_dev, scale_b_dev, bias_dev, y_dev, M, N, K, lda, ldb, ldy, out_kind, compute_units,
                             workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
}

int ep_hip_gemm_i8(const int8_t* a_dev, const int8_t* b_dev, const float* scale_a_dev, const float* scale_b_dev,
                   const void* bias_dev, void* y_dev, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                   int64_t ldy, int out_kind, void* stream) {
  using namespace ep;
  if (a_dev == nullptr || b_dev == nullptr || scale_a_dev == nullptr || scale_b_dev == nullptr || y_dev == nullptr) return EP_HIP_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF) return EP_HIP_EINVAL;
  if (K % 16 != 0 || lda % 16 != 0 || ldb % 16 != 0 || lda < K || ldb < K || ldy < N) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(a_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(b_dev) % 16 != 0) return EP_HIP_EINVAL;
  if (!out_kind_valid(out_kind)) return EP_HIP_EINVAL;
  if (const int columns = small_whole_tiles<true>(M, N, K) ? whole_k_tiling(M, N, K, current_compute_units()) : big_tile_columns(M, N, K)) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    return columns == 256 ? launch_big<true, 256>(a_dev, b_dev, scale_a_dev, scale_b_dev, bias_dev, y_dev, M, N, K, lda, ldb, ldy, out_kind, s)
                          : launch_big<true, 192>(a_dev, b_dev, scale_a_dev, scale_b_dev, bias_dev, y_dev, M, N, K, lda, ldb, ldy, out_kind, s);
  }
  if (small_whole_tiles<true>(M, N, K))
    return launch_direct_small<true>(a_dev, b_dev, scale_a_dev, scale_b_dev, bias_dev, y_dev, M, N, K, lda, ldb, ldy, out_kind, static_cast<hipStream_t>(stream));
  const dim3 grid(static_cast<unsigned>((N + kBlockN - 1) / kBlockN), static_cast<unsigned>((M + kBlockM - 1) / kBlockM));
  if (grid.y > 65535) return EP_HIP_EUNSUPPORTED;
  hipLaunchKernelGGL(gemm_i8_nt_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a_dev, b_dev, scale_a_dev,
                     scale_b_dev, bias_dev, y_dev, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), lda, ldb,
                     ldy, out_kind);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

int ep_hip_quantize_rows(const void* x_dev, int in_kind, int64_t rows, int64_t K, int64_t ldx, int8_t* codes_dev,
                         float* scales_dev, void* stream) {
  using namespace ep;
  if (x_dev == nullptr || codes_dev == nullptr || scales_dev == nullptr) return EP_HIP_EINVAL;
  if (rows <= 0 || K <= 0 || rows > 0x7FFFFFFF || K > 0x7FFFFFFF || ldx < K || !out_kind_valid(in_kind)) return EP_HIP_EINVAL;
  // Two-byte activations in whole 16-byte pieces: one wave per row.
  if (in_kind != kOutF32 && K % 8 == 0 && K <= 8192 && ldx % 8 == 0 && reinterpret_cast<uintptr_t>(x_dev) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(codes_dev) % 8 == 0) {
    const dim3 grid(static_cast<unsigned>((rows + 3) / 4));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t* x = static_cast<const uint16_t*>(x_dev);
    const int k = static_cast<int>(K), m = static_cast<int>(rows);
#define EP_QUANTISE_WAVE(KIND, CHUNKS) hipLaunchKernelGGL((quantize_rows_wave_kernel<KIND, CHUNKS>), grid, dim3(256), 0, s, x, ldx, k, m, codes_dev, scales_dev)
    // A chunk is 512 elements of the row: no more of them than the row has.
#define EP_QUANTISE_WAVE_KIND(KIND)                      \
    if (K <= 1024) EP_QUANTISE_WAVE(KIND, 2);            \
    else if (K <= 2048) EP_QUANTISE_WAVE(KIND, 4);       \
    else if (K <= 3072) EP_QUANTISE_WAVE(KIND, 6);       \
    else if (K <= 4096) EP_QUANTISE_WAVE(KIND, 8);       \
    else if (K <= 6144) EP_QUANTISE_WAVE(KIND, 12);      \
    else EP_QUANTISE_WAVE(KIND, 16)
    if (in_kind == kOutBF16) {
      EP_QUANTISE_WAVE_KIND(kOutBF16);
    } else {
      EP_QUANTISE_WAVE_KIND(kOutF16);
    }
#undef EP_QUANTISE_WAVE_KIND
#undef EP_QUANTISE_WAVE
    EP_HIP_TRY(hipGetLastError());
    return EP_HIP_OK;
  }
  if (rows_take_wide_loads(x_dev, in_kind, K, ldx, codes_dev)) return launch_rotate_quantize(x_dev, in_kind, rows, K, ldx, 0, codes_dev, scales_dev, stream);
  hipLaunchKernelGGL(quantize_rows_kernel, dim3(static_cast<unsigned>(rows)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     x_dev, in_kind, ldx, static_cast<int>(K), codes_dev, scales_dev);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

int ep_hip_rotate_quantize_rows(const void* x_dev, int in_kind, int64_t rows, int64_t K, int64_t ldx, int group,
                                int8_t* codes_dev, float* scales_dev, void* stream) {
  using namespace ep;
  if (x_dev == nullptr || codes_dev == nullptr || scales_dev == nullptr) return EP_HIP_EINVAL;
  if (rows <= 0 || K <= 0 || rows > 0x7FFFFFFF || K > 0x7FFFFFFF || ldx < K || !out_kind_valid(in_kind)) return EP_HIP_EINVAL;
  int stages = 0;
  while (stages < 16 && (1 << (2 * stages)) < group) ++stages;
  if (group < 4 || (1 << (2 * stages)) != group || K % group != 0) return EP_HIP_EINVAL;       // a power of four dividing K
  if (group > 256) return EP_HIP_EUNSUPPORTED;                                                   // a wave holds 256 elements
  if (!rows_take_wide_loads(x_dev, in_kind, K, ldx, codes_dev)) return EP_HIP_EUNSUPPORTED;
  return launch_rotate_quantize(x_dev, in_kind, rows, K, ldx, stages, codes_dev, scales_dev, stream);
}

}  // extern "C"
