// Decode kernel arguments and the container casts / vector stores shared by the decode kernels.
#pragma once

#include "ep_common.hpp"

namespace ep {

struct DecodeArgs {
  const uint16_t* payload;
  uint64_t payload_words;
  const uint32_t* offsets;
  const uint32_t* states;
  const float* scales;
  const uint32_t* plan;     // header + tables
  void* out;
  int store_kind;
  int vecs_per_row;
  uint32_t row_magic;       // row = umulhi(v << row_pre, row_magic) >> row_shift
  int row_shift;
  int row_pre;
  int64_t num_vectors;
  int tile_vectors;
  int num_tiles;
  int* error;
  uint32_t lut_bytes;       // LDS_RANK: bytes of tables to stage, and where the value and rank/select parts start
  uint32_t rank_val_offset;
  uint32_t rank_rs_offset;
  uint32_t rank_half;       // LDS_RANK: the value table holds half-precision coordinates
  const uint8_t* sym_tables;   // the plan's two-level (LDS_SYM) section, or null
  uint32_t store_cached;       // bf16 stores go through the cache instead of streaming (tiles that split 64-byte pieces between groups)
  uint32_t reserved;
  // Multiply-on-the-fly kernels only: activations x[m_rows][ldx] (bf16) and the f32 accumulator y32[m_rows][ldy32].
  int m_rows;
  const uint16_t* x;
  int64_t ldx;
  float* y32;
  int64_t ldy32;
};

__device__ __forceinline__ void flag_error(int* error, int code) { atomicCAS(error, 0, code); }

// ---- container casts (format.py:153-168 / lattice_rans.cu:560-653 of the reference) -----------------------

__device__ __forceinline__ uint32_t bf16_bits_rne(float v) {
  const uint32_t bits = __float_as_uint(v);
  return (bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16;      // finite input
}

__device__ __forceinline__ float clamp_bf16(float v) {
  return __builtin_fminf(__builtin_fmaxf(v, -3.3895313892515355e38f), 3.3895313892515355e38f);
}

__device__ __forceinline__ uint32_t f16_bits(float v) {
  const _Float16 h = static_cast<_Float16>(__builtin_fminf(__builtin_fmaxf(v, -65504.0f), 65504.0f));
  return __builtin_bit_cast(unsigned short, h);
}

// Round-to-nearest-even float -> OCP fp8 after saturating to the largest finite value.
template <int MBITS, int BIAS>
__device__ __forceinline__ uint32_t fp8_bits(float v, float limit) {
  const uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
  float a = __builtin_fminf(__builtin_fabsf(v), limit);
  const float min_normal = __uint_as_float(static_cast<uint32_t>(127 + 1 - BIAS) << 23);
  if (!(a >= min_normal)) {
    const float quantum = __uint_as_float(static_cast<uint32_t>(127 + 1 - BIAS - MBITS) << 23);
    return sign | static_cast<uint32_t>(__builtin_rintf(a / quantum));
  }
  const uint32_t bits = __float_as_uint(a);
  const int exponent = static_cast<int>(bits >> 23) - 127 + BIAS;
  constexpr int kShift = 23 - MBITS;
  const uint32_t mant = bits & 0x7FFFFFu;
  uint32_t r = mant >> kShift;
  const uint32_t rest = mant & ((1u << kShift) - 1u);
  constexpr uint32_t kHalf = 1u << (kShift - 1);
  r += (rest > kHalf) || (rest == kHalf && (r & 1u));
  return sign | ((static_cast<uint32_t>(exponent) << MBITS) + r);
}

template <typename T>
__device__ __forceinline__ T snap_integer(float v, float low, float high_exclusive) {
  const float high = __uint_as_float(__float_as_uint(high_exclusive) - 1u);   // nextafter(high_exclusive, 0)
  return static_cast<T>(__builtin_fminf(__builtin_fmaxf(__builtin_rintf(v), low), high));
}

// The decoded tensor is written once and not read back by the kernel: streaming (non-temporal) stores keep the write
// traffic from queueing in front of the payload prefetches that share the memory counter with it.
typedef uint32_t ep_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ep_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void stream_store16(void* at, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const ep_u32x4 v = {a, b, c, d};
  __builtin_nontemporal_store(v, reinterpret_cast<ep_u32x4*>(at));
}
__device__ __forceinline__ void stream_store8(void* at, uint32_t a, uint32_t b) {
  const ep_u32x2 v = {a, b};
  __builtin_nontemporal_store(v, reinterpret_cast<ep_u32x2*>(at));
}

// int8 container, the kind the int8 linear layer decodes to: rint (half to even), clamp to [-128, 127], pack.
// Clamping first gives the same result (the bounds are integers). Adding 1.5 * 2^23 to a value in [-128, 127] rounds it
// to an integer, ties to even, in the sum's mantissa, whose low byte is then the two's-complement code; the add writes
// that byte straight into its place in the packed word (sub-dword destination select), so a weight costs a clamp and an add.
__device__ __forceinline__ void codes_i8(const float (&w)[8], uint32_t& low, uint32_t& high) {
  float magic = 12582912.0f;
  asm volatile("" : "+v"(magic));          // a vector register: the sub-dword form takes no literal
  // Few vectors hold a value outside [-128, 127]: one magnitude test for all eight instead of eight clamps.
  float c[8];
  float top = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    c[i] = w[i];
    top = __builtin_fmaxf(top, __builtin_fabsf(w[i]));
  }
  if (__builtin_expect(top > 127.0f, 0)) {
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = __builtin_fminf(__builtin_fmaxf(w[i], -128.0f), 127.0f);
  }
  // The two words alternate: an instruction that keeps the other bytes of its destination must not directly follow
  // the one that wrote them (sub-dword writes need one instruction in between on this hardware).
#define EP_I8_ADD(DST, SRC, BYTE, UNUSED) \
  "v_add_f32_sdwa " DST ", " SRC ", %10 dst_sel:" BYTE " dst_unused:" UNUSED " src0_sel:DWORD src1_sel:DWORD\n"
  asm(EP_I8_ADD("%0", "%2", "BYTE_0", "UNUSED_PAD") EP_I8_ADD("%1", "%6", "BYTE_0", "UNUSED_PAD")
      EP_I8_ADD("%0", "%3", "BYTE_1", "UNUSED_PRESERVE") EP_I8_ADD("%1", "%7", "BYTE_1", "UNUSED_PRESERVE")
      EP_I8_ADD("%0", "%4", "BYTE_2", "UNUSED_PRESERVE") EP_I8_ADD("%1", "%8", "BYTE_2", "UNUSED_PRESERVE")
      EP_I8_ADD("%0", "%5", "BYTE_3", "UNUSED_PRESERVE") EP_I8_ADD("%1", "%9", "BYTE_3", "UNUSED_PRESERVE")
      "s_nop 0\n"
      : "=&v"(low), "=&v"(high)
      : "v"(c[0]), "v"(c[1]), "v"(c[2]), "v"(c[3]), "v"(c[4]), "v"(c[5]), "v"(c[6]), "v"(c[7]), "v"(magic));
#undef EP_I8_ADD
}

__device__ __forceinline__ void store_vector_i8(void* out, int64_t vector, const float (&w)[8]) {
  uint32_t low, high;
  codes_i8(w, low, high);
  stream_store8(reinterpret_cast<uint2*>(out) + vector, low, high);
}

// Writes the eight values of vector `vector` in any container kind.
__device__ __forceinline__ void store_vector(void* out, int kind, int64_t vector, const float (&w)[8]) {
  switch (kind) {
    case EP_STORE_BF16: {
      uint32_t p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) p[i] = bf16_bits_rne(clamp_bf16(w[2 * i])) | (bf16_bits_rne(clamp_bf16(w[2 * i + 1])) << 16);
      stream_store16(reinterpret_cast<uint4*>(out) + vector, p[0], p[1], p[2], p[3]);
      break;
    }
    case EP_STORE_F16: {
      // Saturation to the largest finite half is needed by very few vectors: one magnitude test for all eight
      // values, then packed round-to-nearest-even conversions.
      float v[8];
      float top = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[i] = w[i];
        top = __builtin_fmaxf(top, __builtin_fabsf(w[i]));
      }
      if (__builtin_expect(top > 65504.0f, 0)) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_fminf(__builtin_fmaxf(w[i], -65504.0f), 65504.0f);
      }
      uint32_t p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        typedef float float2v __attribute__((ext_vector_type(2)));
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        const float2v two = {v[2 * i], v[2 * i + 1]};
        p[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(two, half2v));
      }
      stream_store16(reinterpret_cast<uint4*>(out) + vector, p[0], p[1], p[2], p[3]);
      break;
    }
    case EP_STORE_F32: {
      // 32 bytes per lane: two stores that each leave 16-byte gaps, which streaming stores handle badly (389 us
      // against 344 us on 8192 x 28672), so these go through the cache.
      float4* dst = reinterpret_cast<float4*>(out) + vector * 2;
      dst[0] = make_float4(w[0], w[1], w[2], w[3]);
      dst[1] = make_float4(w[4], w[5], w[6], w[7]);
      break;
    }
    case EP_STORE_F8E4M3FN:
    case EP_STORE_F8E5M2:
    case EP_STORE_I8:
    case EP_STORE_U8:
    case EP_STORE_BOOL: {
      uint32_t b[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (kind == EP_STORE_F8E4M3FN) b[i] = fp8_bits<3, 7>(w[i], 448.0f);
        else if (kind == EP_STORE_F8E5M2) b[i] = fp8_bits<2, 15>(w[i], 57344.0f);
        else if (kind == EP_STORE_I8) b[i] = static_cast<uint8_t>(snap_integer<int8_t>(w[i], -128.0f, 128.0f));
        else if (kind == EP_STORE_U8) b[i] = snap_integer<uint8_t>(w[i], 0.0f, 256.0f);
        else b[i] = __builtin_rintf(w[i]) != 0.0f;
      }
      stream_store8(reinterpret_cast<uint2*>(out) + vector, b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24),
                    b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24));
      break;
    }
    case EP_STORE_I16:
    case EP_STORE_U16: {
      uint32_t b[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        b[i] = kind == EP_STORE_I16 ? static_cast<uint16_t>(snap_integer<int16_t>(w[i], -32768.0f, 32768.0f))
                                    : snap_integer<uint16_t>(w[i], 0.0f, 65536.0f);
      }
      stream_store16(reinterpret_cast<uint4*>(out) + vector, b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16));
      break;
    }
    case EP_STORE_I32:
    case EP_STORE_U32: {
      uint32_t b[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        b[i] = kind == EP_STORE_I32 ? static_cast<uint32_t>(snap_integer<int32_t>(w[i], -2147483648.0f, 2147483648.0f))
                                    : snap_integer<uint32_t>(w[i], 0.0f, 4294967296.0f);
      }
      uint4* dst = reinterpret_cast<uint4*>(out) + vector * 2;
      dst[0] = make_uint4(b[0], b[1], b[2], b[3]);
      dst[1] = make_uint4(b[4], b[5], b[6], b[7]);
      break;
    }
    default: {   // EP_STORE_I64 / EP_STORE_U64
      uint64_t* dst = reinterpret_cast<uint64_t*>(out) + vector * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        dst[i] = kind == EP_STORE_I64
                     ? static_cast<uint64_t>(snap_integer<int64_t>(w[i], -9223372036854775808.0f, 9223372036854775808.0f))
                     : snap_integer<uint64_t>(w[i], 0.0f, 18446744073709551616.0f);
      }
      break;
    }
  }
}

__device__ __forceinline__ uint32_t row_of(const DecodeArgs& a, uint32_t vector) {
  return __umulhi(vector << a.row_pre, a.row_magic) >> a.row_shift;
}

// Launches the LDS-table decode kernel (ep_decode_lds.hip) for an EP_TABLE_LDS_* plan.
// A block's share of a batch: pairs [first_pair, first_pair + n_pairs) of container `job`.
struct BlockJob {
  int job;
  int first_pair;
  int n_pairs;
  int reserved;
};

// Launch shape of the LDS-table kernels for one container, or for the containers of a batch that share it.
struct LdsLaunch {
  int table_kind;
  int prob_bits;
  int kind;         // EP_STORE_BF16 (specialised store), -1 (any container), -2 / -3 (multiply on the fly, 1 / up to 4 rows)
  int ilp;          // tile pairs per wave
  int threads;
  int lds_bytes;
  int blocks;
};

// Kernel variant for a container kind: the two kinds the linear layers decode to have specialised stores, the rest
// share the generic one (-1).
inline int kernel_kind_of(int store_kind) { return store_kind == EP_STORE_BF16 || store_kind == EP_STORE_I8 ? store_kind : -1; }

int lds_resident_blocks(int table_kind, int prob_bits, int lut_bytes);
LdsLaunch choose_lds_launch(int table_kind, int prob_bits, int lut_bytes, int kind, int pairs, int cus);
int launch_lds(const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, const DecodeArgs* jobs, const BlockJob* block_jobs,
               uint8_t* arena, hipStream_t stream);
int launch_rank(const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, const DecodeArgs* jobs, const BlockJob* block_jobs,
                uint8_t* arena, hipStream_t stream);
int launch_dot(const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, hipStream_t stream);
int launch_sym(const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, const DecodeArgs* jobs, const BlockJob* block_jobs,
               uint8_t* arena, hipStream_t stream);
// The table form a launch of `pairs` tile pairs really uses: byte plans with a two-level section switch to it once
// the launch is larger than one pass of resident waves (where occupancy, not the length of a step, sets the pace).
int effective_table_kind(const ep_hip_plan_desc& desc, int kind, int64_t pairs, int cus);
int launch_lds_decode(const DecodeArgs& args, const ep_hip_plan_desc& desc, int kind, int num_pairs, hipStream_t stream);
// Decode-to-GEMM through LDS (ep_decode_mfma.hip): args.x / m_rows / y32 set, one workgroup per batch and block of rows.
int launch_fused_mfma(const DecodeArgs& args, const ep_hip_plan_desc& desc, const ep_hip_fused_batch* batches, int n_batches, bool int8,
                      const float* scale_a, const float* scale_b, const void* bias, void* y, int64_t ldy, int out_kind, hipStream_t stream);
size_t fused_workspace_bytes(int64_t rows, int64_t cols_padded, int tile_elements, int64_t m_rows, int element_bytes);

}  // namespace ep
