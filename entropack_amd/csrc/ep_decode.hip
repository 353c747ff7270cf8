// lattice_rans decode for gfx950: the C-ABI entry point and the catch-all kernel.
//
// A tile owns 32 interleaved rANS lanes, so one wave64 carries two tiles, one per 32-lane half; every ballot and
// prefix count is taken per half. Per vector: coset c from stream 0, fields f = 0..7 from stream 1 + 2f + c,
// z7 = 2 m + parity, w_j = f32_mul(float(z_j) + c / 2, scale[row]), then the container cast of w_j.
//
//   decode_global64_kernel (here)      any container: u64 slot table and payload words read from global memory,
//                                      every renormalisation read bounds-checked.
//   decode_lds_kernel (ep_decode_lds)  prob_bits <= 11: u32 slot table staged in LDS, payload streamed through an
//                                      LDS ring.
// Both produce bit-identical output.
#include "ep_store.hpp"

namespace ep {

// ---- any container: tables and payload in global memory ----------------------------------------------------

__global__ __launch_bounds__(256) void decode_global64_kernel(DecodeArgs a) {
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int64_t tile = 2 * (static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) + half;
  const int pb = static_cast<int>(a.plan[kHdrProbBits]);
  const uint32_t slot_mask = (1u << pb) - 1u;
  const uint64_t* lut = reinterpret_cast<const uint64_t*>(reinterpret_cast<const uint8_t*>(a.plan) + kHeaderBytes);
  const int32_t* sym_min = reinterpret_cast<const int32_t*>(a.plan) + kHdrSymMin;

  int64_t word_begin = 0, pointer = 0;
  int count = 0;
  uint32_t x = kStateMin;
  const int64_t vector_begin = tile * a.tile_vectors;
  if (tile < a.num_tiles) {
    word_begin = a.offsets[tile];
    pointer = a.offsets[tile + 1];
    const int64_t left = a.num_vectors - vector_begin;
    count = static_cast<int>(left < a.tile_vectors ? left : a.tile_vectors);
    if (word_begin > pointer || static_cast<uint64_t>(pointer) > a.payload_words) {
      flag_error(a.error, EP_DECODE_BAD_OFFSETS);
      count = 0;
    } else {
      x = a.states[tile * kStatesPerTile + l32];
    }
  }
  const bool checked_tile = count > 0;
  const int groups = (count + 31) >> 5;
  const int rem = count & 31;
  const int other = __shfl_xor(groups, 32);
  const int rounds = groups > other ? groups : other;

  auto renormalise = [&](bool valid) {
    const bool read = valid && x < kStateMin;
    const uint64_t vote = __ballot(read);
    const uint32_t mine = half ? static_cast<uint32_t>(vote >> 32) : static_cast<uint32_t>(vote);
    if (read) {
      const int64_t at = pointer - __popc(mine >> l32);    // readers at or above this lane, itself included
      uint32_t word = 0;
      if (at >= word_begin) word = a.payload[at];
      else flag_error(a.error, EP_DECODE_OVERREAD);
      x = (x << 16) | word;
    }
    pointer -= __popc(mine);
  };

  for (int round = 0; round < rounds; ++round) {
    const bool active = round < groups;
    const int offset = (groups - 1 - round) << 5;
    const int lanes = (round == 0 && rem != 0) ? rem : 32;
    const bool valid = active && l32 < lanes;
    int c = 0;
    int value[8];
    if (valid) {
      const uint32_t slot = x & slot_mask;
      const uint64_t entry = lut[slot];
      c = static_cast<int>(entry & 1u);
      x = (static_cast<uint32_t>(entry >> 16) & 0xFFFFu) * (x >> pb) + static_cast<uint32_t>(entry >> 32);
    }
    renormalise(valid);
#pragma unroll
    for (int f = 0; f < kFields; ++f) {
      if (valid) {
        const int table = 1 + 2 * f + c;
        const uint32_t slot = x & slot_mask;
        const uint64_t entry = lut[(static_cast<size_t>(table) << pb) + slot];
        value[f] = static_cast<int>(entry & 0xFFFFu) + sym_min[table];
        x = (static_cast<uint32_t>(entry >> 16) & 0xFFFFu) * (x >> pb) + static_cast<uint32_t>(entry >> 32);
      }
      renormalise(valid);
    }
    if (valid) {
      int parity = 0;
#pragma unroll
      for (int f = 0; f < 7; ++f) parity += value[f];
      value[7] = 2 * value[7] + (parity & 1);
      const int64_t vector = vector_begin + offset + l32;
      const float scale = a.scales[vector / a.vecs_per_row];
      const float shift = c ? 0.5f : 0.0f;
      float w[8];
#pragma unroll
      for (int f = 0; f < 8; ++f) w[f] = __fmul_rn(__fadd_rn(static_cast<float>(value[f]), shift), scale);
      store_vector(a.out, a.store_kind, vector, w);
    }
  }
  if (checked_tile && (pointer != word_begin || x != kStateMin)) flag_error(a.error, EP_DECODE_NOT_CONSUMED);
}

}  // namespace ep

extern "C" int ep_hip_decode_lattice(const uint16_t* payload_dev, uint64_t payload_words, const uint32_t* offsets_dev,
                                     const uint32_t* states_dev, const float* scales_dev, const void* tables_dev,
                                     const ep_hip_plan_desc* desc, void* out_dev, int store_kind, int64_t rows,
                                     int64_t cols_padded, int tile_elements, int32_t* error_dev, void* stream) {
  using namespace ep;
  if (offsets_dev == nullptr || states_dev == nullptr || scales_dev == nullptr || tables_dev == nullptr ||
      desc == nullptr || out_dev == nullptr || error_dev == nullptr) return EP_HIP_EINVAL;
  if (payload_dev == nullptr && payload_words != 0) return EP_HIP_EINVAL;
  if (rows <= 0 || cols_padded <= 0 || cols_padded % 8 != 0 || tile_elements <= 0) return EP_HIP_EINVAL;
  if (store_kind < EP_STORE_F32 || store_kind > EP_STORE_BF16) return EP_HIP_EINVAL;
  if (desc->prob_bits < 9 || desc->prob_bits > 15) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(payload_dev) % 4 != 0 || reinterpret_cast<uintptr_t>(out_dev) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(tables_dev) % 256 != 0) return EP_HIP_EINVAL;
  if (payload_words > 0xFFFFFFFFull) return EP_HIP_EINVAL;           // offsets are 32-bit
  const int64_t vecs_per_row = cols_padded / 8;
  if (vecs_per_row > 0x7FFFFFFF) return EP_HIP_EINVAL;
  const int64_t vectors = rows * vecs_per_row;
  const int tv = tile_vectors_of(tile_elements);
  const int64_t tiles = (vectors + tv - 1) / tv;
  if (vectors >= (int64_t{1} << 31) || tiles >= (int64_t{1} << 30)) return EP_HIP_EUNSUPPORTED;

  DecodeArgs args;
  args.payload = payload_dev;
  args.payload_words = payload_words;
  args.offsets = offsets_dev;
  args.states = states_dev;
  args.scales = scales_dev;
  args.plan = static_cast<const uint32_t*>(tables_dev);
  args.out = out_dev;
  args.store_kind = store_kind;
  args.vecs_per_row = static_cast<int>(vecs_per_row);
  args.num_vectors = vectors;
  args.tile_vectors = tv;
  args.num_tiles = static_cast<int>(tiles);
  args.error = error_dev;
  args.lut_bytes = args.rank_val_offset = args.rank_rs_offset = 0;
  // row = floor(v / d) for v < 2^31 as umulhi(v, ceil(2^p / d)) >> (p - 32), p = 31 + ceil(log2 d), d >= 2.
  // d == 1 is handled as floor(2 v / 2): umulhi(2 v, 2^31) is exact for every 32-bit 2 v.
  {
    const int64_t divisor = vecs_per_row > 1 ? vecs_per_row : 2;
    int log2_ceil = 0;
    while ((int64_t{1} << log2_ceil) < divisor) ++log2_ceil;
    const int p = 31 + log2_ceil;
    const unsigned __int128 power = static_cast<unsigned __int128>(1) << p;
    args.row_magic = static_cast<uint32_t>((power + divisor - 1) / divisor);
    args.row_shift = p - 32;
    args.row_pre = vecs_per_row > 1 ? 0 : 1;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int pairs = static_cast<int>((tiles + 1) / 2);

  if (desc->table_kind == EP_TABLE_GLOBAL64) {
    const int waves_per_block = 4;
    const int blocks = (pairs + waves_per_block - 1) / waves_per_block;
    hipLaunchKernelGGL(decode_global64_kernel, dim3(blocks), dim3(waves_per_block * 64), 0, s, args);
    EP_HIP_TRY(hipGetLastError());
    return EP_HIP_OK;
  }
  if (desc->table_kind == EP_TABLE_LDS_RANK) {
    const int present = desc->present_offset[kStreams];
    if (present < 0 || present > 65535 || desc->lds_bytes != static_cast<int>(rank_table_bytes(present, desc->prob_bits))) return EP_HIP_EINVAL;
    args.lut_bytes = static_cast<uint32_t>(desc->lds_bytes);
    args.rank_val_offset = static_cast<uint32_t>(rank_fb_bytes(present));
    args.rank_rs_offset = static_cast<uint32_t>(rank_rs_offset(present, desc->prob_bits));
    return launch_lds_decode(args, *desc, pairs, s);
  }
  if (desc->table_kind != EP_TABLE_LDS_BYTE && desc->table_kind != EP_TABLE_LDS_WIDE) return EP_HIP_EINVAL;
  if (desc->prob_bits > 11) return EP_HIP_EINVAL;

  return launch_lds_decode(args, *desc, pairs, s);
}
