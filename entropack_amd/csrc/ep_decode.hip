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
#include <hip/hip_fp16.h>
#include <string.h>

#include <mutex>

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

namespace ep {

// Validates one container's arguments and fills the kernels' argument block. `pairs` = wave-sized tile pairs.
static int fill_decode_args(const uint16_t* payload_dev, uint64_t payload_words, const uint32_t* offsets_dev,
                            const uint32_t* states_dev, const float* scales_dev, const void* tables_dev,
                            const ep_hip_plan_desc* desc, void* out_dev, int store_kind, int64_t rows, int64_t cols_padded,
                            int tile_elements, int32_t* error_dev, DecodeArgs& args, int& pairs) {
  if (offsets_dev == nullptr || states_dev == nullptr || scales_dev == nullptr || tables_dev == nullptr ||
      desc == nullptr || error_dev == nullptr) return EP_HIP_EINVAL;
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
  args.lut_bytes = args.rank_val_offset = args.rank_rs_offset = args.rank_half = 0;
  args.sym_tables = nullptr;
  args.store_cached = 0;
  args.reserved = 0;
  args.m_rows = 0;
  args.x = nullptr;
  args.y32 = nullptr;
  args.ldx = args.ldy32 = 0;
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
  pairs = static_cast<int>((tiles + 1) / 2);

  // The LDS-table kernels address a pair of tiles with 32-bit byte offsets (16 bytes per vector) and count a tile's
  // window slides (one per 64 payload words, at most nine words per vector) in 16 bits.
  if (desc->table_kind != EP_TABLE_GLOBAL64 && tv > kMaxLdsTileVectors) return EP_HIP_EUNSUPPORTED;
  switch (desc->table_kind) {
    case EP_TABLE_GLOBAL64:
      return EP_HIP_OK;
    case EP_TABLE_LDS_RANK: {
      const int present = desc->present_offset[kStreams];
      if (present < 0 || present > 65535 || desc->lds_bytes != static_cast<int>(rank_table_bytes(present, desc->prob_bits))) return EP_HIP_EINVAL;
      args.lut_bytes = static_cast<uint32_t>(desc->lds_bytes);
      args.rank_val_offset = static_cast<uint32_t>(rank_fb_bytes(present));
      args.rank_rs_offset = static_cast<uint32_t>(rank_rs_offset(present, desc->prob_bits));
      if (desc->rank_values_half != 0 && desc->prob_bits > 14) return EP_HIP_EINVAL;
      args.rank_half = desc->rank_values_half != 0;
      return EP_HIP_OK;
    }
    case EP_TABLE_LDS_SYM:
      if (desc->sym_offset == 0) return EP_HIP_EINVAL;
      [[fallthrough]];
    case EP_TABLE_LDS_BYTE:
    case EP_TABLE_LDS_WIDE:
      if (desc->prob_bits > 11 || desc->sym_offset < 0) return EP_HIP_EINVAL;
      if (desc->sym_offset != 0) args.sym_tables = static_cast<const uint8_t*>(tables_dev) + desc->sym_offset;
      return EP_HIP_OK;
    default:
      return EP_HIP_EINVAL;
  }
}

static int launch_global64(const DecodeArgs& args, int pairs, hipStream_t s) {
  const int waves_per_block = 4;
  const int blocks = (pairs + waves_per_block - 1) / waves_per_block;
  hipLaunchKernelGGL(decode_global64_kernel, dim3(blocks), dim3(waves_per_block * 64), 0, s, args);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

// ---- batch plan: a position-independent blob, identical on host and device -------------------------------------------

constexpr uint32_t kBatchMagic = 0x45504254u;
constexpr int kBatchMaxLaunches = 64;       // (table kind, prob_bits, bf16 or not) combinations, far below this in practice

struct BatchLaunch {
  LdsLaunch cfg;            // cfg.blocks = number of block jobs; for GLOBAL64: cfg.blocks = job index
  int first_block;
  int pairs;                // GLOBAL64 only
};

struct BatchHeader {
  uint32_t magic;
  int n_jobs;
  int n_launches;
  int n_blocks;
  uint64_t args_offset;     // DecodeArgs[n_jobs]; `out` holds the byte offset into the arena
  uint64_t blocks_offset;   // BlockJob[n_blocks]
  uint64_t total_bytes;
  BatchLaunch launches[kBatchMaxLaunches];
};

static size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace ep

extern "C" int ep_hip_decode_lattice(const uint16_t* payload_dev, uint64_t payload_words, const uint32_t* offsets_dev,
                                     const uint32_t* states_dev, const float* scales_dev, const void* tables_dev,
                                     const ep_hip_plan_desc* desc, void* out_dev, int store_kind, int64_t rows,
                                     int64_t cols_padded, int tile_elements, int32_t* error_dev, void* stream) {
  using namespace ep;
  if (out_dev == nullptr) return EP_HIP_EINVAL;
  DecodeArgs args;
  int pairs = 0;
  const int status = fill_decode_args(payload_dev, payload_words, offsets_dev, states_dev, scales_dev, tables_dev, desc, out_dev,
                                      store_kind, rows, cols_padded, tile_elements, error_dev, args, pairs);
  if (status != EP_HIP_OK) return status;
  // Memory takes writes in pieces of 64 bytes = four bf16 vectors, and a group writes 32 consecutive vectors from the tile's
  // first vector + a multiple of 32. When the tile length is no multiple of four vectors (the default tiles from 5 bpp up:
  // 910 and 455 vectors), the piece at either end of a group is shared with the neighbouring group, which streams its part
  // out microseconds apart; written through the cache the two parts meet in L2. With the container read from memory (a
  // layer decoded once per forward) that is 7-8 % faster at 5, 6 and 8 bpp (8192 x 28672: 176 -> 161, 183 -> 168, 215 ->
  // 200 us); whole tiles keep the streaming stores, which are the faster ones there (156 against 161 us at 4 bpp), and so
  // do batches, where layers of both kinds share a launch (the 120-layer pass measured 2 % slower with mixed policies).
  args.store_cached = store_kind == EP_STORE_BF16 && args.tile_vectors % 4 != 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (desc->table_kind == EP_TABLE_GLOBAL64) return launch_global64(args, pairs, s);
  return launch_lds_decode(args, *desc, kernel_kind_of(store_kind), pairs, s);
}

extern "C" int ep_hip_decode_table_kind(const ep_hip_plan_desc* desc, int store_kind, int64_t rows, int64_t cols_padded, int tile_elements,
                                        int compute_units) {
  using namespace ep;
  if (desc == nullptr || rows <= 0 || cols_padded <= 0 || tile_elements <= 0 || compute_units <= 0) return -1;
  const int64_t vectors = rows * (cols_padded / 8);
  const int tv = tile_vectors_of(tile_elements);
  const int64_t pairs = ((vectors + tv - 1) / tv + 1) / 2;
  return effective_table_kind(*desc, kernel_kind_of(store_kind), pairs, compute_units);
}

extern "C" int ep_hip_batch_plan(const ep_hip_decode_job* jobs, int n_jobs, int compute_units, void* blob_host, size_t* blob_bytes) {
  using namespace ep;
  if (jobs == nullptr || n_jobs <= 0 || blob_bytes == nullptr || compute_units <= 0) return EP_HIP_EINVAL;

  struct Group { int table_kind, prob_bits, kind, lut_bytes; int64_t pairs; };
  Group groups[kBatchMaxLaunches];
  int n_groups = 0;
  auto group_of = [&](const ep_hip_plan_desc& d, int store_kind) {
    const int kind = kernel_kind_of(store_kind);
    const int tables = effective_table_kind(d, kind, int64_t{1} << 40, compute_units);     // a batch is always a large launch
    for (int g = 0; g < n_groups; ++g) {
      if (groups[g].table_kind == tables && groups[g].prob_bits == d.prob_bits && groups[g].kind == kind) return g;
    }
    return -1;
  };

  // Pass 1: validate every job, count GLOBAL64 jobs (one launch each) and the pairs of each LDS group.
  int n_global = 0;
  for (int i = 0; i < n_jobs; ++i) {
    const ep_hip_decode_job& j = jobs[i];
    if (j.out_offset % 16 != 0) return EP_HIP_EINVAL;
    DecodeArgs args;
    int pairs = 0;
    const int status = fill_decode_args(j.payload_dev, j.payload_words, j.offsets_dev, j.states_dev, j.scales_dev, j.tables_dev, j.desc,
                                        nullptr, j.store_kind, j.rows, j.cols_padded, j.tile_elements, j.error_dev, args, pairs);
    if (status != EP_HIP_OK) return status;
    if (j.desc->table_kind == EP_TABLE_GLOBAL64) {
      ++n_global;
      continue;
    }
    int g = group_of(*j.desc, j.store_kind);
    if (g < 0) {
      if (n_groups == kBatchMaxLaunches) return EP_HIP_EUNSUPPORTED;
      g = n_groups++;
      const int kind = kernel_kind_of(j.store_kind);
      groups[g] = {effective_table_kind(*j.desc, kind, int64_t{1} << 40, compute_units), j.desc->prob_bits, kind, 0, 0};
    }
    groups[g].pairs += pairs;
    if (j.desc->lds_bytes > groups[g].lut_bytes) groups[g].lut_bytes = j.desc->lds_bytes;
  }
  if (n_groups + n_global > kBatchMaxLaunches) return EP_HIP_EUNSUPPORTED;

  // Slice size per group: full blocks (16 waves x ilp pairs per round), about eight slices per resident block so the
  // tail of the launch stays short whatever the mix of tile lengths.
  LdsLaunch cfgs[kBatchMaxLaunches];
  int slice[kBatchMaxLaunches];
  for (int g = 0; g < n_groups; ++g) {
    const int big = groups[g].pairs > 0x7FFFFFFF ? 0x7FFFFFFF : static_cast<int>(groups[g].pairs);
    cfgs[g] = choose_lds_launch(groups[g].table_kind, groups[g].prob_bits, groups[g].lut_bytes, groups[g].kind, big, compute_units);
    const int per_round = (cfgs[g].threads / 64) * cfgs[g].ilp;
    const int resident = lds_resident_blocks(groups[g].table_kind, groups[g].prob_bits, groups[g].lut_bytes) * compute_units;
    int64_t rounds = groups[g].pairs / (static_cast<int64_t>(per_round) * resident * 8);
    rounds = rounds < 1 ? 1 : (rounds > 64 ? 64 : rounds);
    slice[g] = per_round * static_cast<int>(rounds);
  }

  // Pass 2: count (sizing) or emit block jobs.
  int64_t n_blocks = 0;
  for (int i = 0; i < n_jobs; ++i) {
    const ep_hip_decode_job& j = jobs[i];
    if (j.desc->table_kind == EP_TABLE_GLOBAL64) continue;
    const int g = group_of(*j.desc, j.store_kind);
    const int64_t vectors = j.rows * (j.cols_padded / 8);
    const int tv = tile_vectors_of(j.tile_elements);
    const int64_t pairs = ((vectors + tv - 1) / tv + 1) / 2;
    n_blocks += (pairs + slice[g] - 1) / slice[g];
  }
  if (n_blocks > 0x7FFFFFFF) return EP_HIP_EUNSUPPORTED;
  const size_t args_offset = align_up(sizeof(BatchHeader), 256);
  const size_t blocks_offset = align_up(args_offset + sizeof(DecodeArgs) * static_cast<size_t>(n_jobs), 256);
  const size_t total = align_up(blocks_offset + sizeof(BlockJob) * static_cast<size_t>(n_blocks > 0 ? n_blocks : 1), 256);
  if (blob_host == nullptr) {
    *blob_bytes = total;
    return EP_HIP_OK;
  }
  if (*blob_bytes < total) return EP_HIP_EINVAL;

  memset(blob_host, 0, total);
  BatchHeader* header = static_cast<BatchHeader*>(blob_host);
  DecodeArgs* args_out = reinterpret_cast<DecodeArgs*>(static_cast<uint8_t*>(blob_host) + args_offset);
  BlockJob* blocks_out = reinterpret_cast<BlockJob*>(static_cast<uint8_t*>(blob_host) + blocks_offset);
  header->magic = kBatchMagic;
  header->n_jobs = n_jobs;
  header->n_blocks = static_cast<int>(n_blocks);
  header->args_offset = args_offset;
  header->blocks_offset = blocks_offset;
  header->total_bytes = total;
  for (int i = 0; i < n_jobs; ++i) {
    const ep_hip_decode_job& j = jobs[i];
    int pairs = 0;
    fill_decode_args(j.payload_dev, j.payload_words, j.offsets_dev, j.states_dev, j.scales_dev, j.tables_dev, j.desc, nullptr,
                     j.store_kind, j.rows, j.cols_padded, j.tile_elements, j.error_dev, args_out[i], pairs);
    args_out[i].out = reinterpret_cast<void*>(static_cast<uintptr_t>(j.out_offset));
  }
  int n_launches = 0, cursor = 0;
  for (int g = 0; g < n_groups; ++g) {       // block jobs grouped by launch, containers in caller order inside a group
    BatchLaunch& launch = header->launches[n_launches++];
    launch.cfg = cfgs[g];
    launch.first_block = cursor;
    for (int i = 0; i < n_jobs; ++i) {
      const ep_hip_decode_job& j = jobs[i];
      if (j.desc->table_kind == EP_TABLE_GLOBAL64 || group_of(*j.desc, j.store_kind) != g) continue;
      const int pairs = (args_out[i].num_tiles + 1) / 2;
      for (int first = 0; first < pairs; first += slice[g]) {
        BlockJob& b = blocks_out[cursor++];
        b.job = i;
        b.first_pair = first;
        b.n_pairs = pairs - first < slice[g] ? pairs - first : slice[g];
      }
    }
    launch.cfg.blocks = cursor - launch.first_block;      // threads and LDS stay as chosen for the group's total
  }
  for (int i = 0; i < n_jobs; ++i) {
    if (jobs[i].desc->table_kind != EP_TABLE_GLOBAL64) continue;
    BatchLaunch& launch = header->launches[n_launches++];
    launch.cfg.table_kind = EP_TABLE_GLOBAL64;
    launch.cfg.blocks = i;
    launch.pairs = (args_out[i].num_tiles + 1) / 2;
  }
  header->n_launches = n_launches;
  *blob_bytes = total;
  return EP_HIP_OK;
}

extern "C" int ep_hip_decode_lattice_batch(const void* blob_host, const void* blob_dev, void* out_arena_dev, void* stream) {
  using namespace ep;
  if (blob_host == nullptr || blob_dev == nullptr || out_arena_dev == nullptr) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(out_arena_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(blob_dev) % 256 != 0) return EP_HIP_EINVAL;
  const BatchHeader* header = static_cast<const BatchHeader*>(blob_host);
  if (header->magic != kBatchMagic || header->n_launches < 0 || header->n_launches > kBatchMaxLaunches) return EP_HIP_EINVAL;
  const DecodeArgs* args_host = reinterpret_cast<const DecodeArgs*>(static_cast<const uint8_t*>(blob_host) + header->args_offset);
  const DecodeArgs* args_dev = reinterpret_cast<const DecodeArgs*>(static_cast<const uint8_t*>(blob_dev) + header->args_offset);
  const BlockJob* blocks_dev = reinterpret_cast<const BlockJob*>(static_cast<const uint8_t*>(blob_dev) + header->blocks_offset);
  uint8_t* arena = static_cast<uint8_t*>(out_arena_dev);
  hipStream_t s = static_cast<hipStream_t>(stream);
  for (int l = 0; l < header->n_launches; ++l) {
    const BatchLaunch& launch = header->launches[l];
    if (launch.cfg.table_kind == EP_TABLE_GLOBAL64) {
      DecodeArgs args = args_host[launch.cfg.blocks];
      args.out = arena + reinterpret_cast<uintptr_t>(args.out);
      const int status = launch_global64(args, launch.pairs, s);
      if (status != EP_HIP_OK) return status;
      continue;
    }
    if (launch.cfg.blocks == 0) continue;
    const int status = launch_lds(launch.cfg, args_host[0], 0, args_dev, blocks_dev + launch.first_block, arena, s);
    if (status != EP_HIP_OK) return status;
  }
  return EP_HIP_OK;
}

// ---- fused linear for a few activation rows ----------------------------------------------------------------------------

namespace ep {

__global__ __launch_bounds__(256) void zero_f32_kernel(float* __restrict__ p, int64_t count) {
  for (int64_t i = blockIdx.x * int64_t{256} + threadIdx.x; i < count; i += gridDim.x * int64_t{256}) p[i] = 0.0f;
}

// y[m][n] = cast(y32[m][n] + bias[n]); bias has the output's type.
__global__ __launch_bounds__(256) void finish_linear_kernel(const float* __restrict__ y32, const void* __restrict__ bias, void* __restrict__ y,
                                                            int rows, int64_t outer, int64_t ldy, int out_kind) {
  const int64_t n = blockIdx.x * int64_t{256} + threadIdx.x;
  if (n >= outer) return;
  float add = 0.0f;
  if (bias != nullptr) {
    if (out_kind == EP_FLOAT_BF16) add = __uint_as_float(static_cast<uint32_t>(static_cast<const uint16_t*>(bias)[n]) << 16);
    else if (out_kind == EP_FLOAT_F16) add = __half2float(static_cast<const __half*>(bias)[n]);
    else add = static_cast<const float*>(bias)[n];
  }
  for (int m = 0; m < rows; ++m) {
    const float v = __fadd_rn(y32[m * outer + n], add);
    if (out_kind == EP_FLOAT_BF16) static_cast<uint16_t*>(y)[m * ldy + n] = static_cast<uint16_t>(bf16_bits_rne(v));
    else if (out_kind == EP_FLOAT_F16) static_cast<__half*>(y)[m * ldy + n] = __float2half_rn(v);
    else static_cast<float*>(y)[m * ldy + n] = v;
  }
}

}  // namespace ep

namespace ep {

// Decode-and-multiply for one to four activation rows with the f32 accumulator `y32` given by the caller.
static int linear_fused_bf16(const ep_hip_decode_job* weight, const void* x_dev, int64_t m_rows, int64_t ldx, const void* bias_dev,
                             void* y_dev, int64_t ldy, int out_kind, float* y32, hipStream_t s) {
  const int64_t outer = weight->rows, inner = weight->cols_padded;
  if (ldx < inner || ldy < outer || reinterpret_cast<uintptr_t>(x_dev) % 16 != 0 || ldx % 8 != 0) return EP_HIP_EINVAL;
  // The kernels carry at most four activation rows in registers, need whole weight rows of at least 32 vectors (a
  // group of 32 vectors then touches at most two rows), bf16 weights, and an LDS-table plan.
  if (m_rows > 4 || inner < 256 || weight->store_kind != EP_STORE_BF16 || weight->desc->table_kind == EP_TABLE_GLOBAL64) return EP_HIP_EUNSUPPORTED;
  DecodeArgs args;
  int pairs = 0;
  const int status = fill_decode_args(weight->payload_dev, weight->payload_words, weight->offsets_dev, weight->states_dev, weight->scales_dev,
                                      weight->tables_dev, weight->desc, nullptr, weight->store_kind, weight->rows, weight->cols_padded,
                                      weight->tile_elements, weight->error_dev, args, pairs);
  if (status != EP_HIP_OK) return status;
  args.m_rows = static_cast<int>(m_rows);
  args.x = static_cast<const uint16_t*>(x_dev);
  args.ldx = ldx;
  args.y32 = y32;
  args.ldy32 = outer;
  const int64_t cells = m_rows * outer;
  // The accumulator is cleared by a kernel, never a memset node: the sequence may be captured into a graph.
  hipLaunchKernelGGL(zero_f32_kernel, dim3(static_cast<unsigned>((cells + 255) / 256 < 1024 ? (cells + 255) / 256 : 1024)), dim3(256), 0, s,
                     y32, cells);
  EP_HIP_TRY(hipGetLastError());
  const int launched = launch_lds_decode(args, *weight->desc, m_rows == 1 ? -2 : -3, pairs, s);
  if (launched != EP_HIP_OK) return launched;
  hipLaunchKernelGGL(finish_linear_kernel, dim3(static_cast<unsigned>((outer + 255) / 256)), dim3(256), 0, s, y32, bias_dev, y_dev,
                     static_cast<int>(m_rows), outer, ldy, out_kind);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

// The accumulator of ep_hip_linear_fused_bf16_static: one copy per GPU, held until the process ends. In host code the
// array's name is only a handle; its device address comes from hipGetSymbolAddress, once per device: by
// ep_hip_device_query for the device that is current then (the library's set-up call, outside any stream capture), else by
// the entry point's first call on the device.
static __device__ __align__(256) float scratch[EP_HIP_STATIC_ACCUMULATOR_FLOATS];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_lock;
static float* g_scratch_of_device[kMaxDevices];      // device ordinal -> address of that device's `scratch`

int static_accumulator(float** address) {
  int device = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return EP_HIP_EUNSUPPORTED;
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (g_scratch_of_device[device] == nullptr) {
    float* found = nullptr;
    EP_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void**>(&found), HIP_SYMBOL(scratch)));
    if (found == nullptr) return EP_HIP_ERUNTIME;
    g_scratch_of_device[device] = found;
  }
  *address = g_scratch_of_device[device];
  return EP_HIP_OK;
}

}  // namespace ep

extern "C" int ep_hip_linear_fused_bf16(const ep_hip_decode_job* weight, const void* x_dev, int64_t m_rows, int64_t ldx,
                                        const void* bias_dev, void* y_dev, int64_t ldy, int out_kind, float* workspace_dev,
                                        void* stream) {
  using namespace ep;
  if (weight == nullptr || x_dev == nullptr || y_dev == nullptr || workspace_dev == nullptr) return EP_HIP_EINVAL;
  if (out_kind < EP_FLOAT_BF16 || out_kind > EP_FLOAT_F32 || m_rows <= 0) return EP_HIP_EINVAL;
  if (weight->desc == nullptr) return EP_HIP_EINVAL;
  return linear_fused_bf16(weight, x_dev, m_rows, ldx, bias_dev, y_dev, ldy, out_kind, workspace_dev, static_cast<hipStream_t>(stream));
}

extern "C" int ep_hip_linear_fused_bf16_static(const ep_hip_decode_job* weight, const void* x_dev, int64_t m_rows, int64_t ldx,
                                               const void* bias_dev, void* y_dev, int64_t ldy, int out_kind, void* stream) {
  using namespace ep;
  if (weight == nullptr || x_dev == nullptr || y_dev == nullptr) return EP_HIP_EINVAL;
  if (out_kind < EP_FLOAT_BF16 || out_kind > EP_FLOAT_F32 || m_rows <= 0) return EP_HIP_EINVAL;
  if (weight->desc == nullptr || weight->rows <= 0) return EP_HIP_EINVAL;
  if (m_rows > 4) return EP_HIP_EUNSUPPORTED;
  if (m_rows * weight->rows > EP_HIP_STATIC_ACCUMULATOR_FLOATS) return EP_HIP_ETOOLARGE;
  float* accumulator = nullptr;
  const int status = static_accumulator(&accumulator);
  if (status != EP_HIP_OK) return status;
  return linear_fused_bf16(weight, x_dev, m_rows, ldx, bias_dev, y_dev, ldy, out_kind, accumulator, static_cast<hipStream_t>(stream));
}

namespace ep {

// Shared by the two decode-to-GEMM entry points: argument checks, the kernels' argument block, the launch.
static int linear_fused_mfma(const ep_hip_decode_job* weight, const ep_hip_fused_batch* batches_dev, int n_batches, bool int8, const void* x_dev,
                             int64_t m_rows, int64_t ldx, const float* scale_a_dev, const float* scale_b_dev, const void* bias_dev, void* y_dev,
                             int64_t ldy, int out_kind, void* workspace_dev, hipStream_t stream) {
  if (weight == nullptr || batches_dev == nullptr || x_dev == nullptr || y_dev == nullptr || workspace_dev == nullptr) return EP_HIP_EINVAL;
  if (out_kind < EP_FLOAT_BF16 || out_kind > EP_FLOAT_F32 || m_rows <= 0 || n_batches <= 0 || weight->desc == nullptr) return EP_HIP_EINVAL;
  if (int8 && (scale_a_dev == nullptr || scale_b_dev == nullptr)) return EP_HIP_EINVAL;
  const int64_t outer = weight->rows, inner = weight->cols_padded;
  if (ldx < inner || ldy < outer || reinterpret_cast<uintptr_t>(x_dev) % 16 != 0 || ldx % (int8 ? 16 : 8) != 0) return EP_HIP_EINVAL;
  if (m_rows > 0x7FFFFFFF || weight->store_kind != (int8 ? EP_STORE_I8 : EP_STORE_BF16) || weight->desc->table_kind == EP_TABLE_GLOBAL64) {
    return EP_HIP_EUNSUPPORTED;
  }
  DecodeArgs args;
  int pairs = 0;
  const int status = fill_decode_args(weight->payload_dev, weight->payload_words, weight->offsets_dev, weight->states_dev, weight->scales_dev,
                                      weight->tables_dev, weight->desc, nullptr, weight->store_kind, weight->rows, weight->cols_padded,
                                      weight->tile_elements, weight->error_dev, args, pairs);
  if (status != EP_HIP_OK) return status;
  // The kernel takes nothing in the batch table on trust (tile indices, shifts and bases are range-checked there), so a
  // stale table yields an error code or wrong sums, never an access outside the buffers.
  if (n_batches > args.num_tiles || reinterpret_cast<uintptr_t>(workspace_dev) % 256 != 0) return EP_HIP_EINVAL;
  args.m_rows = static_cast<int>(m_rows);
  args.x = static_cast<const uint16_t*>(x_dev);
  args.ldx = ldx;
  args.y32 = static_cast<float*>(workspace_dev);
  return launch_fused_mfma(args, *weight->desc, batches_dev, n_batches, int8, scale_a_dev, scale_b_dev, bias_dev, y_dev, ldy, out_kind, stream);
}

}  // namespace ep

extern "C" int ep_hip_linear_fused_mfma_bf16(const ep_hip_decode_job* weight, const ep_hip_fused_batch* batches_dev, int n_batches,
                                             const void* x_dev, int64_t m_rows, int64_t ldx, const void* bias_dev, void* y_dev,
                                             int64_t ldy, int out_kind, void* workspace_dev, void* stream) {
  return ep::linear_fused_mfma(weight, batches_dev, n_batches, false, x_dev, m_rows, ldx, nullptr, nullptr, bias_dev, y_dev, ldy, out_kind,
                               workspace_dev, static_cast<hipStream_t>(stream));
}

extern "C" int ep_hip_linear_fused_mfma_i8(const ep_hip_decode_job* weight, const ep_hip_fused_batch* batches_dev, int n_batches,
                                           const int8_t* a_dev, int64_t m_rows, int64_t lda, const float* scale_a_dev, const float* scale_b_dev,
                                           const void* bias_dev, void* y_dev, int64_t ldy, int out_kind, void* workspace_dev, void* stream) {
  return ep::linear_fused_mfma(weight, batches_dev, n_batches, true, a_dev, m_rows, lda, scale_a_dev, scale_b_dev, bias_dev, y_dev, ldy, out_kind,
                               workspace_dev, static_cast<hipStream_t>(stream));
}

extern "C" size_t ep_hip_linear_fused_mfma_workspace(int64_t rows, int64_t cols_padded, int tile_elements, int64_t m_rows, int int8) {
  if (rows <= 0 || cols_padded < 8 || tile_elements <= 0 || m_rows <= 0) return 0;
  return ep::fused_workspace_bytes(rows, cols_padded, tile_elements, m_rows, int8 ? 1 : 2);
}
