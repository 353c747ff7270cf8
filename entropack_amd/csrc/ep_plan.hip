// Library bookkeeping, device query, and the decode plan: choosing a table representation on the host and
// building the slot tables on the device.
#include <string.h>

#include "ep_common.hpp"

namespace ep {

static thread_local int g_last_runtime_error = 0;

void set_runtime_error(hipError_t e) { g_last_runtime_error = static_cast<int>(e); }

__global__ __launch_bounds__(256) void zero_fill_kernel(uint4* __restrict__ p, size_t quads) {
  for (size_t i = blockIdx.x * size_t{256} + threadIdx.x; i < quads; i += gridDim.x * size_t{256}) p[i] = make_uint4(0, 0, 0, 0);
}

// The table builders run one block of 256 threads per stream. Threads split the alphabet into contiguous chunks and
// scan the chunk sums, which gives every symbol its cumulative frequency; the slots are then filled slot by slot (thread
// t takes slots t, t + 256, ...), each finding its symbol by bisection of the cumulative frequencies kept in LDS, so the
// work is even however skewed the frequencies are. (Filling symbol by symbol left one thread writing the hundreds of
// slots of the likeliest symbol while the others idled: 55 us per container against 6 us.)
constexpr int kScanThreads = 256;
constexpr int kCdfInLds = 4096;          // alphabets up to this size keep their cumulative frequencies in LDS

// Exclusive prefix sums of one value per thread over the block, in place in `values` (256 entries of LDS).
__device__ __forceinline__ void block_exclusive_scan(uint32_t* values, int tid) {
  __syncthreads();
  const uint32_t own = values[tid];
  uint32_t sum = own;
  for (int step = 1; step < kScanThreads; step <<= 1) {
    const uint32_t below = tid >= step ? values[tid - step] : 0u;
    __syncthreads();
    sum += below;
    values[tid] = sum;
    __syncthreads();
  }
  values[tid] = sum - own;
  __syncthreads();
}

// Symbol of `slot`: the last symbol whose cumulative frequency is at most `slot`; cdf[0 .. alphabet] ascending, cdf[0] = 0,
// cdf[alphabet] = table size. Symbols of frequency zero share their neighbour's value and are never the answer.
__device__ __forceinline__ int symbol_of_slot(const uint32_t* cdf, int alphabet, uint32_t slot) {
  int low = 0, high = alphabet;          // cdf[low] <= slot < cdf[high]
  while (high - low > 1) {
    const int mid = (low + high) >> 1;
    if (cdf[mid] <= slot) low = mid; else high = mid;
  }
  return low;
}

// LDS_SYM section of a byte-valued plan: one block per field stream.
__global__ __launch_bounds__(256) void build_sym_tables_kernel(const int32_t* __restrict__ meta, const uint16_t* __restrict__ freq_tables,
                                                               int prob_bits, uint8_t* __restrict__ section) {
  __shared__ uint32_t chunk_sum[kScanThreads];
  __shared__ uint32_t cdf[256 + 1];
  const int stream = blockIdx.x + 1;
  const int tid = threadIdx.x;
  const uint32_t size = 1u << prob_bits;
  const int sym_min = meta[stream * kMetaWidth + 1];
  const int freq_off = meta[stream * kMetaWidth + 2];
  const int alphabet = meta[stream * kMetaWidth + 3];
  if (alphabet <= 0 || alphabet > 256) return;            // byte-valued plans have alphabets of at most 256 symbols
  const uint16_t* freq = freq_tables + freq_off;
  const uint32_t f = tid < alphabet ? freq[tid] : 0u;     // one symbol per thread
  chunk_sum[tid] = f;
  block_exclusive_scan(chunk_sum, tid);
  const uint32_t begin = chunk_sum[tid];
  if (tid < alphabet) cdf[tid] = begin;
  if (tid == 0) cdf[alphabet] = size;
  // The decode step forms slot | (2048 * coset), reads the slot table there, and subtracts the low half of the second
  // word from freq * (x >> pb) + that, so the coset offset is folded into the stored cdf.
  const uint32_t slot_table_at = static_cast<uint32_t>(kSymFbBytes) + static_cast<uint32_t>(stream - 1) * kSymSlotStreamBytes;
  const uint32_t folded = (static_cast<uint32_t>(stream - 1) & 1u) * kSymSlotStreamBytes;
  uint2* fb = reinterpret_cast<uint2*>(section) + (stream - 1) * 256;
  uint8_t* slots = section + slot_table_at;
  if (tid < alphabet && f != 0) {
    // The half-precision value is the lattice coordinate itself, coset shift included: z + c / 2, and for the last field,
    // whose z7 = 2 m + parity the kernel forms with one multiply-add, m + c / 4. |z| <= 128, so quarters are exact.
    const int z = tid + sym_min;
    const int coset = (stream - 1) & 1, field = (stream - 1) >> 1;
    const float coordinate = static_cast<float>(z) + (field == kFields - 1 ? 0.25f : 0.5f) * static_cast<float>(coset);
    const uint32_t z_half = __builtin_bit_cast(uint16_t, static_cast<_Float16>(coordinate));
    fb[z + 128] = make_uint2(f | ((z & 1) ? 0x3C000000u : 0u), (begin + folded) | (z_half << 16));
  }
  __syncthreads();
  for (uint32_t slot = tid; slot < size; slot += kScanThreads) {
    slots[slot] = static_cast<uint8_t>(symbol_of_slot(cdf, alphabet, slot) + sym_min + 128);
  }
}

struct RankLayout {
  int present_offset[18];
  uint32_t val_offset;     // byte offsets inside the table area
  uint32_t rs_offset;
  int values_half;         // values as half-precision coordinates (coset shift included) instead of 16-bit integers
};

__global__ __launch_bounds__(256) void build_tables_kernel(const int32_t* __restrict__ meta,
                                                           const uint16_t* __restrict__ freq_tables, int kind,
                                                           int prob_bits, uint32_t* __restrict__ plan, RankLayout rank) {
  __shared__ uint32_t chunk_sum[kScanThreads];
  __shared__ uint32_t chunk_present[kScanThreads];
  __shared__ uint32_t cdf[kCdfInLds + 1];
  const int stream = blockIdx.x;
  const int tid = threadIdx.x;
  const uint32_t size = 1u << prob_bits;
  const int sym_min = meta[stream * kMetaWidth + 1];
  const int freq_off = meta[stream * kMetaWidth + 2];
  const int alphabet = meta[stream * kMetaWidth + 3];

  if (tid == 0) {
    plan[kHdrSymMin + stream] = static_cast<uint32_t>(sym_min);
    plan[kHdrAlphabet + stream] = static_cast<uint32_t>(alphabet);
    if (stream == 0) {
      plan[kHdrMagic] = kPlanMagic;
      plan[kHdrKind] = static_cast<uint32_t>(kind);
      plan[kHdrProbBits] = static_cast<uint32_t>(prob_bits);
      // Symbol-0 frequency of the coset stream; an empty coset stream cannot occur in a valid container.
      plan[kHdrCosetFreq0] = alphabet > 0 ? freq_tables[freq_off] : size;
    }
  }
  if (kind != EP_TABLE_GLOBAL64 && stream == 0) return;   // the coset stream is decoded in closed form
  if (alphabet <= 0) return;

  const uint16_t* freq = freq_tables + freq_off;
  const int per = (alphabet + kScanThreads - 1) / kScanThreads;
  const int first = tid * per;
  const int last = first + per < alphabet ? first + per : alphabet;
  uint32_t local = 0, local_present = 0;
  for (int s = first; s < last; ++s) {
    local += freq[s];
    local_present += freq[s] != 0;
  }
  chunk_sum[tid] = local;
  chunk_present[tid] = local_present;
  block_exclusive_scan(chunk_sum, tid);
  block_exclusive_scan(chunk_present, tid);
  uint32_t running = chunk_sum[tid];
  uint8_t* tables = reinterpret_cast<uint8_t*>(plan) + kHeaderBytes;
  if (kind == EP_TABLE_LDS_RANK) {
    // Symbol-end bitmap + running symbol count per 32 slots, and per present symbol cdf | freq << 16 | (value odd) << 31
    // and its value: a 16-bit integer, or the lattice coordinate in half precision (z + c / 2; m + c / 4 for the last
    // field, whose z7 = 2 m + parity the kernel forms with one multiply-add).
    uint32_t* fb = reinterpret_cast<uint32_t*>(tables);
    int16_t* val = reinterpret_cast<int16_t*>(tables + rank.val_offset);
    uint32_t* rs = reinterpret_cast<uint32_t*>(tables + rank.rs_offset) + (static_cast<size_t>(stream - 1) << prob_bits) / 32 * 2;
    uint32_t index = static_cast<uint32_t>(rank.present_offset[stream]) + chunk_present[tid];
    for (int s = first; s < last; ++s) {
      const uint32_t f = freq[s];
      if (f == 0) continue;
      const int z = s + sym_min;
      fb[index] = running | (f << 16) | (rank.values_half ? static_cast<uint32_t>(z & 1) << 31 : 0u);
      if (rank.values_half) {
        const int coset = (stream - 1) & 1, field = (stream - 1) >> 1;
        const float coordinate = static_cast<float>(z) + (field == kFields - 1 ? 0.25f : 0.5f) * static_cast<float>(coset);
        val[index] = __builtin_bit_cast(int16_t, static_cast<_Float16>(coordinate));
      } else {
        val[index] = static_cast<int16_t>(z);
      }
      const uint32_t end = running + f - 1;
      if (end < size) atomicOr(&rs[(end >> 5) * 2], 1u << (end & 31));
      running += f;
      ++index;
    }
    __threadfence_block();
    __syncthreads();
    // Symbols that end before each word: a scan of the words' bit counts, 256 words at a time.
    uint32_t carried = static_cast<uint32_t>(rank.present_offset[stream]);
    for (uint32_t base = 0; base < size / 32; base += kScanThreads) {
      const uint32_t w = base + static_cast<uint32_t>(tid);
      const uint32_t bits = w < size / 32 ? static_cast<uint32_t>(__popc(rs[w * 2])) : 0u;
      chunk_sum[tid] = bits;
      block_exclusive_scan(chunk_sum, tid);
      if (w < size / 32) rs[w * 2 + 1] = carried + chunk_sum[tid];
      const uint32_t total = chunk_sum[kScanThreads - 1] + __shfl(bits, 63);      // meaningful in the last wave only
      __syncthreads();
      if (tid == kScanThreads - 1) chunk_present[0] = total;
      __syncthreads();
      carried += chunk_present[0];
      __syncthreads();
    }
    return;
  }
  auto entry_of = [&](uint32_t slot, uint32_t s, uint32_t f, uint32_t d) {
    if (kind == EP_TABLE_GLOBAL64) {
      uint64_t* lut = reinterpret_cast<uint64_t*>(tables) + (static_cast<size_t>(stream) << prob_bits);
      lut[slot] = (static_cast<uint64_t>(d) << 32) | (static_cast<uint64_t>(f) << 16) | static_cast<uint64_t>(s);
    } else {
      uint32_t* lut = reinterpret_cast<uint32_t*>(tables) + (static_cast<size_t>(stream - 1) << prob_bits);
      if (kind == EP_TABLE_LDS_BYTE) {
        lut[slot] = f | (d << 12) | (static_cast<uint32_t>(static_cast<int>(s) + sym_min) << 24);     // top byte: the value, two's complement
      } else {
        lut[slot] = f | (d << 11) | (s << 22);
      }
    }
  };
  if (alphabet <= kCdfInLds) {
    for (int s = first; s < last; ++s) {
      cdf[s] = running;
      running += freq[s];
    }
    if (tid == 0) cdf[alphabet] = size;
    __syncthreads();
    for (uint32_t slot = tid; slot < size; slot += kScanThreads) {
      const uint32_t s = static_cast<uint32_t>(symbol_of_slot(cdf, alphabet, slot));
      entry_of(slot, s, cdf[s + 1] - cdf[s], slot - cdf[s]);
    }
    return;
  }
  for (int s = first; s < last; ++s) {      // very large alphabets (global tables only): symbol by symbol
    const uint32_t f = freq[s];
    for (uint32_t d = 0; d < f && running + d < size; ++d) entry_of(running + d, static_cast<uint32_t>(s), f, d);
    running += f;
  }
}

}  // namespace ep

extern "C" {

int ep_hip_abi_version(void) { return EP_HIP_ABI_VERSION; }

const char* ep_hip_error_string(int status) {
  switch (status) {
    case EP_HIP_OK: return "ok";
    case EP_HIP_EINVAL: return "invalid argument";
    case EP_HIP_EUNSUPPORTED: return "unsupported by this build";
    case EP_HIP_ERUNTIME: return "HIP runtime call failed";
    case EP_HIP_ENODEVICE: return "no gfx950 device";
    case EP_HIP_ETOOLARGE: return "request exceeds the library's fixed scratch buffer";
    default: return "unknown status";
  }
}

int ep_hip_last_runtime_error(void) { return ep::g_last_runtime_error; }

int ep_hip_device_query(int device, ep_hip_device_info* info) {
  if (info == nullptr) return EP_HIP_EINVAL;
  memset(info, 0, sizeof(*info));
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return EP_HIP_ENODEVICE;
  if (device < 0) EP_HIP_TRY(hipGetDevice(&device));
  if (device >= count) return EP_HIP_EINVAL;
  hipDeviceProp_t prop;
  EP_HIP_TRY(hipGetDeviceProperties(&prop, device));
  info->device = device;
  info->compute_units = prop.multiProcessorCount;
  info->wavefront_size = prop.warpSize;
  int lds = 0;
  if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess) lds = 65536;
  info->lds_bytes_per_block = lds;
  strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
  info->is_gfx950 = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
  if (!info->is_gfx950) return EP_HIP_ENODEVICE;
  // Set-up for the entry point that allocates nothing: its accumulator's address on this device is looked up here, outside
  // any stream capture, when the queried device is the current one (a symbol lookup may load the code object, which a
  // capture in progress does not survive).
  int current = -1;
  if (hipGetDevice(&current) == hipSuccess && current == device) {
    float* unused = nullptr;
    const int status = ep::static_accumulator(&unused);
    if (status != EP_HIP_OK) return status;
  }
  return EP_HIP_OK;
}

int ep_hip_plan_describe(const int32_t* meta, const uint16_t* freq, size_t n_freq, int prob_bits, int tile_elements,
                         int lds_limit_bytes, int force_kind, ep_hip_plan_desc* desc) {
  if (meta == nullptr || desc == nullptr || (freq == nullptr && n_freq != 0)) return EP_HIP_EINVAL;
  if (prob_bits < 9 || prob_bits > 15 || tile_elements <= 0) return EP_HIP_EINVAL;
  memset(desc, 0, sizeof(*desc));
  const int64_t size = int64_t{1} << prob_bits;
  int64_t cursor = 0;
  int max_alphabet = 0;
  bool byte_ok = true, wide_ok = true, rank_ok = true;
  // Half precision holds z + 1/2 exactly for |z| < 1024 and m + 1/4 for |m| < 512; its entry keeps one bit beside a 15-bit frequency.
  bool half_ok = prob_bits <= 14;
  int64_t present = 0;       // symbols with non-zero frequency in the field streams so far
  for (int s = 0; s < ep::kStreams; ++s) {
    const int64_t sym_min = meta[s * 4 + 1], off = meta[s * 4 + 2], alphabet = meta[s * 4 + 3];
    if (meta[s * 4 + 0] < 0 || alphabet < 0 || off != cursor || off + alphabet > static_cast<int64_t>(n_freq)) return EP_HIP_EINVAL;
    if (alphabet > size) return EP_HIP_EINVAL;
    if (alphabet > 0) {
      int64_t sum = 0, top = 0;
      for (int64_t i = 0; i < alphabet; ++i) {
        sum += freq[off + i];
        top = freq[off + i] > top ? freq[off + i] : top;
      }
      if (sum != size) return EP_HIP_EINVAL;
      if (s == 0) {
        if (alphabet > 2 || sym_min != 0) return EP_HIP_EINVAL;   // the coset stream codes 0/1
      } else {
        if (sym_min < -128 || sym_min + alphabet - 1 > 127) byte_ok = false;
        if (alphabet > 1024 || top > 2047) wide_ok = false;
        if (sym_min < -32768 || sym_min + alphabet - 1 > 32767) rank_ok = false;
        const int64_t exact = s >= ep::kStreams - 2 ? 511 : 1023;       // the last field's two streams code m, z7 = 2 m + parity
        if (sym_min < -exact || sym_min + alphabet - 1 > exact) half_ok = false;
        for (int64_t i = 0; i < alphabet; ++i) present += freq[off + i] != 0;
      }
    }
    desc->present_offset[s + 1] = static_cast<int>(present);
    if (alphabet > max_alphabet) max_alphabet = static_cast<int>(alphabet);
    cursor += alphabet;
  }
  if (cursor != static_cast<int64_t>(n_freq)) return EP_HIP_EINVAL;
  if (meta[0 * 4 + 3] == 0) return EP_HIP_EINVAL;

  // The LDS-table kernels take tiles of at most 2^18 vectors (32-bit byte offsets inside a tile pair, 16-bit slide
  // counts); larger tiles get the global tables.
  const bool tile_fits = ep::tile_vectors_of(tile_elements) <= ep::kMaxLdsTileVectors;
  const bool lds_fits = tile_fits && prob_bits <= 11 && ep::lds_decode_bytes(prob_bits, 1, 1) <= lds_limit_bytes;
  const bool sym_ok = byte_ok && lds_fits;
  rank_ok = rank_ok && tile_fits && present <= 65535 && ep::lds_rank_decode_bytes(static_cast<int>(present), prob_bits, 4) <= lds_limit_bytes;
  int kind = EP_TABLE_GLOBAL64;
  if (lds_fits && byte_ok) kind = EP_TABLE_LDS_BYTE;
  else if (lds_fits && wide_ok) kind = EP_TABLE_LDS_WIDE;
  else if (rank_ok) kind = EP_TABLE_LDS_RANK;
  if (force_kind >= 0) {
    const bool allowed = force_kind == EP_TABLE_GLOBAL64 || (force_kind == EP_TABLE_LDS_BYTE && lds_fits && byte_ok) ||
                         (force_kind == EP_TABLE_LDS_WIDE && lds_fits && wide_ok) || (force_kind == EP_TABLE_LDS_RANK && rank_ok) ||
                         (force_kind == EP_TABLE_LDS_SYM && sym_ok);
    if (!allowed) return EP_HIP_EUNSUPPORTED;
    kind = force_kind;
  }
  if (kind != EP_TABLE_LDS_RANK) memset(desc->present_offset, 0, sizeof(desc->present_offset));
  desc->table_kind = kind;
  desc->prob_bits = prob_bits;
  desc->max_alphabet = max_alphabet;
  desc->alphabet_sum = static_cast<int>(cursor);
  if (kind == EP_TABLE_GLOBAL64) {
    desc->table_bytes = ep::kHeaderBytes + (static_cast<size_t>(ep::kStreams) << prob_bits) * 8;
    desc->lds_bytes = 0;
  } else if (kind == EP_TABLE_LDS_RANK) {
    desc->lds_bytes = static_cast<int>(ep::rank_table_bytes(static_cast<int>(present), prob_bits));
    desc->rank_values_half = half_ok ? 1 : 0;
    desc->table_bytes = ep::kHeaderBytes + static_cast<size_t>(desc->lds_bytes);
  } else {
    desc->table_bytes = ep::kHeaderBytes + (static_cast<size_t>(ep::kFieldStreams) << prob_bits) * 4;
    desc->lds_bytes = (ep::kFieldStreams << prob_bits) * 4;
    // Byte-valued plans whose slot tables leave room for only one workgroup per CU also carry the two-level form,
    // which fits twice: launches with more tile pairs than one pass of resident waves use it.
    const bool crowded = 2 * ep::lds_decode_bytes(prob_bits, 16, 1) > 160 * 1024;
    if (kind == EP_TABLE_LDS_SYM || (kind == EP_TABLE_LDS_BYTE && crowded && 2 * ep::lds_sym_decode_bytes(prob_bits, 16) <= 160 * 1024)) {
      desc->sym_offset = static_cast<int>((desc->table_bytes + 255) / 256 * 256);
      desc->table_bytes = static_cast<size_t>(desc->sym_offset) + static_cast<size_t>(ep::sym_table_bytes(prob_bits));
    }
  }
  return EP_HIP_OK;
}

int ep_hip_plan_build(const int32_t* stream_meta_dev, const uint16_t* freq_tables_dev, const ep_hip_plan_desc* desc,
                      void* tables_dev, void* stream) {
  if (stream_meta_dev == nullptr || desc == nullptr || tables_dev == nullptr) return EP_HIP_EINVAL;
  if (freq_tables_dev == nullptr && desc->alphabet_sum != 0) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(tables_dev) % 256 != 0) return EP_HIP_EINVAL;
  if (desc->prob_bits < 9 || desc->prob_bits > 15 || desc->table_kind < 0 || desc->table_kind > EP_TABLE_LDS_SYM) return EP_HIP_EINVAL;
  if (desc->sym_offset != 0 && (desc->sym_offset % 256 != 0 || desc->prob_bits > 11 ||
                                static_cast<size_t>(desc->sym_offset) + ep::sym_table_bytes(desc->prob_bits) > desc->table_bytes)) return EP_HIP_EINVAL;
  if (desc->table_kind == EP_TABLE_LDS_SYM && desc->sym_offset == 0) return EP_HIP_EINVAL;
  if (desc->table_bytes < ep::kHeaderBytes || desc->table_bytes % 16 != 0) return EP_HIP_EINVAL;
  ep::RankLayout rank = {};
  if (desc->table_kind == EP_TABLE_LDS_RANK) {
    const int present = desc->present_offset[ep::kStreams];
    if (present < 0 || present > 65535 || desc->table_bytes != ep::kHeaderBytes + ep::rank_table_bytes(present, desc->prob_bits)) return EP_HIP_EINVAL;
    for (int i = 0; i < 18; ++i) {
      if (desc->present_offset[i] < 0 || desc->present_offset[i] > present) return EP_HIP_EINVAL;
      rank.present_offset[i] = desc->present_offset[i];
    }
    rank.val_offset = static_cast<uint32_t>(ep::rank_fb_bytes(present));
    rank.rs_offset = static_cast<uint32_t>(ep::rank_rs_offset(present, desc->prob_bits));
    rank.values_half = desc->rank_values_half != 0;
    if (rank.values_half && desc->prob_bits > 14) return EP_HIP_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Slots of empty streams are never read, but keep the buffer deterministic; the rank form ORs into zeroed bitmaps.
  // A fill kernel rather than a memset node, so the call can be captured into a graph.
  const size_t quads = desc->table_bytes / 16;
  hipLaunchKernelGGL(ep::zero_fill_kernel, dim3(static_cast<unsigned>((quads + 255) / 256 < 1024 ? (quads + 255) / 256 : 1024)),
                     dim3(256), 0, s, static_cast<uint4*>(tables_dev), quads);
  EP_HIP_TRY(hipGetLastError());
  // A plan of kind LDS_SYM holds the byte tables too (the kernels without a two-level form read those).
  const int built_kind = desc->table_kind == EP_TABLE_LDS_SYM ? EP_TABLE_LDS_BYTE : desc->table_kind;
  hipLaunchKernelGGL(ep::build_tables_kernel, dim3(ep::kStreams), dim3(256), 0, s, stream_meta_dev, freq_tables_dev,
                     built_kind, desc->prob_bits, static_cast<uint32_t*>(tables_dev), rank);
  EP_HIP_TRY(hipGetLastError());
  if (desc->sym_offset != 0) {
    hipLaunchKernelGGL(ep::build_sym_tables_kernel, dim3(ep::kFieldStreams), dim3(256), 0, s, stream_meta_dev, freq_tables_dev,
                       desc->prob_bits, static_cast<uint8_t*>(tables_dev) + desc->sym_offset);
    EP_HIP_TRY(hipGetLastError());
  }
  return EP_HIP_OK;
}

}  // extern "C"
