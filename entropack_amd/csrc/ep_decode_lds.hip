// Launch side of the LDS-table decode kernels: byte / wide slot tables (prob_bits <= 11), stores to memory.
// The kernels themselves are templates in ep_decode_lds.hpp; the rank/select and multiply-on-the-fly instantiations
// are compiled in ep_decode_rank.hip and ep_decode_dot.hip.
#include "ep_decode_lds.hpp"

namespace ep {

#define EP_LAUNCH_PARAMS const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, const DecodeArgs* jobs, const BlockJob* block_jobs, uint8_t* arena, hipStream_t stream
#define EP_LAUNCH_ARGS cfg, args, num_pairs, jobs, block_jobs, arena, stream

template <int PB, int MODE, int ILP, int KIND>
static int launch_one(EP_LAUNCH_PARAMS) {
  static thread_local int configured_for[2] = {-1, -1};
  if (block_jobs != nullptr) return launch_batch(decode_lds_batch_kernel<PB, MODE, ILP, KIND>, configured_for[1], cfg, jobs, block_jobs, arena, stream);
  return launch_single(decode_lds_kernel<PB, MODE, ILP, KIND>, configured_for[0], cfg, args, num_pairs, stream);
}

template <int PB, int MODE>
static int launch_pb(EP_LAUNCH_PARAMS) {
  if (cfg.ilp == 2) {
    if (cfg.kind == EP_STORE_BF16) return launch_one<PB, MODE, 2, EP_STORE_BF16>(EP_LAUNCH_ARGS);
    if (cfg.kind == EP_STORE_I8) return launch_one<PB, MODE, 2, EP_STORE_I8>(EP_LAUNCH_ARGS);
    return launch_one<PB, MODE, 2, kKindAny>(EP_LAUNCH_ARGS);
  }
  if (cfg.kind == EP_STORE_BF16) return launch_one<PB, MODE, 1, EP_STORE_BF16>(EP_LAUNCH_ARGS);
  if (cfg.kind == EP_STORE_I8) return launch_one<PB, MODE, 1, EP_STORE_I8>(EP_LAUNCH_ARGS);
  return launch_one<PB, MODE, 1, kKindAny>(EP_LAUNCH_ARGS);
}

static int lds_bytes_for(int table_kind, int prob_bits, int lut_bytes, int waves, int ilp) {
  if (table_kind == EP_TABLE_LDS_RANK) return lds_rank_decode_bytes_of(lut_bytes, waves);
  if (table_kind == EP_TABLE_LDS_SYM) return lds_sym_decode_bytes(prob_bits, waves);
  return lds_decode_bytes(prob_bits, waves, ilp);
}

// Workgroups per CU and the largest workgroup (in waves) for a table form: two workgroups when their tables and
// at least 12 waves' windows each fit the CU's LDS together (8 waves per SIMD with 16), else one of 16 waves.
static void lds_block_shape(int table_kind, int prob_bits, int lut_bytes, int& resident, int& most_waves) {
  for (int waves = 16; waves >= 12; --waves) {
    if (2 * lds_bytes_for(table_kind, prob_bits, lut_bytes, waves, 1) <= 160 * 1024) {
      resident = 2;
      most_waves = waves;
      return;
    }
  }
  resident = 1;
  most_waves = 16;
}

int lds_resident_blocks(int table_kind, int prob_bits, int lut_bytes) {
  int resident = 1, most_waves = 16;
  lds_block_shape(table_kind, prob_bits, lut_bytes, resident, most_waves);
  return resident;
}

int effective_table_kind(const ep_hip_plan_desc& desc, int kind, int64_t pairs, int cus) {
  const bool has_kernel = kind == EP_STORE_BF16 || kind == EP_STORE_I8 || kind == kKindAny || kind == kKindDot1;
  if (desc.table_kind == EP_TABLE_LDS_SYM) return has_kernel ? EP_TABLE_LDS_SYM : EP_TABLE_LDS_BYTE;     // the byte tables are there too
  if (desc.table_kind == EP_TABLE_LDS_BYTE && desc.sym_offset != 0 && has_kernel && pairs > static_cast<int64_t>(cus) * 16) return EP_TABLE_LDS_SYM;
  return desc.table_kind;
}

LdsLaunch choose_lds_launch(int table_kind, int prob_bits, int lut_bytes, int kind, int pairs, int cus) {
  LdsLaunch cfg;
  cfg.table_kind = table_kind;
  cfg.prob_bits = prob_bits;
  cfg.kind = kind;
  // Tables that leave room for two blocks per CU run one pair per wave on twice the waves, which hides latency best.
  // Otherwise one block per CU, and two interleaved pairs per wave once 16 waves on every CU cannot hold all pairs.
  int resident = 1, most_waves = 16;
  lds_block_shape(table_kind, prob_bits, lut_bytes, resident, most_waves);
  const bool single_pair_only = table_kind == EP_TABLE_LDS_RANK || table_kind == EP_TABLE_LDS_SYM;
  cfg.ilp = !single_pair_only && resident == 1 && pairs > cus * 16 ? 2 : 1;
  int waves = (pairs + cus * resident * cfg.ilp - 1) / (cus * resident * cfg.ilp);
  waves = waves < 1 ? 1 : (waves > most_waves ? most_waves : waves);
  int blocks = (pairs + waves * cfg.ilp - 1) / (waves * cfg.ilp);
  cfg.blocks = blocks > cus * resident ? cus * resident : blocks;
  cfg.threads = waves * 64;
  cfg.lds_bytes = lds_bytes_for(table_kind, prob_bits, lut_bytes, waves, cfg.ilp);
  return cfg;
}

int launch_lds(EP_LAUNCH_PARAMS) {
  if (cfg.table_kind == EP_TABLE_LDS_RANK) return launch_rank(EP_LAUNCH_ARGS);
  if (cfg.table_kind == EP_TABLE_LDS_SYM) return launch_sym(EP_LAUNCH_ARGS);
  if (cfg.kind == kKindDot1 || cfg.kind == kKindDot4) return block_jobs == nullptr ? launch_dot(cfg, args, num_pairs, stream) : EP_HIP_EINVAL;
  const bool wide = cfg.table_kind == EP_TABLE_LDS_WIDE;
  switch (cfg.prob_bits) {
    case 9: return wide ? launch_pb<9, kModeWide>(EP_LAUNCH_ARGS) : launch_pb<9, kModeByte>(EP_LAUNCH_ARGS);
    case 10: return wide ? launch_pb<10, kModeWide>(EP_LAUNCH_ARGS) : launch_pb<10, kModeByte>(EP_LAUNCH_ARGS);
    case 11: return wide ? launch_pb<11, kModeWide>(EP_LAUNCH_ARGS) : launch_pb<11, kModeByte>(EP_LAUNCH_ARGS);
    default: return EP_HIP_EINVAL;
  }
}

int launch_lds_decode(const DecodeArgs& args, const ep_hip_plan_desc& desc, int kind, int pairs, hipStream_t stream) {
  int device = 0, cus = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  EP_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  if (cus <= 0) cus = 256;
  const LdsLaunch cfg = choose_lds_launch(effective_table_kind(desc, kind, pairs, cus), desc.prob_bits, desc.lds_bytes, kind, pairs, cus);
  return launch_lds(cfg, args, pairs, nullptr, nullptr, nullptr, stream);
}

}  // namespace ep
