// Rank/select instantiations of the LDS-table decode kernels (any prob_bits): stores, batches and multiply-on-the-fly.
#include "ep_decode_lds.hpp"

namespace ep {

#define EP_LAUNCH_PARAMS const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, const DecodeArgs* jobs, const BlockJob* block_jobs, uint8_t* arena, hipStream_t stream
#define EP_LAUNCH_ARGS cfg, args, num_pairs, jobs, block_jobs, arena, stream

template <int PB, int KIND>
static int launch_rank_one(EP_LAUNCH_PARAMS) {
  static thread_local int configured_for[2] = {-1, -1};
  if (block_jobs != nullptr) {
    if constexpr (KIND == kKindDot1 || KIND == kKindDot4) return EP_HIP_EINVAL;
    else return launch_batch(decode_rank_batch_kernel<PB, KIND>, configured_for[1], cfg, jobs, block_jobs, arena, stream);
  }
  return launch_single(decode_rank_kernel<PB, KIND>, configured_for[0], cfg, args, num_pairs, stream);
}

template <int PB>
static int launch_rank_pb(EP_LAUNCH_PARAMS) {
  switch (cfg.kind) {
    case EP_STORE_BF16: return launch_rank_one<PB, EP_STORE_BF16>(EP_LAUNCH_ARGS);
    case EP_STORE_I8: return launch_rank_one<PB, EP_STORE_I8>(EP_LAUNCH_ARGS);
    case kKindDot1: return launch_rank_one<PB, kKindDot1>(EP_LAUNCH_ARGS);
    case kKindDot4: return launch_rank_one<PB, kKindDot4>(EP_LAUNCH_ARGS);
    default: return launch_rank_one<PB, kKindAny>(EP_LAUNCH_ARGS);
  }
}

int launch_rank(EP_LAUNCH_PARAMS) {
  switch (cfg.prob_bits) {
    case 9: return launch_rank_pb<9>(EP_LAUNCH_ARGS);
    case 10: return launch_rank_pb<10>(EP_LAUNCH_ARGS);
    case 11: return launch_rank_pb<11>(EP_LAUNCH_ARGS);
    case 12: return launch_rank_pb<12>(EP_LAUNCH_ARGS);
    case 13: return launch_rank_pb<13>(EP_LAUNCH_ARGS);
    case 14: return launch_rank_pb<14>(EP_LAUNCH_ARGS);
    case 15: return launch_rank_pb<15>(EP_LAUNCH_ARGS);
    default: return EP_HIP_EINVAL;
  }
}

}  // namespace ep
