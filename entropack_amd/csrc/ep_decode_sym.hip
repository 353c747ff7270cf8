// Two-level-table instantiations of the LDS-table decode kernels (byte values, prob_bits <= 11): stores, batches and
// multiply-on-the-fly.
#include "ep_decode_lds.hpp"

namespace ep {

#define EP_LAUNCH_PARAMS const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, const DecodeArgs* jobs, const BlockJob* block_jobs, uint8_t* arena, hipStream_t stream
#define EP_LAUNCH_ARGS cfg, args, num_pairs, jobs, block_jobs, arena, stream

template <int PB, int KIND>
static int launch_sym_one(EP_LAUNCH_PARAMS) {
  static thread_local int configured_for[2] = {-1, -1};
  if (block_jobs != nullptr) return launch_batch(decode_sym_batch_kernel<PB, KIND>, configured_for[1], cfg, jobs, block_jobs, arena, stream);
  return launch_single(decode_sym_kernel<PB, KIND>, configured_for[0], cfg, args, num_pairs, stream);
}

template <int PB, int KIND>
static int launch_sym_dot(EP_LAUNCH_PARAMS) {
  static thread_local int configured_for = -1;
  if (block_jobs != nullptr) return EP_HIP_EINVAL;
  return launch_single(decode_sym_kernel<PB, KIND>, configured_for, cfg, args, num_pairs, stream);
}

template <int PB>
static int launch_sym_pb(EP_LAUNCH_PARAMS) {
  switch (cfg.kind) {
    case EP_STORE_BF16: return launch_sym_one<PB, EP_STORE_BF16>(EP_LAUNCH_ARGS);
    case EP_STORE_I8: return launch_sym_one<PB, EP_STORE_I8>(EP_LAUNCH_ARGS);
    case kKindDot1: return launch_sym_dot<PB, kKindDot1>(EP_LAUNCH_ARGS);
    case kKindDot4: return EP_HIP_EINVAL;       // four activation rows do not fit this kernel's 64 registers
    default: return launch_sym_one<PB, kKindAny>(EP_LAUNCH_ARGS);
  }
}

int launch_sym(EP_LAUNCH_PARAMS) {
  switch (cfg.prob_bits) {
    case 9: return launch_sym_pb<9>(EP_LAUNCH_ARGS);
    case 10: return launch_sym_pb<10>(EP_LAUNCH_ARGS);
    case 11: return launch_sym_pb<11>(EP_LAUNCH_ARGS);
    default: return EP_HIP_EINVAL;
  }
}

}  // namespace ep
