// Multiply-on-the-fly instantiations of the byte / wide LDS-table decode kernels (prob_bits <= 11): the decoded weights
// meet one to four activation rows in registers and only y = x W^T leaves the kernel.
#include "ep_decode_lds.hpp"

namespace ep {

template <int PB, int MODE, int ILP, int KIND>
static int launch_dot_one(const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, hipStream_t stream) {
  static thread_local int configured_for = -1;
  return launch_single(decode_lds_kernel<PB, MODE, ILP, KIND>, configured_for, cfg, args, num_pairs, stream);
}

template <int PB, int MODE>
static int launch_dot_pb(const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, hipStream_t stream) {
  const bool one = cfg.kind == kKindDot1;
  if (cfg.ilp == 2) return one ? launch_dot_one<PB, MODE, 2, kKindDot1>(cfg, args, num_pairs, stream) : launch_dot_one<PB, MODE, 2, kKindDot4>(cfg, args, num_pairs, stream);
  return one ? launch_dot_one<PB, MODE, 1, kKindDot1>(cfg, args, num_pairs, stream) : launch_dot_one<PB, MODE, 1, kKindDot4>(cfg, args, num_pairs, stream);
}

int launch_dot(const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, hipStream_t stream) {
  const bool wide = cfg.table_kind == EP_TABLE_LDS_WIDE;
  switch (cfg.prob_bits) {
    case 9: return wide ? launch_dot_pb<9, kModeWide>(cfg, args, num_pairs, stream) : launch_dot_pb<9, kModeByte>(cfg, args, num_pairs, stream);
    case 10: return wide ? launch_dot_pb<10, kModeWide>(cfg, args, num_pairs, stream) : launch_dot_pb<10, kModeByte>(cfg, args, num_pairs, stream);
    case 11: return wide ? launch_dot_pb<11, kModeWide>(cfg, args, num_pairs, stream) : launch_dot_pb<11, kModeByte>(cfg, args, num_pairs, stream);
    default: return EP_HIP_EINVAL;
  }
}

}  // namespace ep
