// decode_lds_kernel: lattice_rans decode for prob_bits <= 11 with every table in LDS (gfx950, wave64).
//
// Work split. A tile owns 32 rANS lanes; a wave carries a *pair* of tiles (lower half = tile 2p, upper half =
// tile 2p + 1) and, when the grid is large enough, two pairs interleaved to hide LDS latency. One workgroup per
// CU stages the 16 field tables once (u32 per slot: frequency | slot - cdf | symbol) and then walks its pairs.
//
// Payload. Renormalisation words are consumed from the tile's end downwards, at most 32 per step. Each half keeps
// a 192-word LDS window holding payload[W, W + 192), W a multiple of 64, with the read position p = ptr - W. The 64
// words below W are already in flight in a register (one dword per lane). After every second step the window is
// checked: when p has dropped below 64 it slides down by 64 words (its lower chunk moves up, the prefetched words
// become the lower chunk and the next 64 are requested), so p is in [64, 128) before a pair of steps, at least 32
// between them and at least 0 after them, whatever the stream holds, and no renormalisation ever waits on HBM.
// Both halves' p live in one scalar register, biased by 64 so that the packed arithmetic never borrows; the
// requests address the payload as a wave-uniform origin plus a saturating 32-bit offset per lane, and slides are
// counted (the end-of-tile check needs to know where each window ended up).
//
// The nine dependent symbol steps of a group are written in inline assembly: the compiler's version of the same
// C++ spent more scalar than vector instructions on mask bookkeeping. Per step and pair: 12 VALU, 8 SALU, one
// ds_read_b32 (slot table) and one ds_read_u16 (window). The scalar part turns the vote of "state < 2^15" into
// the two halves' word counts; lane l then reads window[p_half - n_half + rank_in_half(l)], which is the
// reference's "i-th reader in ascending lane order takes words[ptr - n + i]".
//
// Everything around the steps (tile set-up, ring refill, E8 reconstruction, row scale, container cast, stores,
// end-of-tile checks) is ordinary HIP C++. Tiles hold at most kMaxLdsTileVectors vectors: positions inside a pair
// of tiles are 32-bit byte offsets and a tile's slides are counted in 16 bits.
#pragma once

#include <type_traits>

#include "ep_store.hpp"

namespace ep {

constexpr int kModeByte = 0, kModeWide = 1, kModeRank = 2, kModeSym = 3;
constexpr uint32_t kPosBias = 64;
// KIND template values besides an ep_hip_store_kind: any container through the generic store, or no store at all:
// the decoded weights are multiplied with a few activation rows on the fly (a.x, a.y32).
constexpr int kKindAny = -1, kKindDot1 = -2, kKindDot4 = -3;    // one activation row, or up to four
constexpr int kDotRows = 4;

template <int PB, int MODE>
struct Layout {
  static constexpr bool WIDE = MODE == kModeWide;
  static constexpr uint32_t kTable = 1u << PB;
  static constexpr uint32_t kTableBytes = 4u << PB;             // one stream's table
  static constexpr uint32_t kLutBytes = kFieldStreams * kTableBytes;
  static constexpr uint32_t kSlotMask4 = kTableBytes - 4u;      // (slot << 2) mask
  static constexpr uint32_t kHighBase = 8u * kTableBytes;       // fields 4..7 are addressed from base + this
  static constexpr int kFreqMask = WIDE ? 0x7FF : 0xFFF;
  static constexpr int kDeltaShift = WIDE ? 11 : 12;
  static constexpr int kDeltaWidth = WIDE ? 11 : 12;            // byte form: bits 12..23 (lattice containers use 11 of them)
  static constexpr int kSymShift = WIDE ? 22 : 24;
};

// One pair of tiles as a wave sees it. `pos` is wave-uniform; the rest is per lane.
struct Pair {
  uint32_t x;            // rANS state
  uint32_t prefetch;     // the 64 payload words below the ring, 2 per lane
  uint32_t fetch_at;     // byte offset from `origin` of the dword `prefetch` came from
  const uint8_t* origin; // wave-uniform: a 64-word boundary of the payload at or below every word the pair still needs
  uint32_t ring;         // half the LDS byte address of position 0 of this half's 128-word window
  uint32_t ring_lane;    // ring + 4 * (lane & 31): where this lane's dword of a 64-word chunk goes
  uint32_t vector0;      // first vector of this lane's tile
  int count;             // vectors in this lane's tile (0 = no tile)
  uint32_t pos;          // (pA + 64) | (pB + 64) << 16: read positions inside the windows, biased by kPosBias so that the
                         // scalar arithmetic of a step never borrows across the fields while pA, pB fall to 0
  int windowA, windowB;  // where the windows started, relative to a 64-aligned base below each tile's first word
  uint64_t slid;         // slides so far: the lower half's count from bit 7 (16 bits), the upper half's from bit 23
  int beginA, beginB;    // position of each tile's first word, relative to that base
  uint32_t coset_base;   // LDS byte offset of this lane's coset inside a field's table pair (0 or one table)
  uint64_t coset_mask;   // wave-uniform: the lanes whose current vector lies in coset 1
  uint32_t e[8];         // slot-table entries of the eight fields of the current vector
  uint32_t ey[8];        // two-level tables only: the entries' second words (the value in half precision in the high half)
  int dot_row;           // multiply-on-the-fly only: the weight row `dot_acc` belongs to (same in all lanes of a half), -1 = none
  float dot_acc[kDotRows];
};

// ---- the symbol steps ----------------------------------------------------------------------------------------------
//
// Operand names: x state, pos packed positions, e entry out, t/h/d temporaries, na/nb scalar temporaries,
// cb table base (coset | field group), ring ring base, shv 0 (lower half) or 16 (upper half).

#define EP_ASM_MASK_ON "s_mov_b64 %[sv], exec\n s_and_b64 exec, exec, %[valid]\n"
#define EP_ASM_MASK_OFF "s_mov_b64 exec, %[sv]\n"

// state -> table address -> issue the gather; h = state >> PB meanwhile.
#define EP_ASM_LOOKUP(S)                                        \
  "v_lshlrev_b32 %[t" S "], 2, %[x" S "]\n"                      \
  "v_and_or_b32 %[t" S "], %[t" S "], %[kslot], %[cb" S "]\n"    \
  "ds_read_b32 %[e" S "], %[t" S "] offset:%[off]\n"             \
  "v_lshrrev_b32 %[h" S "], %[pb], %[x" S "]\n"

// x = freq * (x >> PB) + (slot - cdf)
#define EP_ASM_ADVANCE(S)                                       \
  "v_and_b32 %[t" S "], %[fmask], %[e" S "]\n"                   \
  "v_bfe_u32 %[d" S "], %[e" S "], %[dshift], %[dwidth]\n"       \
  "v_mad_u32_u24 %[x" S "], %[t" S "], %[h" S "], %[d" S "]\n"

// Vote, per-half counts, window address, issue the window read, new positions. Leaves the vote in vcc.
// With n_a, n_b the halves' counts: lane l of the lower half reads at p_a - n_a + rank(l), and a lane of the upper
// half, whose rank as the two mbcnt instructions count it includes n_a, at p_b - (n_a + n_b) + rank(l). Both bases
// come from one subtraction of (n_a | (n_a + n_b) << 16); the positions themselves (p - n per half) follow after
// the read is issued. The lane ranks are counted on top of half the window's byte address while the scalar side is
// still busy, so that only two vector instructions separate the scalar result from the read. pos stays >= 32 in both halves, so no subtraction borrows across the 16-bit fields.
#define EP_ASM_VOTE(S)                                          \
  "v_cmp_gt_u32 vcc, 0x8000, %[x" S "]\n"                        \
  "s_bcnt1_i32_b32 %[na], vcc_lo\n"                              \
  "s_bcnt1_i32_b64 %[nb], vcc\n"                                 \
  "v_mbcnt_lo_u32_b32 %[t" S "], vcc_lo, %[ring" S "]\n"         \
  "s_pack_ll_b32_b16 %[nb], %[na], %[nb]\n"                      \
  "v_mbcnt_hi_u32_b32 %[t" S "], vcc_hi, %[t" S "]\n"            \
  "s_sub_u32 %[nb], %[pos" S "], %[nb]\n"                        \
  "v_bfe_u32 %[d" S "], %[nb], %[shv], 16\n"                     \
  "v_add_lshl_u32 %[t" S "], %[t" S "], %[d" S "], 1\n"          \
  "ds_read_u16 %[d" S "], %[t" S "]\n"                           \
  "s_lshl_b32 %[na], %[na], 16\n"                                \
  "s_add_u32 %[pos" S "], %[nb], %[na]\n"

// x = voted ? x << 16 | word : x
#define EP_ASM_TAKE_VCC(S)                                      \
  "v_lshl_or_b32 %[t" S "], %[x" S "], 16, %[d" S "]\n"          \
  "v_cndmask_b32 %[x" S "], %[x" S "], %[t" S "], vcc\n"
#define EP_ASM_TAKE_SAVED(S)                                    \
  "v_lshl_or_b32 %[t" S "], %[x" S "], 16, %[d" S "]\n"          \
  "v_cndmask_b32_e64 %[x" S "], %[x" S "], %[t" S "], %[m0]\n"
// The same with the vote as execution mask (one vector instruction less). Only the unmasked steps use it: they run
// with every lane active, so the mask is restored to all ones without having been saved.
#define EP_ASM_TAKE_EXEC_VCC(S) "s_mov_b64 exec, vcc\n v_lshl_or_b32 %[x" S "], %[x" S "], 16, %[d" S "]\n"
#define EP_ASM_TAKE_EXEC_SAVED(S) "s_mov_b64 exec, %[m0]\n v_lshl_or_b32 %[x" S "], %[x" S "], 16, %[d" S "]\n"
#define EP_ASM_RESTORE_FULL "s_mov_b64 exec, -1\n"

// Coset symbol in closed form: c = slot >= f0; freq = c ? T - f0 : f0; begin = c ? f0 : 0. The lanes with c = 1
// are also left as a mask in scalar registers (cm), for selections that would otherwise compare cb with 0 again.
#define EP_ASM_COSET(S)                                         \
  "v_and_b32 %[t" S "], %[slotmask], %[x" S "]\n"                \
  "v_lshrrev_b32 %[h" S "], %[pb], %[x" S "]\n"                  \
  "v_cmp_le_u32 vcc, %[f0s], %[t" S "]\n"                        \
  "s_mov_b64 %[cm" S "], vcc\n"                                  \
  "v_cndmask_b32 %[cb" S "], 0, %[f0v], vcc\n"                   \
  "v_sub_u32 %[t" S "], %[t" S "], %[cb" S "]\n"                 \
  "v_cndmask_b32 %[d" S "], %[f0v], %[f1v], vcc\n"               \
  "v_mad_u32_u24 %[x" S "], %[d" S "], %[h" S "], %[t" S "]\n"   \
  "v_cndmask_b32 %[cb" S "], 0, %[ktab], vcc\n"

// Values the steps take in scalar registers. They are wave-uniform by construction; saying so explicitly keeps the
// register allocator from ever holding them per lane (a no-op when it already has them in scalar registers).
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint64_t uniform(uint64_t v) {
  return static_cast<uint64_t>(uniform(static_cast<uint32_t>(v))) | (static_cast<uint64_t>(uniform(static_cast<uint32_t>(v >> 32))) << 32);
}

__device__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
  return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);     // one v_bitop3_b32
}

struct StepConsts {
  uint32_t shv;      // per lane: 0 or 16
  uint32_t f0v;      // per lane copies of the coset frequencies and one table's byte size
  uint32_t f1v;
  uint32_t ktab;
  uint32_t f0s;      // wave-uniform
};

template <int PB, int MODE, bool MASKED>
__device__ __forceinline__ void field_step_single(Pair& p, int field, uint32_t off, uint32_t cb, const StepConsts& k,
                                                  uint64_t valid) {
  using L = Layout<PB, MODE>;
  uint32_t t, h, d, e, na, nb;
  uint64_t sv;
  const uint32_t kslot = L::kSlotMask4;
  uint32_t pos = uniform(p.pos);
  valid = uniform(valid);
#define EP_FIELD_SINGLE_BODY                                                                           \
  EP_ASM_LOOKUP("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_ADVANCE("0") EP_ASM_VOTE("0") "s_waitcnt lgkmcnt(0)\n" \
      EP_ASM_TAKE_VCC("0")
#define EP_FIELD_SINGLE_FAST                                                                                   \
  EP_ASM_LOOKUP("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_ADVANCE("0") EP_ASM_VOTE("0")              \
      "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_EXEC_VCC("0") EP_ASM_RESTORE_FULL
#define EP_FIELD_SINGLE_OPERANDS(OFF)                                                                           \
  : [x0] "+v"(p.x), [pos0] "+s"(pos), [e0] "=&v"(e), [t0] "=&v"(t), [h0] "=&v"(h), [d0] "=&v"(d), [na] "=&s"(na),   \
    [nb] "=&s"(nb), [sv] "=&s"(sv)                                                                               \
  : [cb0] "v"(cb), [ring0] "v"(p.ring), [shv] "v"(k.shv), [kslot] "s"(kslot), [valid] "s"(valid), \
    [off] "n"(OFF), [pb] "n"(PB), [fmask] "n"(L::kFreqMask), [dshift] "n"(L::kDeltaShift), [dwidth] "n"(L::kDeltaWidth)                           \
  : "vcc", "scc", "memory"
  // The LDS offset must be an immediate, so the four field positions inside a group are spelled out.
#define EP_FIELD_SINGLE_CASE(OFF)                                                                              \
  if constexpr (MASKED) asm volatile(EP_ASM_MASK_ON EP_FIELD_SINGLE_BODY EP_ASM_MASK_OFF EP_FIELD_SINGLE_OPERANDS(OFF)); \
  else asm volatile(EP_FIELD_SINGLE_FAST EP_FIELD_SINGLE_OPERANDS(OFF))
  switch (off) {
    case 0: EP_FIELD_SINGLE_CASE(0 * 2 * L::kTableBytes); break;
    case 1: EP_FIELD_SINGLE_CASE(1 * 2 * L::kTableBytes); break;
    case 2: EP_FIELD_SINGLE_CASE(2 * 2 * L::kTableBytes); break;
    default: EP_FIELD_SINGLE_CASE(3 * 2 * L::kTableBytes); break;
  }
  p.e[field] = e;
  p.pos = pos;
}

template <int PB, int MODE, bool MASKED>
__device__ __forceinline__ void field_step_dual(Pair& p0, Pair& p1, int field, uint32_t off, uint32_t cb0, uint32_t cb1,
                                                const StepConsts& k, uint64_t valid) {
  using L = Layout<PB, MODE>;
  uint32_t t0, h0, d0, e0, t1, h1, d1, e1, na, nb;
  uint64_t sv, m0;
  const uint32_t kslot = L::kSlotMask4;
  uint32_t pos0 = uniform(p0.pos), pos1 = uniform(p1.pos);
  valid = uniform(valid);
  // Issue order: both gathers, pair 0 advances and issues its ring read while pair 1's gather lands, and so on;
  // LDS returns in order, so lgkmcnt(1) always means "everything but the newest read has arrived".
#define EP_FIELD_DUAL_BODY                                                                                    \
  EP_ASM_LOOKUP("0") EP_ASM_LOOKUP("1") "s_waitcnt lgkmcnt(1)\n" EP_ASM_ADVANCE("0") EP_ASM_VOTE("0")            \
      "s_mov_b64 %[m0], vcc\n s_waitcnt lgkmcnt(1)\n" EP_ASM_ADVANCE("1") EP_ASM_VOTE("1") "s_waitcnt lgkmcnt(1)\n" \
          EP_ASM_TAKE_SAVED("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_VCC("1")
#define EP_FIELD_DUAL_FAST                                                                                     \
  EP_ASM_LOOKUP("0") EP_ASM_LOOKUP("1") "s_waitcnt lgkmcnt(1)\n" EP_ASM_ADVANCE("0")            \
      EP_ASM_VOTE("0") "s_mov_b64 %[m0], vcc\n s_waitcnt lgkmcnt(1)\n" EP_ASM_ADVANCE("1") EP_ASM_VOTE("1")      \
          "s_waitcnt lgkmcnt(1)\n" EP_ASM_TAKE_EXEC_SAVED("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_EXEC_VCC("1") \
              EP_ASM_RESTORE_FULL
#define EP_FIELD_DUAL_OPERANDS(OFF)                                                                             \
  : [x0] "+v"(p0.x), [x1] "+v"(p1.x), [pos0] "+s"(pos0), [pos1] "+s"(pos1), [e0] "=&v"(e0), [e1] "=&v"(e1),       \
    [t0] "=&v"(t0), [t1] "=&v"(t1), [h0] "=&v"(h0), [h1] "=&v"(h1), [d0] "=&v"(d0), [d1] "=&v"(d1), [na] "=&s"(na), \
    [nb] "=&s"(nb), [sv] "=&s"(sv), [m0] "=&s"(m0)                                                               \
  : [cb0] "v"(cb0), [cb1] "v"(cb1), [ring0] "v"(p0.ring), [ring1] "v"(p1.ring), [shv] "v"(k.shv),                \
    [kslot] "s"(kslot), [valid] "s"(valid), [off] "n"(OFF), [pb] "n"(PB),                    \
    [fmask] "n"(L::kFreqMask), [dshift] "n"(L::kDeltaShift), [dwidth] "n"(L::kDeltaWidth)                                                      \
  : "vcc", "scc", "memory"
#define EP_FIELD_DUAL_CASE(OFF)                                                                            \
  if constexpr (MASKED) asm volatile(EP_ASM_MASK_ON EP_FIELD_DUAL_BODY EP_ASM_MASK_OFF EP_FIELD_DUAL_OPERANDS(OFF)); \
  else asm volatile(EP_FIELD_DUAL_FAST EP_FIELD_DUAL_OPERANDS(OFF))
  switch (off) {
    case 0: EP_FIELD_DUAL_CASE(0 * 2 * L::kTableBytes); break;
    case 1: EP_FIELD_DUAL_CASE(1 * 2 * L::kTableBytes); break;
    case 2: EP_FIELD_DUAL_CASE(2 * 2 * L::kTableBytes); break;
    default: EP_FIELD_DUAL_CASE(3 * 2 * L::kTableBytes); break;
  }
  p0.e[field] = e0;
  p1.e[field] = e1;
  p0.pos = pos0;
  p1.pos = pos1;
}

template <int PB, int MODE, bool MASKED>
__device__ __forceinline__ void coset_step_single(Pair& p, const StepConsts& k, uint64_t valid) {
  using L = Layout<PB, MODE>;
  uint32_t t, h, d, cb, na, nb;
  uint64_t sv, cm;
  const uint32_t f0s = k.f0s;
  uint32_t pos = uniform(p.pos);
  valid = uniform(valid);
#define EP_COSET_SINGLE_BODY EP_ASM_COSET("0") EP_ASM_VOTE("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_VCC("0")
#define EP_COSET_SINGLE_FAST \
  EP_ASM_COSET("0") EP_ASM_VOTE("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_EXEC_VCC("0") EP_ASM_RESTORE_FULL
#define EP_COSET_SINGLE_OPERANDS                                                                                \
  : [x0] "+v"(p.x), [pos0] "+s"(pos), [cb0] "=&v"(cb), [t0] "=&v"(t), [h0] "=&v"(h), [d0] "=&v"(d), [na] "=&s"(na),  \
    [nb] "=&s"(nb), [sv] "=&s"(sv), [cm0] "=&s"(cm)                                                              \
  : [ring0] "v"(p.ring), [shv] "v"(k.shv), [f0v] "v"(k.f0v), [f1v] "v"(k.f1v), [ktab] "v"(k.ktab), [f0s] "s"(f0s),  \
    [valid] "s"(valid), [pb] "n"(PB), [slotmask] "n"(L::kTable - 1)                          \
  : "vcc", "scc", "memory"
  if constexpr (MASKED) asm volatile(EP_ASM_MASK_ON EP_COSET_SINGLE_BODY EP_ASM_MASK_OFF EP_COSET_SINGLE_OPERANDS);
  else asm volatile(EP_COSET_SINGLE_FAST EP_COSET_SINGLE_OPERANDS);
  p.coset_base = cb;
  p.coset_mask = cm;
  p.pos = pos;
}

template <int PB, int MODE, bool MASKED>
__device__ __forceinline__ void coset_step_dual(Pair& p0, Pair& p1, const StepConsts& k, uint64_t valid) {
  using L = Layout<PB, MODE>;
  uint32_t t0, h0, d0, cb0, t1, h1, d1, cb1, na, nb;
  uint64_t sv, m0, cm0, cm1;
  const uint32_t f0s = k.f0s;
  uint32_t pos0 = uniform(p0.pos), pos1 = uniform(p1.pos);
  valid = uniform(valid);
#define EP_COSET_DUAL_BODY                                                                              \
  EP_ASM_COSET("0") EP_ASM_VOTE("0") "s_mov_b64 %[m0], vcc\n" EP_ASM_COSET("1") EP_ASM_VOTE("1")          \
      "s_waitcnt lgkmcnt(1)\n" EP_ASM_TAKE_SAVED("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_VCC("1")
#define EP_COSET_DUAL_FAST                                                                               \
  EP_ASM_COSET("0") EP_ASM_VOTE("0") "s_mov_b64 %[m0], vcc\n" EP_ASM_COSET("1") EP_ASM_VOTE("1") \
      "s_waitcnt lgkmcnt(1)\n" EP_ASM_TAKE_EXEC_SAVED("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_EXEC_VCC("1")     \
          EP_ASM_RESTORE_FULL
#define EP_COSET_DUAL_OPERANDS                                                                                    \
  : [x0] "+v"(p0.x), [x1] "+v"(p1.x), [pos0] "+s"(pos0), [pos1] "+s"(pos1), [cb0] "=&v"(cb0), [cb1] "=&v"(cb1),     \
    [t0] "=&v"(t0), [t1] "=&v"(t1), [h0] "=&v"(h0), [h1] "=&v"(h1), [d0] "=&v"(d0), [d1] "=&v"(d1), [na] "=&s"(na),   \
    [nb] "=&s"(nb), [sv] "=&s"(sv), [m0] "=&s"(m0), [cm0] "=&s"(cm0), [cm1] "=&s"(cm1)                             \
  : [ring0] "v"(p0.ring), [ring1] "v"(p1.ring), [shv] "v"(k.shv), [f0v] "v"(k.f0v), [f1v] "v"(k.f1v),              \
    [ktab] "v"(k.ktab), [f0s] "s"(f0s), [valid] "s"(valid), [pb] "n"(PB),                      \
    [slotmask] "n"(L::kTable - 1)                                                                                  \
  : "vcc", "scc", "memory"
  if constexpr (MASKED) asm volatile(EP_ASM_MASK_ON EP_COSET_DUAL_BODY EP_ASM_MASK_OFF EP_COSET_DUAL_OPERANDS);
  else asm volatile(EP_COSET_DUAL_FAST EP_COSET_DUAL_OPERANDS);
  p0.coset_base = cb0;
  p1.coset_base = cb1;
  p0.coset_mask = cm0;
  p1.coset_mask = cm1;
  p0.pos = pos0;
  p1.pos = pos1;
}

// ---- rank/select tables (any prob_bits) ---------------------------------------------------------------------------
//
// A slot table of 2^PB entries per stream does not fit LDS beyond prob_bits 11, but the alphabet does. Per stream and
// 32 slots the table keeps {bits, count}: bit b is set when slot 32 w + b is the last slot of its symbol, count is the
// number of symbols (of all field streams before this one, plus this stream's) that end before slot 32 w. The symbol
// of a slot is then count + popcount(bits below the slot): one 8-byte read, and a second read fetches that symbol's
// cdf | freq << 16 (the subtraction takes the low half where it lies; with half-precision values bit 31 marks an odd
// value and the frequency is the 15 bits below it, `freq_width`); its 16-bit value is read off the critical path. The
// lookups are ordinary C++; renormalisation is the same scalar vote as above.
template <int PB, bool MASKED>
__device__ __forceinline__ void rank_step(Pair& p, int field, uint32_t rs_group, uint32_t val0, uint32_t freq_width,
                                          const StepConsts& k, bool valid_lane) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(3))) const u32x2* lds_u2;
  typedef __attribute__((address_space(3))) const uint32_t* lds_u32;
  typedef __attribute__((address_space(3))) const uint16_t* lds_u16;
  constexpr uint32_t kTable = 1u << PB;
  const uint32_t x = p.x;
  const uint32_t slot = x & (kTable - 1u);
  // rs_group = the LDS address of field 0's words for this lane's coset, a multiple of one stream's size: the word
  // offset is OR-ed in, and the field's distance is a constant the read takes as its immediate offset.
  constexpr uint32_t kStreamBytes = (kTable / 32u) * 8u;
  const uint32_t word_at = ((x >> 2) & (kStreamBytes - 8u)) | rs_group;
  const u32x2 rs = *reinterpret_cast<lds_u2>(static_cast<uintptr_t>(word_at + static_cast<uint32_t>(2 * field) * kStreamBytes));
  // The bit-field extract takes its width from the low five bits of x: the bits of rs.x below slot % 32.
  const uint32_t index = static_cast<uint32_t>(__builtin_popcount(__builtin_amdgcn_ubfe(rs.x, 0u, x))) + rs.y;
  const uint32_t fb = *reinterpret_cast<lds_u32>(static_cast<uintptr_t>(index << 2));
  p.e[field] = *reinterpret_cast<lds_u16>(static_cast<uintptr_t>((index << 1) + val0));      // 16 bits, not extended
  p.ey[field] = fb;
  const uint32_t next = __umul24(__builtin_amdgcn_ubfe(fb, 16u, freq_width), x >> PB) + (slot - (fb & 0xFFFFu));
  p.x = (!MASKED || valid_lane) ? next : x;
  uint32_t t, d, na, nb;
  uint32_t pos = uniform(p.pos);
  if constexpr (MASKED) {
    asm volatile(EP_ASM_VOTE("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_VCC("0")
                 : [x0] "+v"(p.x), [pos0] "+s"(pos), [t0] "=&v"(t), [d0] "=&v"(d), [na] "=&s"(na), [nb] "=&s"(nb)
                 : [ring0] "v"(p.ring), [shv] "v"(k.shv)
                 : "vcc", "scc", "memory");
  } else {
    asm volatile(EP_ASM_VOTE("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_EXEC_VCC("0") EP_ASM_RESTORE_FULL
                 : [x0] "+v"(p.x), [pos0] "+s"(pos), [t0] "=&v"(t), [d0] "=&v"(d), [na] "=&s"(na), [nb] "=&s"(nb)
                 : [ring0] "v"(p.ring), [shv] "v"(k.shv)
                 : "vcc", "scc", "memory");
  }
  p.pos = pos;
}

// ---- two-level tables (byte values, prob_bits <= 11) --------------------------------------------------------------------
//
// slot -> value + 128 (one byte) -> {freq | parity mark, cdf | half(value) << 16}. A quarter of the slot table of the
// byte form, so two workgroups share a CU; one more dependent LDS read per step, one vector instruction less. The stored
// cdf already contains the coset offset that `slot | coset offset` carries. The entry holds the value as a
// half-precision number and its parity as a half-precision 0.0 / 1.0 pattern, so reconstruction needs no integer to
// float conversion (see sym_point below).
template <int PB, bool MASKED>
__device__ __forceinline__ void sym_step(Pair& p, int field, const StepConsts& k, bool valid_lane) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(3))) const u32x2* lds_u2;
  typedef __attribute__((address_space(3))) const uint8_t* lds_u8;
  constexpr uint32_t kTable = 1u << PB;
  const uint32_t x = p.x;
  const uint32_t at = (x & (kTable - 1u)) | p.coset_base;
  const uint32_t value = *reinterpret_cast<lds_u8>(static_cast<uintptr_t>(at + static_cast<uint32_t>(kSymFbBytes) + static_cast<uint32_t>(field) * 2u * kSymSlotStreamBytes));
  const u32x2 entry = *reinterpret_cast<lds_u2>(static_cast<uintptr_t>((value << 3) + p.coset_base + static_cast<uint32_t>(field) * 2u * kSymFbStreamBytes));
  const uint32_t next = __umul24(entry.x, x >> PB) + at - (entry.y & 0xFFFFu);
  p.e[field] = entry.x;
  p.ey[field] = entry.y;
  p.x = (!MASKED || valid_lane) ? next : x;
  uint32_t t, d, na, nb;
  uint32_t pos = uniform(p.pos);
  if constexpr (MASKED) {
    asm volatile(EP_ASM_VOTE("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_VCC("0")
                 : [x0] "+v"(p.x), [pos0] "+s"(pos), [t0] "=&v"(t), [d0] "=&v"(d), [na] "=&s"(na), [nb] "=&s"(nb)
                 : [ring0] "v"(p.ring), [shv] "v"(k.shv)
                 : "vcc", "scc", "memory");
  } else {
    asm volatile(EP_ASM_VOTE("0") "s_waitcnt lgkmcnt(0)\n" EP_ASM_TAKE_EXEC_VCC("0") EP_ASM_RESTORE_FULL
                 : [x0] "+v"(p.x), [pos0] "+s"(pos), [t0] "=&v"(t), [d0] "=&v"(d), [na] "=&s"(na), [nb] "=&s"(nb)
                 : [ring0] "v"(p.ring), [shv] "v"(k.shv)
                 : "vcc", "scc", "memory");
  }
  p.pos = pos;
}

// (half in the high 16 bits of `packed`) * b in float32 with one rounding: v_fma_mix_f32 reads the half-precision
// operand where it lies, so a value the table holds in that form costs no conversion.
__device__ __forceinline__ float mul_high_half(uint32_t packed, float b) {
  float r;
  asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "v"(b));
  return r;
}
// The same for a half in the low 16 bits.
__device__ __forceinline__ float mul_low_half(uint32_t packed, float b) {
  float r;
  asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "v"(b));
  return r;
}
// fma(half in the low 16 bits of `packed`, 2, addend)
__device__ __forceinline__ float twice_low_half_plus(uint32_t packed, float addend) {
  float r;
  asm("v_fma_mix_f32 %0, %1, 2.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "v"(addend));
  return r;
}
// fma(half in the high 16 bits of `packed`, 2, half in the high 16 bits of `addend`)
__device__ __forceinline__ float twice_high_half_plus(uint32_t packed, uint32_t addend) {
  float r;
  asm("v_fma_mix_f32 %0, %1, 2.0, %2 op_sel:[1,0,1] op_sel_hi:[1,0,1]" : "=v"(r) : "v"(packed), "v"(addend));
  return r;
}

// ---- payload windows ---------------------------------------------------------------------------------------------------

__device__ __forceinline__ void lds_store32(uint32_t at, uint32_t value) {
  *reinterpret_cast<__attribute__((address_space(3))) uint32_t*>(static_cast<uintptr_t>(at)) = value;
}

// Opens the window of each half's stream, words [word_begin, word_end) of `payload` (per-half values; lanes of a
// half agree; `live` = the half has a stream): fills the 128 LDS words at `window_at` with the stream's last one or
// two 64-word chunks, requests the 64 words below them, and sets the biased positions and the bookkeeping the
// end-of-stream check needs.
//
// Prefetches address the payload as one wave-uniform origin plus a 32-bit byte offset per lane, the form that
// costs no address arithmetic. The origin lies three chunks below the lower live stream's first chunk (or at the
// payload's start): lower than anything a valid stream consumes. Offsets saturate at the origin, so requests that
// reach further down (the last ones of a stream always do) re-read the origin chunk, and those words are never used.
// `readable` points at four readable bytes that stand in for a payload of fewer than two words.
__device__ __forceinline__ void open_window(Pair& s, uint32_t window_at, uint32_t word_begin, uint32_t word_end, bool live,
                                            const uint16_t* __restrict__ payload, uint64_t payload_words, const void* readable,
                                            int l32) {
  s.ring = window_at / 2u - kPosBias;                    // positions are kept biased, see Pair::pos
  const uint32_t base = word_begin & ~63u;               // absolute index of relative position 0
  const int begin = static_cast<int>(word_begin - base);
  const int ptr = static_cast<int>(word_end - base);
  const int low = (ptr & ~63) - 64;                       // the window holds relative [low, low + 128)
  s.ring_lane = window_at + 4u * static_cast<uint32_t>(l32);
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int64_t at = static_cast<int64_t>(base) + low + 64 * c + 2 * l32;
    uint32_t lo = 0, hi = 0;
    if (at >= 0 && static_cast<uint64_t>(at) < payload_words) lo = payload[at];
    if (at + 1 >= 0 && static_cast<uint64_t>(at + 1) < payload_words) hi = payload[at + 1];
    lds_store32(s.ring_lane + 128u * c, lo | (hi << 16));
  }
  const uint32_t floor_of = live ? (base >= 192u ? base - 192u : 0u) : ~0u;
  const uint32_t floor_a = __builtin_amdgcn_readlane(floor_of, 0), floor_b = __builtin_amdgcn_readlane(floor_of, 32);
  const uint32_t lowest = floor_a < floor_b ? floor_a : floor_b;
  const uint32_t origin_word = lowest == ~0u ? 0u : lowest;
  s.origin = payload_words >= 2 ? reinterpret_cast<const uint8_t*>(payload) + 2ull * origin_word : static_cast<const uint8_t*>(readable);
  const int64_t wanted = 2 * (static_cast<int64_t>(base) + low - 64 - static_cast<int64_t>(origin_word)) + 4 * l32;
  s.fetch_at = live && wanted > 0 ? static_cast<uint32_t>(wanted) : 0u;
  s.prefetch = *reinterpret_cast<const uint32_t*>(s.origin + s.fetch_at);
  const int p = ptr - low + static_cast<int>(kPosBias);  // position in [64, 128), stored biased
  s.pos = static_cast<uint32_t>(__builtin_amdgcn_readlane(p, 0)) | (static_cast<uint32_t>(__builtin_amdgcn_readlane(p, 32)) << 16);
  s.slid = 0;
  s.windowA = __builtin_amdgcn_readlane(low, 0);
  s.windowB = __builtin_amdgcn_readlane(low, 32);
  s.beginA = __builtin_amdgcn_readlane(begin, 0);
  s.beginB = __builtin_amdgcn_readlane(begin, 32);
}

// After a step (or two): a half whose position fell below 64 slides its window down by 64 words, and the other half
// slides along if it can (its position is below 128, so that it stays inside the 192-word window afterwards): the two
// streams of a wave are consumed at about the same rate, so this keeps their slides together, one event and one
// request for both instead of two. All 32 lanes of a sliding half (voting or not) move their dwords of the two lower
// chunks up, drop their prefetched dword in the lowest and ask for the next 64 words down. Which halves slide is a
// scalar decision, and the lanes are picked by a mask built from it; the scalar side is kept short (it is what the
// common, non-sliding case pays for: three instructions).
__device__ __forceinline__ void slide_window(Pair& s) {
  const uint32_t low_bits = ~s.pos & 0x00800080u;        // bit 7 of a biased field clear <=> that position < 64
  if (__builtin_expect(low_bits != 0, 0)) {
    asm volatile("" ::: "memory");     // keep this a scalar branch: the common case must cost no vector work
    const uint32_t sliding = ~(s.pos & (s.pos << 1)) & 0x00800080u;    // bits 7 and 6 not both set <=> position < 128
    const uint32_t lower = static_cast<uint32_t>(static_cast<int32_t>(sliding << 24) >> 31);
    const uint32_t upper = static_cast<uint32_t>(static_cast<int32_t>(sliding << 8) >> 31);
    if (__builtin_amdgcn_inverse_ballot_w64(static_cast<uint64_t>(lower) | (static_cast<uint64_t>(upper) << 32))) {
      typedef __attribute__((address_space(3))) uint32_t* lds_u32;
      const uint32_t kept0 = *reinterpret_cast<lds_u32>(static_cast<uintptr_t>(s.ring_lane));
      const uint32_t kept1 = *reinterpret_cast<lds_u32>(static_cast<uintptr_t>(s.ring_lane + 128u));
      lds_store32(s.ring_lane + 256u, kept1);
      lds_store32(s.ring_lane + 128u, kept0);
      lds_store32(s.ring_lane, s.prefetch);
      s.fetch_at = s.fetch_at >= 128u ? s.fetch_at - 128u : 0u;
      s.prefetch = *reinterpret_cast<const uint32_t*>(s.origin + s.fetch_at);
    }
    s.pos += sliding >> 1;              // + 64 in the fields that slid
    s.slid += sliding;                  // one more slide for them
  }
}

// Where each half's stream stands, relative to the same base as Pair::beginA / beginB.
__device__ __forceinline__ int window_pointer_a(const Pair& s) {
  return s.windowA - 64 * static_cast<int>((s.slid >> 7) & 0xFFFFu) + static_cast<int>(s.pos & 0xFFFFu) - static_cast<int>(kPosBias);
}
__device__ __forceinline__ int window_pointer_b(const Pair& s) {
  return s.windowB - 64 * static_cast<int>(s.slid >> 23) + static_cast<int>(s.pos >> 16) - static_cast<int>(kPosBias);
}

// One 16-byte store of a bf16 vector, streaming or through the cache as the container's tile length asks. Written as
// two instructions the compiler cannot merge: given two ordinary stores of one value to one address on the two sides of
// a branch it keeps a single store and drops the streaming hint. (A store the compiler does not know about only makes
// its later waits on the memory counter stricter.)
typedef uint32_t lds_store_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_bf16_vector(lds_store_u32x4* to, lds_store_u32x4 value, bool through_cache) {
  if (through_cache) asm volatile("global_store_dwordx4 %0, %1, off" ::"v"(to), "v"(value) : "memory");
  else asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(to), "v"(value) : "memory");
}

// ---- the kernel ------------------------------------------------------------------------------------------------------

// A wave alternates between a chain of dependent symbol steps, where every instruction waits for the one before, and a
// burst of independent work (reconstruction, products, the store). The chain runs at the higher wave priority: the
// bursts of a SIMD's other waves then fill the issue slots that its chains leave open instead of delaying them.
__device__ __forceinline__ void chain_priority() { __builtin_amdgcn_s_setprio(1); }
__device__ __forceinline__ void emit_priority() { __builtin_amdgcn_s_setprio(0); }

template <int PB, int MODE, int ILP, int KIND>
__device__ __forceinline__ void decode_lds_body(const DecodeArgs& a, int pair_begin, int pair_end, int pair_stride) {
  extern __shared__ __align__(16) uint8_t smem[];
  using L = Layout<PB, MODE>;
  constexpr bool WIDE = MODE == kModeWide || MODE == kModeRank;    // symbols as integers, not as biased bytes in bits 24..31
  static_assert((MODE != kModeRank && MODE != kModeSym) || ILP == 1, "the rank/select and two-level steps are single-pair");
  const uint32_t lut_bytes = MODE == kModeRank ? (a.lut_bytes + 255u) / 256u * 256u
                                               : (MODE == kModeSym ? static_cast<uint32_t>(sym_table_bytes(PB)) : L::kLutBytes);
  typedef __attribute__((address_space(3))) uint8_t* lds_ptr;

  const int waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));   // uniform for the compiler too
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  // Absolute LDS byte addresses: tables first (so that table bases have their low 13 bits clear), then the rings.
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr)smem));
  const uint32_t rings0 = lds0 + lut_bytes;
  const uint32_t minima0 = rings0 + static_cast<uint32_t>(waves) * ILP * 2 * kRingBytes;

  if (lds0 != 0) {      // the steps address the tables from LDS offset 0 and OR table bases into slot offsets
    if (threadIdx.x == 0) flag_error(a.error, EP_DECODE_BAD_OFFSETS);
    return;
  }
  // Staging the tables. The slot-table forms are whole KiB: they are loaded straight into LDS (one wave instruction
  // moves 1 KiB, lane l the 16 bytes at 16 l, no registers in between), and the loads are left in flight while the
  // wave sets its first tiles up (offsets, states and payload chunks: two dependent trips to memory); the wait and the
  // barrier that publish the tables come after that set-up, inside the loop below. The rank/select tables have any
  // multiple of 16 bytes and are copied through registers.
  constexpr bool kStageDirect = MODE != kModeRank;
  {
    const uint8_t* src = MODE == kModeSym ? a.sym_tables : reinterpret_cast<const uint8_t*>(a.plan) + kHeaderBytes;
    if (threadIdx.x < kStreams) {
      reinterpret_cast<int32_t*>(smem + lut_bytes + static_cast<uint32_t>(waves) * ILP * 2 * kRingBytes)[threadIdx.x] =
          static_cast<int32_t>(a.plan[kHdrSymMin + threadIdx.x]);
    }
    if constexpr (kStageDirect) {
      static_assert(L::kLutBytes % 1024 == 0 && sym_table_bytes(PB) % 1024 == 0, "slot tables are whole KiB");
      for (uint32_t kib = static_cast<uint32_t>(wave); kib < lut_bytes / 1024u; kib += static_cast<uint32_t>(waves)) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + kib * 1024u + static_cast<uint32_t>(lane) * 16u),
                                         (__attribute__((address_space(3))) void*)(smem + kib * 1024u), 16, 0, 0);
      }
    } else {
      const uint4* from = reinterpret_cast<const uint4*>(src);
      uint4* dst = reinterpret_cast<uint4*>(smem);
      for (uint32_t i = threadIdx.x; i < a.lut_bytes / 16; i += blockDim.x) dst[i] = from[i];
    }
  }
  bool tables_published = false;
  auto publish_tables = [&]() {
    if (!tables_published) {
      __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): this wave's part of the tables has landed
      __syncthreads();
      tables_published = true;
    }
  };

  StepConsts k;
  k.f0s = uniform(a.plan[kHdrCosetFreq0]);
  k.f0v = k.f0s;
  k.f1v = L::kTable - k.f0s;
  // Byte distance between a field's two cosets, in the table the coset offset is added to.
  k.ktab = MODE == kModeRank ? (L::kTable / 32u) * 8u : (MODE == kModeSym ? static_cast<uint32_t>(kSymFbStreamBytes) : L::kTableBytes);
  const uint32_t rank_val0 = uniform(a.rank_val_offset), rank_rs0 = uniform(a.rank_rs_offset);
  // Rank/select tables with half-precision values (the usual case): reconstruction as for the two-level tables.
  const bool rank_half = MODE == kModeRank && uniform(a.rank_half) != 0;
  const uint32_t rank_freq_width = rank_half ? 15u : 16u;
  k.shv = half ? 16u : 0u;
  // Keep the per-lane constants in vector registers (the steps name them as VGPR operands).
  asm volatile("" : "+v"(k.f0v), "+v"(k.f1v), "+v"(k.ktab), "+v"(k.shv));
  const uint64_t all_lanes = ~0ull;

  for (int first_pair = pair_begin + wave * ILP; first_pair < pair_end; first_pair += pair_stride) {
    Pair st[ILP];
    bool full = true;

    // ---- set up each tile: positions, initial states, the ring's two chunks, the first prefetch ---------------------
#pragma unroll
    for (int j = 0; j < ILP; ++j) {
      Pair& s = st[j];
      const int64_t tile = 2 * static_cast<int64_t>(first_pair + j) + half;
      const uint32_t window_at = rings0 + static_cast<uint32_t>((wave * ILP + j) * 2 + half) * kRingBytes;
      uint32_t word_begin = 0, word_end = 0;
      s.count = 0;
      s.x = kStateMin;
      s.vector0 = 0;
      s.coset_base = 0;
      s.coset_mask = 0;
      s.dot_row = -1;
#pragma unroll
      for (int m = 0; m < kDotRows; ++m) s.dot_acc[m] = 0.0f;
      if (first_pair + j < pair_end && tile < a.num_tiles) {
        word_begin = a.offsets[tile];
        word_end = a.offsets[tile + 1];
        const int64_t v0 = tile * a.tile_vectors;
        const int64_t left = a.num_vectors - v0;
        s.vector0 = static_cast<uint32_t>(v0);
        s.count = static_cast<int>(left < a.tile_vectors ? left : a.tile_vectors);
        if (word_begin > word_end || word_end > a.payload_words) {
          flag_error(a.error, EP_DECODE_BAD_OFFSETS);
          s.count = 0;
          word_begin = word_end = 0;
        } else {
          s.x = a.states[tile * kStatesPerTile + l32];
        }
      }
      full = full && s.count == a.tile_vectors;
      open_window(s, window_at, word_begin, word_end, s.count > 0, a.payload, a.payload_words, a.offsets, l32);
    }
    const bool all_full = __builtin_amdgcn_readfirstlane(__all(full) ? 1 : 0) != 0;
    publish_tables();

    // After a step: a half whose position fell below 64 slides its window down by 64 words. All 32 lanes of the half
    // (voting or not) move their dword of the lower chunk up, drop their prefetched dword in its place and ask for
    // the next 64 words down.
    auto top_up = [&](Pair& s) { slide_window(s); };

    // E8 point and row scale of the vector each valid lane just decoded. The reference forms (z + c / 2) * scale with
    // one rounding. For an ordinary scale (positive, neither tiny nor huge) fma(z, scale, c * scale / 2) is the same
    // number rounded once, c * scale / 2 being exact, and costs one instruction per weight less. Any other scale
    // (zero, negative: the sign of a zero weight; subnormal; beyond 1e30: bf16 saturation) takes the literal form.
    auto lattice_point = [&](const Pair& s, float (&z)[8]) {
      if constexpr (MODE == kModeSym) {
        // The entries hold the coordinates, coset shift included, in half precision (second word, high half); the first
        // words' high halves XOR to the parity of z0..z6 as a half-precision 0.0 or 1.0.
        const uint32_t folded = xor3(xor3(s.e[0], s.e[1], s.e[2]), xor3(s.e[3], s.e[4], s.e[5]), s.e[6]);
#pragma unroll
        for (int f = 0; f < 7; ++f) z[f] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(s.ey[f] >> 16)));
        z[7] = twice_high_half_plus(s.ey[7], folded);
      } else if constexpr (!WIDE) {
        // Top byte = the value as a signed byte; the parity of z0..z6 is the parity of those bytes.
        const uint32_t folded = xor3(xor3(s.e[0], s.e[1], s.e[2]), xor3(s.e[3], s.e[4], s.e[5]), s.e[6]);
        const float parity = static_cast<float>((folded >> 24) & 1u);
#pragma unroll
        for (int f = 0; f < 8; ++f) z[f] = static_cast<float>(static_cast<int32_t>(s.e[f]) >> 24);
        z[7] = __fmaf_rn(z[7], 2.0f, parity);
      } else if (MODE == kModeRank && rank_half) {
        // The values are the coordinates, coset shift included, in half precision; bit 31 of an entry marks an odd value.
        const uint32_t folded = xor3(xor3(s.ey[0], s.ey[1], s.ey[2]), xor3(s.ey[3], s.ey[4], s.ey[5]), s.ey[6]);
#pragma unroll
        for (int f = 0; f < 7; ++f) z[f] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(s.e[f])));
        z[7] = twice_low_half_plus(s.e[7], static_cast<float>(folded >> 31));
      } else {
        const bool c = s.coset_base != 0;
        const int32_t* minima = reinterpret_cast<const int32_t*>(smem + (minima0 - lds0)) + 1 + (c ? 1 : 0);
        int v[8];
#pragma unroll
        for (int f = 0; f < 8; ++f) {
          if constexpr (MODE == kModeRank) v[f] = static_cast<int16_t>(s.e[f]);
          else v[f] = static_cast<int>(s.e[f] >> L::kSymShift) + minima[2 * f];
        }
        const int parity = (v[0] + v[1] + v[2] + v[3] + v[4] + v[5] + v[6]) & 1;
        v[7] = 2 * v[7] + parity;
#pragma unroll
        for (int f = 0; f < 8; ++f) z[f] = static_cast<float>(v[f]);
      }
    };
    // w = fma(z, scale, shift) for an ordinary scale. The two-level tables hold z + c / 2 itself in half precision, so
    // there the weight is one product, literally the reference's (z + c / 2) * scale, and `shift` is not used.
    auto scaled_point = [&](const Pair& s, float scale, float shift, float (&w)[8]) {
      if constexpr (MODE == kModeSym) {
        const uint32_t folded = xor3(xor3(s.e[0], s.e[1], s.e[2]), xor3(s.e[3], s.e[4], s.e[5]), s.e[6]);
#pragma unroll
        for (int f = 0; f < 7; ++f) w[f] = mul_high_half(s.ey[f], scale);
        w[7] = __fmul_rn(twice_high_half_plus(s.ey[7], folded), scale);
      } else if (MODE == kModeRank && rank_half) {
        const uint32_t folded = xor3(xor3(s.ey[0], s.ey[1], s.ey[2]), xor3(s.ey[3], s.ey[4], s.ey[5]), s.ey[6]);
#pragma unroll
        for (int f = 0; f < 7; ++f) w[f] = mul_low_half(s.e[f], scale);
        w[7] = __fmul_rn(twice_low_half_plus(s.e[7], static_cast<float>(folded >> 31)), scale);
      } else {
        float z[8];
        lattice_point(s, z);
#pragma unroll
        for (int f = 0; f < 8; ++f) w[f] = __fmaf_rn(z[f], scale, shift);
      }
    };
    auto weights_of = [&](const Pair& s, float scale, float (&w)[8]) {
      const bool c = s.coset_base != 0;
      // 1e-30 <= scale <= 1e30 as one unsigned comparison of the bit patterns (fails for negative values and NaN).
      const bool ordinary = __float_as_uint(scale) - 0x0DA24260u <= 0x7149F2CAu - 0x0DA24260u;
      if (__builtin_expect(ordinary, 1)) {
        scaled_point(s, scale, c ? __fmul_rn(scale, 0.5f) : 0.0f, w);
      } else {
        float z[8];
        lattice_point(s, z);
        const float shift = MODE != kModeSym && !rank_half && c ? 0.5f : 0.0f;       // half-precision table values include it
#pragma unroll
        for (int f = 0; f < 8; ++f) w[f] = __fmul_rn(__fadd_rn(z[f], shift), scale);
      }
    };

    // bf16 pairs of a vector's weights, rounded to nearest even, saturated like the reference's CPU lane.
    auto pack_bf16 = [&](float (&w)[8], float scale, uint32_t (&packed)[4]) {
      // |w| can pass the largest finite bf16 only for scales beyond 1e30; the reference's CPU lane saturates.
      if (__builtin_fabsf(scale) > 1.0e30f) {
#pragma unroll
        for (int f = 0; f < 8; ++f) w[f] = clamp_bf16(w[f]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        typedef float float2v __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const float2v two = {w[2 * i], w[2 * i + 1]};
        packed[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(two, bf16x2));
      }
    };

    auto emit = [&](const Pair& s, uint32_t vector, float scale) {
      float w[8];
      weights_of(s, scale, w);
      if constexpr (KIND == EP_STORE_BF16) {
        uint32_t packed[4];
        pack_bf16(w, scale, packed);
        // Streaming store: the dense weight is written once and not read back by this kernel, and waves must not
        // queue behind write-allocate traffic when they next wait on their payload prefetch (store_cached: see below).
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 quad = {packed[0], packed[1], packed[2], packed[3]};
        store_bf16_vector(reinterpret_cast<u32x4*>(a.out) + vector, quad, a.store_cached != 0);
      } else if constexpr (KIND == EP_STORE_I8) {
        store_vector_i8(a.out, vector, w);
      } else {
        store_vector(a.out, a.store_kind, vector, w);
      }
    };


    // ---- multiply on the fly: y32[m][row] += sum_k w[row][k] x[m][k], the dense weight never reaches memory -----------
    //
    // Every lane multiplies the vector it just decoded (rounded to bf16 exactly as the store would) with the matching
    // eight activations of each row m and adds the result to a per-lane partial sum. All 32 vectors of a group lie in
    // one weight row, or in two when a row ends inside the group (rows are at least 32 vectors long here). A half's
    // partial sums therefore belong to one row; when a group brings a different one they are reduced over the half
    // and added to y32 with one atomic per activation row.
    constexpr int DOT_ROWS = KIND == kKindDot1 ? 1 : (KIND == kKindDot4 ? kDotRows : 0);
    struct DotInput {
      int row;
      uint4 x[DOT_ROWS > 0 ? DOT_ROWS : 1];
    };
    auto dot_prefetch = [&](uint32_t vector, uint32_t row, bool valid_lane, DotInput& in) {
      in.row = static_cast<int>(row);
      const uint32_t in_row = vector - row * static_cast<uint32_t>(a.vecs_per_row);
#pragma unroll
      for (int m = 0; m < DOT_ROWS; ++m) {
        in.x[m] = make_uint4(0, 0, 0, 0);
        if (valid_lane && m < a.m_rows) in.x[m] = *reinterpret_cast<const uint4*>(a.x + static_cast<int64_t>(m) * a.ldx + static_cast<int64_t>(in_row) * 8);
      }
    };
    auto half_sum = [](float v) {
#pragma unroll
      for (int d = 16; d >= 1; d >>= 1) v += __shfl_xor(v, d);     // partners differ below bit 5: never across halves
      return v;
    };
    auto dot_add = [&](int m, int row, float value) {
      if (l32 == 0 && row >= 0) unsafeAtomicAdd(a.y32 + static_cast<int64_t>(m) * a.ldy32 + row, value);
    };
    auto dot_emit = [&](Pair& s, float scale, bool valid_lane, const DotInput& in) {
      float w[8];
      uint32_t packed[4];
      weights_of(s, scale, w);
      pack_bf16(w, scale, packed);
      float dot[DOT_ROWS > 0 ? DOT_ROWS : 1];
#pragma unroll
      for (int m = 0; m < DOT_ROWS; ++m) {
        // Two bf16 products and the running sum per instruction (v_dot2_f32_bf16): the operands are used as they lie,
        // packed in pairs, instead of being widened to float32 one by one.
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const uint32_t xw[4] = {in.x[m].x, in.x[m].y, in.x[m].z, in.x[m].w};
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed[i]), __builtin_bit_cast(bf16x2, xw[i]), sum, false);
        }
        dot[m] = valid_lane ? sum : 0.0f;
      }
      const uint64_t moved = __builtin_amdgcn_ballot_w64(valid_lane && in.row != s.dot_row);
      if (__builtin_expect(moved == 0, 1)) {
#pragma unroll
        for (int m = 0; m < DOT_ROWS; ++m) s.dot_acc[m] += dot[m];
        return;
      }
      // Valid lanes are a prefix of each half. low / high: the rows of its first and last valid lane.
      const uint64_t valid = __builtin_amdgcn_ballot_w64(valid_lane);
      const int count_a = __builtin_popcount(static_cast<uint32_t>(valid)), count_b = __builtin_popcount(static_cast<uint32_t>(valid >> 32));
      const int low_a = __builtin_amdgcn_readlane(in.row, 0), low_b = __builtin_amdgcn_readlane(in.row, 32);
      const int high_a = __builtin_amdgcn_readlane(in.row, count_a > 0 ? count_a - 1 : 0);
      const int high_b = __builtin_amdgcn_readlane(in.row, 32 + (count_b > 0 ? count_b - 1 : 0));
      const bool any = (half ? count_b : count_a) > 0;
      const int low = half ? low_b : low_a, high = half ? high_b : high_a;
      const bool keep = valid_lane && in.row == s.dot_row;
      const bool fresh = valid_lane && !keep && in.row == low;
      const bool stray = valid_lane && !keep && in.row != low;       // the group's second row, when it is not the carried one
#pragma unroll
      for (int m = 0; m < DOT_ROWS; ++m) {
        if (m >= a.m_rows) break;
        dot_add(m, s.dot_row, half_sum(s.dot_acc[m] + (keep ? dot[m] : 0.0f)));
        const float second = half_sum(stray ? dot[m] : 0.0f);
        if (any && high != low && high != s.dot_row) dot_add(m, high, second);
        s.dot_acc[m] = fresh ? dot[m] : 0.0f;
      }
      s.dot_row = any ? low : -1;
    };

    using Masked = std::integral_constant<bool, true>;
    using Unmasked = std::integral_constant<bool, false>;

    // The nine steps of a group for the wave's pairs in lock step, windows kept filled. `valid` is the wave's lane mask.
    // A window is checked (and slid) after every second step: a step consumes at most 32 words per half and a check
    // leaves at least 64 in the window. The checks sit after fields 0, 2, 4, 6 and after the group's last step.
    auto group_steps = [&](auto masked_tag, bool valid_lane, uint64_t valid) {
      constexpr bool MASKED = decltype(masked_tag)::value;
      if constexpr (ILP == 2) coset_step_dual<PB, MODE, MASKED>(st[0], st[ILP - 1], k, valid);
      else coset_step_single<PB, MODE, MASKED>(st[0], k, valid);
      uint32_t high[ILP];
#pragma unroll
      for (int j = 0; j < ILP; ++j) high[j] = st[j].coset_base + L::kHighBase;
      const uint32_t rank_group = st[0].coset_base + rank_rs0;
#pragma unroll
      for (int f = 0; f < kFields; ++f) {
        if constexpr (MODE == kModeRank) {
          rank_step<PB, MASKED>(st[0], f, rank_group, rank_val0, rank_freq_width, k, valid_lane);
        } else if constexpr (MODE == kModeSym) {
          sym_step<PB, MASKED>(st[0], f, k, valid_lane);
        } else if constexpr (ILP == 2) {
          field_step_dual<PB, MODE, MASKED>(st[0], st[ILP - 1], f, f & 3, f < 4 ? st[0].coset_base : high[0],
                                            f < 4 ? st[ILP - 1].coset_base : high[ILP - 1], k, valid);
        } else {
          field_step_single<PB, MODE, MASKED>(st[0], f, f & 3, f < 4 ? st[0].coset_base : high[0], k, valid);
        }
        if ((f & 1) == 0 || f == kFields - 1) {
#pragma unroll
          for (int j = 0; j < ILP; ++j) top_up(st[j]);
        }
      }
    };

    // The whole groups of a wave of full tiles (all lanes valid) carry the row's scale from group to group: a lane's
    // vectors walk down through its tile 32 at a time and change rows rarely. Positions are kept relative to the
    // pair's lower tile, in units of one bf16 vector's bytes: the same number is the lane's store offset from a
    // wave-uniform address and, compared with where the lane's current row begins, says when that row is left.
    struct RowCursor {
      int32_t row_begin;      // position of the first vector of the lane's row (INT32_MIN: at or below the pair's first)
      float scale, half_scale;
      uint64_t unusual;       // wave-uniform: lanes whose scale needs the literal formula
    };
    auto lower_tile_of = [&](int j) { return static_cast<uint32_t>(2 * static_cast<int64_t>(first_pair + j) * a.tile_vectors); };

    // One group of 32 vectors per half; every lane looks its row and scale up.
    auto group_dual = [&](auto masked_tag, int offset, bool valid_lane, uint64_t valid) {
      uint32_t vector[ILP];
      float scale[ILP];
      DotInput dot_in[ILP];
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        vector[j] = st[j].vector0 + static_cast<uint32_t>(offset) + l32;
        const uint32_t row = row_of(a, vector[j]);
        scale[j] = valid_lane ? a.scales[row] : 0.0f;
        if constexpr (DOT_ROWS > 0) dot_prefetch(vector[j], row, valid_lane, dot_in[j]);
      }
      chain_priority();
      group_steps(masked_tag, valid_lane, valid);
      emit_priority();
      if constexpr (DOT_ROWS > 0) {
#pragma unroll
        for (int j = 0; j < ILP; ++j) dot_emit(st[j], scale[j], valid_lane, dot_in[j]);
      } else if (valid_lane) {
#pragma unroll
        for (int j = 0; j < ILP; ++j) emit(st[j], vector[j], scale[j]);
      }
    };

    // A whole group on the carried scales. A lane that has left its row makes the wave look its rows up first.
    RowCursor cursor[ILP];
    const uint32_t lane_at = 16u * (static_cast<uint32_t>(half ? a.tile_vectors : 0) + static_cast<uint32_t>(l32));
#pragma unroll
    for (int j = 0; j < ILP; ++j) cursor[j] = RowCursor{0x7FFFFFFF, 0.0f, 0.0f, 0};
    auto group_tracked = [&](int offset) {
      const uint32_t at = lane_at + 16u * static_cast<uint32_t>(offset);
      bool left = false;
#pragma unroll
      for (int j = 0; j < ILP; ++j) left = left || static_cast<int32_t>(at) < cursor[j].row_begin;
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(left) != 0, 0)) {
#pragma unroll
        for (int j = 0; j < ILP; ++j) {
          const uint32_t row = row_of(a, lower_tile_of(j) + (at >> 4));
          const float scale = a.scales[row];
          const int64_t begins = static_cast<int64_t>(row) * a.vecs_per_row - lower_tile_of(j);
          cursor[j].row_begin = begins > 0 ? static_cast<int32_t>(begins * 16) : static_cast<int32_t>(0x80000000u);
          cursor[j].scale = scale;
          cursor[j].half_scale = __fmul_rn(scale, 0.5f);
          cursor[j].unusual = __builtin_amdgcn_ballot_w64(!(__float_as_uint(scale) - 0x0DA24260u <= 0x7149F2CAu - 0x0DA24260u));
        }
      }
      chain_priority();
      group_steps(Unmasked{}, true, all_lanes);
      emit_priority();
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        const RowCursor& c = cursor[j];
        const Pair& s = st[j];
        float w[8];
        if (__builtin_expect(c.unusual == 0, 1)) {
          scaled_point(s, c.scale, __builtin_amdgcn_inverse_ballot_w64(s.coset_mask) ? c.half_scale : 0.0f, w);
        } else {
          weights_of(s, c.scale, w);
        }
        if constexpr (KIND == EP_STORE_BF16) {
          uint32_t packed[4];
          if (__builtin_expect(c.unusual == 0, 1)) pack_bf16(w, 1.0f, packed);     // an ordinary scale never saturates
          else pack_bf16(w, c.scale, packed);
          typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
          const u32x4 quad = {packed[0], packed[1], packed[2], packed[3]};
          uint8_t* lower_out = static_cast<uint8_t*>(a.out) + 16ull * lower_tile_of(j);
          // Streaming stores, except for tiles whose length is no multiple of four vectors (store_cached): their groups
          // share 64-byte pieces with the neighbouring groups, and pieces written through the cache meet there.
          if (a.store_cached) asm volatile("global_store_dwordx4 %0, %1, %2" ::"v"(at), "v"(quad), "s"(lower_out) : "memory");
          else asm volatile("global_store_dwordx4 %0, %1, %2 nt" ::"v"(at), "v"(quad), "s"(lower_out) : "memory");
        } else if constexpr (KIND == EP_STORE_I8) {
          store_vector_i8(a.out, lower_tile_of(j) + (at >> 4), w);
        } else {
          store_vector(a.out, a.store_kind, lower_tile_of(j) + (at >> 4), w);
        }
      }
    };

    // The same for one pair on its own lane mask (waves that hold the container's last, short or missing tiles).
    auto group_single = [&](Pair& s, int offset, bool valid_lane) {
      const uint64_t valid = __builtin_amdgcn_ballot_w64(valid_lane);
      const uint32_t vector = s.vector0 + static_cast<uint32_t>(offset) + l32;
      const uint32_t row = row_of(a, vector);
      const float scale = valid_lane ? a.scales[row] : 0.0f;
      DotInput dot_in;
      if constexpr (DOT_ROWS > 0) dot_prefetch(vector, row, valid_lane, dot_in);
      chain_priority();
      coset_step_single<PB, MODE, true>(s, k, valid);
      const uint32_t high = s.coset_base + L::kHighBase;
#pragma unroll
      for (int f = 0; f < kFields; ++f) {
        if constexpr (MODE == kModeRank) {
          rank_step<PB, true>(s, f, s.coset_base + rank_rs0, rank_val0, rank_freq_width, k, valid_lane);
        } else if constexpr (MODE == kModeSym) {
          sym_step<PB, true>(s, f, k, valid_lane);
        } else {
          field_step_single<PB, MODE, true>(s, f, f & 3, f < 4 ? s.coset_base : high, k, valid);
        }
        if ((f & 1) == 0 || f == kFields - 1) top_up(s);
      }
      emit_priority();
      if constexpr (DOT_ROWS > 0) dot_emit(s, scale, valid_lane, dot_in);
      else if (valid_lane) emit(s, vector, scale);
    };

    if (all_full) {
      // Every tile of this wave is full: one schedule for all halves. The short first group, then whole groups.
      const int rem = a.tile_vectors & 31;
      int offset = a.tile_vectors - rem;
      if (rem != 0) {
        const bool valid_lane = l32 < rem;
        group_dual(Masked{}, offset, valid_lane, __builtin_amdgcn_ballot_w64(valid_lane));
      }
      // Nothing read so far may still be in flight when the loop starts: the compiler would otherwise wait for it
      // inside the loop, on every pass, and each such wait also covers the loop's own newest payload request.
      __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0)
#pragma unroll 1
      while (offset > 0) {
        offset -= 32;
        if constexpr (DOT_ROWS == 0) group_tracked(offset);
        else group_dual(Unmasked{}, offset, true, all_lanes);
      }
    } else {
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        Pair& s = st[j];
        const int groups = (s.count + 31) >> 5;
        const int other = __shfl_xor(groups, 32);
        const int rounds = __builtin_amdgcn_readfirstlane(groups > other ? groups : other);
        const int rem = s.count & 31;
#pragma unroll 1
        for (int round = 0; round < rounds; ++round) {
          const int lanes = (round == 0 && rem != 0) ? rem : 32;
          group_single(s, (groups - 1 - round) << 5, round < groups && l32 < lanes);
        }
      }
    }

    if constexpr (DOT_ROWS > 0) {
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
#pragma unroll
        for (int m = 0; m < DOT_ROWS; ++m) {
          if (m < a.m_rows) dot_add(m, st[j].dot_row, half_sum(st[j].dot_acc[m]));
        }
      }
    }

    // A valid tile ends with every word consumed and every lane back at the encoder's initial state.
#pragma unroll
    for (int j = 0; j < ILP; ++j) {
      const Pair& s = st[j];
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
  }
  publish_tables();      // a wave without tiles still takes part in the workgroup's barrier
}

// One container spread over the whole grid.
template <int PB, int MODE, int ILP, int KIND>
__global__ __launch_bounds__(1024) void decode_lds_kernel(DecodeArgs a, int num_pairs) {
  const int per_block = static_cast<int>(blockDim.x >> 6) * ILP;
  decode_lds_body<PB, MODE, ILP, KIND>(a, static_cast<int>(blockIdx.x) * per_block, num_pairs, static_cast<int>(gridDim.x) * per_block);
}

// The rank/select tables are small enough for two workgroups per CU; eight waves per SIMD need at most 64 registers.
template <int PB, int KIND>
__global__ __launch_bounds__(1024, 8) void decode_rank_kernel(DecodeArgs a, int num_pairs) {
  const int per_block = static_cast<int>(blockDim.x >> 6);
  decode_lds_body<PB, kModeRank, 1, KIND>(a, static_cast<int>(blockIdx.x) * per_block, num_pairs, static_cast<int>(gridDim.x) * per_block);
}

// The two-level tables are a quarter of the byte form's: two workgroups per CU, at most 64 registers.
template <int PB, int KIND>
__global__ __launch_bounds__(1024, 8) void decode_sym_kernel(DecodeArgs a, int num_pairs) {
  const int per_block = static_cast<int>(blockDim.x >> 6);
  decode_lds_body<PB, kModeSym, 1, KIND>(a, static_cast<int>(blockIdx.x) * per_block, num_pairs, static_cast<int>(gridDim.x) * per_block);
}

// Batch: each block decodes its slice of one of many containers. The argument block is read with every word made
// wave-uniform, so that it lives in scalar registers exactly as kernel arguments do.
__device__ __forceinline__ DecodeArgs load_job(const DecodeArgs* __restrict__ jobs, const BlockJob& mine, uint8_t* arena) {
  static_assert(sizeof(DecodeArgs) % 4 == 0, "DecodeArgs is copied as 32-bit words");
  const uint32_t* src = reinterpret_cast<const uint32_t*>(jobs + uniform(static_cast<uint32_t>(mine.job)));
  uint32_t words[sizeof(DecodeArgs) / 4];
#pragma unroll
  for (unsigned i = 0; i < sizeof(DecodeArgs) / 4; ++i) words[i] = uniform(src[i]);
  DecodeArgs a;
  __builtin_memcpy(&a, words, sizeof(a));
  a.out = arena + reinterpret_cast<uintptr_t>(a.out);       // batch jobs carry the byte offset of their output
  return a;
}

template <int PB, int MODE, int ILP, int KIND>
__global__ __launch_bounds__(1024) void decode_lds_batch_kernel(const DecodeArgs* __restrict__ jobs,
                                                                const BlockJob* __restrict__ block_jobs, uint8_t* arena) {
  const BlockJob mine = block_jobs[blockIdx.x];
  const DecodeArgs a = load_job(jobs, mine, arena);
  const int first = static_cast<int>(uniform(static_cast<uint32_t>(mine.first_pair)));
  const int count = static_cast<int>(uniform(static_cast<uint32_t>(mine.n_pairs)));
  decode_lds_body<PB, MODE, ILP, KIND>(a, first, first + count, static_cast<int>(blockDim.x >> 6) * ILP);
}

template <int PB, int KIND>
__global__ __launch_bounds__(1024, 8) void decode_sym_batch_kernel(const DecodeArgs* __restrict__ jobs,
                                                                   const BlockJob* __restrict__ block_jobs, uint8_t* arena) {
  const BlockJob mine = block_jobs[blockIdx.x];
  const DecodeArgs a = load_job(jobs, mine, arena);
  const int first = static_cast<int>(uniform(static_cast<uint32_t>(mine.first_pair)));
  const int count = static_cast<int>(uniform(static_cast<uint32_t>(mine.n_pairs)));
  decode_lds_body<PB, kModeSym, 1, KIND>(a, first, first + count, static_cast<int>(blockDim.x >> 6));
}

template <int PB, int KIND>
__global__ __launch_bounds__(1024, 8) void decode_rank_batch_kernel(const DecodeArgs* __restrict__ jobs,
                                                                    const BlockJob* __restrict__ block_jobs, uint8_t* arena) {
  const BlockJob mine = block_jobs[blockIdx.x];
  const DecodeArgs a = load_job(jobs, mine, arena);
  const int first = static_cast<int>(uniform(static_cast<uint32_t>(mine.first_pair)));
  const int count = static_cast<int>(uniform(static_cast<uint32_t>(mine.n_pairs)));
  decode_lds_body<PB, kModeRank, 1, KIND>(a, first, first + count, static_cast<int>(blockDim.x >> 6));
}

// ---- host side: launching one instantiation ------------------------------------------------------------------------------

// Raises the dynamic LDS cap of `function` once per device (per instantiation and thread: `configured_for` is the
// caller's thread-local slot).
inline int allow_full_lds(const void* function, int& configured_for) {
  int device = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  if (configured_for != device) {
    EP_HIP_TRY(hipFuncSetAttribute(function, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    configured_for = device;
  }
  return EP_HIP_OK;
}

template <typename Single>
static int launch_single(Single single, int& configured_for, const LdsLaunch& cfg, const DecodeArgs& args, int num_pairs, hipStream_t stream) {
  const int status = allow_full_lds(reinterpret_cast<const void*>(single), configured_for);
  if (status != EP_HIP_OK) return status;
  hipLaunchKernelGGL(single, dim3(cfg.blocks), dim3(cfg.threads), cfg.lds_bytes, stream, args, num_pairs);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

template <typename Batch>
static int launch_batch(Batch batch, int& configured_for, const LdsLaunch& cfg, const DecodeArgs* jobs, const BlockJob* block_jobs,
                        uint8_t* arena, hipStream_t stream) {
  const int status = allow_full_lds(reinterpret_cast<const void*>(batch), configured_for);
  if (status != EP_HIP_OK) return status;
  hipLaunchKernelGGL(batch, dim3(cfg.blocks), dim3(cfg.threads), cfg.lds_bytes, stream, jobs, block_jobs, arena);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

}  // namespace ep
