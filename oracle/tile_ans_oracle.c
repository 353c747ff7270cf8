/* CPU oracle for the lossless tile_ans decode -- TEST INFRASTRUCTURE, not product code.
 *
 * The C twin of tile_ans_oracle.py (stream-parallel with OpenMP), fast enough to check the GPU on full-size
 * tensors and to serve as the timed CPU baseline. Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load the library built from this file; the shipped package never does.
 *
 * Follows entropack/schemes/tile_ans/eager.py:231-307 of the reference (table step, shared renormalisation in
 * ascending lane order from the end of the stream, tail group first, raw lanes two bytes per word).
 * Pinning: tests/test_tile_ans_golden.py, against every fixture the reference wrote and against the Python twin.
 */
#include <stdint.h>
#include <string.h>

enum { TAO_OK = 0, TAO_BAD_ARGUMENT = 1, TAO_TRUNCATED = 2, TAO_NOT_CONSUMED = 3, TAO_BAD_RAW_LENGTH = 4 };

static int decode_group(uint32_t* x, const uint32_t* table, const uint16_t* words, int64_t* pointer, uint8_t* out,
                        int64_t base, int valid, int prob_bits, int64_t stride) {
  const uint32_t size = 1u << prob_bits;
  int readers[32];
  int n = 0;
  for (int lane = 0; lane < valid; ++lane) {
    const uint32_t slot = x[lane] & (size - 1u);
    const uint32_t entry = table[slot];
    uint32_t freq = (entry >> 8) & 0xFFFu;
    if (freq == 0) freq = size;
    out[(base + lane) * stride] = (uint8_t)(entry & 0xFFu);
    x[lane] = freq * (x[lane] >> prob_bits) + slot - (entry >> 20);
    if (x[lane] < (1u << 15)) readers[n++] = lane;
  }
  const int64_t first = *pointer - n;
  if (first < 0) return TAO_TRUNCATED;
  for (int i = 0; i < n; ++i) x[readers[i]] = (x[readers[i]] << 16) | words[first + i];
  *pointer = first;
  return TAO_OK;
}

/* out: uint8[elements * lanes]. Returns the first error of any stream. */
int tao_decode(const uint16_t* payload, const uint32_t* offsets, const uint32_t* states, const uint32_t* tables,
               const uint8_t* lane_modes, int64_t tile_elements, int prob_bits, int lanes, int64_t elements, uint8_t* out,
               int threads) {
  if (tile_elements <= 0 || prob_bits < 9 || prob_bits > 12 || lanes <= 0 || elements <= 0) return TAO_BAD_ARGUMENT;
  const int64_t tiles = (elements + tile_elements - 1) / tile_elements;
  int coded_before[64];
  if (lanes > 63) return TAO_BAD_ARGUMENT;
  coded_before[0] = 0;
  for (int lane = 0; lane < lanes; ++lane) coded_before[lane + 1] = coded_before[lane] + (lane_modes[lane] == 0);
  int status = TAO_OK;
#pragma omp parallel for schedule(dynamic, 16) num_threads(threads > 0 ? threads : 1)
  for (int64_t stream = 0; stream < tiles * lanes; ++stream) {
    const int lane = (int)(stream / tiles);
    const int64_t tile = stream % tiles;
    const int64_t first = tile * tile_elements;
    const int64_t count = elements - first < tile_elements ? elements - first : tile_elements;
    const uint16_t* words = payload + offsets[stream];
    const int64_t n_words = (int64_t)offsets[stream + 1] - (int64_t)offsets[stream];
    uint8_t* dst = out + first * lanes + lane;
    int bad = TAO_OK;
    if (lane_modes[lane] != 0) {
      if (n_words != (count + 1) / 2) {
        bad = TAO_BAD_RAW_LENGTH;
      } else {
        for (int64_t e = 0; e < count; ++e) dst[e * lanes] = (uint8_t)((e & 1) ? words[e / 2] >> 8 : words[e / 2] & 0xFFu);
      }
    } else {
      uint32_t x[32];
      memcpy(x, states + ((int64_t)coded_before[lane] * tiles + tile) * 32, sizeof(x));
      int64_t pointer = n_words;
      const int rem = (int)(count % 32);
      int64_t at = count - rem;
      const uint32_t* table = tables + ((int64_t)lane << prob_bits);
      if (rem) bad = decode_group(x, table, words, &pointer, dst, at, rem, prob_bits, lanes);
      while (at > 0 && bad == TAO_OK) {
        at -= 32;
        bad = decode_group(x, table, words, &pointer, dst, at, 32, prob_bits, lanes);
      }
      if (bad == TAO_OK && pointer != 0) bad = TAO_NOT_CONSUMED;
    }
    if (bad != TAO_OK) {
#pragma omp critical
      if (status == TAO_OK) status = bad;
    }
  }
  return status;
}
