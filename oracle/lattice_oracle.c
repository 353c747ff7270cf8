/* CPU oracle for the lattice_rans decode path -- TEST INFRASTRUCTURE, not product code.
 *
 * The C twin of lattice_oracle.py: the same functions, tile-parallel (OpenMP), fast enough to check the GPU on
 * full-size containers and to serve as the timed CPU baseline. Only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may load the library built from this file; the shipped package never does.
 *
 * What each function follows in the reference (paths relative to the reference root):
 *   orc_build_slot_table   entropack/schemes/lattice_rans/rans.py:74-95
 *   step / renormalise     entropack/schemes/lattice_rans/rans.py:98-120
 *   group order            entropack/schemes/lattice_rans/rans.py:123-130
 *   tile schedule          entropack/schemes/lattice_rans/rans.py:189-221
 *   field minima           entropack/schemes/lattice_rans/eager.py:361-367
 *   E8 point               entropack/schemes/lattice_rans/eager.py:54-58
 *   row rescale            entropack/schemes/lattice_rans/eager.py:370-376
 *   container snap         entropack/schemes/lattice_rans/format.py:153-168
 *
 * Pinning: tests/test_oracle_golden.py checks every entry point against the fixtures the reference wrote
 * (tests/golden/), and against the Python twin on seeded inputs. Nothing here is "parity unpinned".
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -ffp-contract=off: the float tail must not fuse multiply-add).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_NUM_STATES 32
#define ORC_STATE_MIN (1u << 15)
#define ORC_STREAMS 17
#define ORC_FIELDS 8

enum {
  ORC_OK = 0,
  ORC_BAD_ARGUMENT = 1,
  ORC_TRUNCATED = 2,      /* a renormalisation read would pass the start of the tile's payload */
  ORC_NOT_CONSUMED = 3,   /* tile finished with unread words or a lane state != 2^15 */
  ORC_BAD_TABLE = 4       /* frequencies do not sum to 2^prob_bits, or the alphabet exceeds it */
};

/* Store kinds: the numbering of the reference's device code (lattice_rans.cu:525-539), plus bf16. */
enum {
  ORC_F32 = 0, ORC_F16 = 1, ORC_I8 = 4, ORC_I16 = 5, ORC_I32 = 6, ORC_I64 = 7,
  ORC_U8 = 8, ORC_U16 = 9, ORC_U32 = 10, ORC_U64 = 11, ORC_BOOL = 12, ORC_BF16 = 100
};

/* slot -> cdf << 32 | freq << 16 | symbol, with freq == 2^prob_bits stored as 0 (rans.py:89-90). */
int orc_build_slot_table(const uint16_t* freq, int alphabet, int prob_bits, uint64_t* lut) {
  const uint32_t size = 1u << prob_bits;
  uint32_t running = 0;
  if (alphabet < 0 || (uint32_t)alphabet > size) return ORC_BAD_TABLE;
  for (int symbol = 0; symbol < alphabet; ++symbol) {
    const uint32_t f = freq[symbol];
    if (f == 0) continue;
    if (running + f > size) return ORC_BAD_TABLE;
    const uint64_t entry = ((uint64_t)running << 32) | ((uint64_t)(f == size ? 0u : f) << 16) | (uint64_t)symbol;
    for (uint32_t s = 0; s < f; ++s) lut[running + s] = entry;
    running += f;
  }
  return running == size ? ORC_OK : ORC_BAD_TABLE;
}

/* One symbol per valid lane, then the shared renormalisation (rans.py:98-120). table_of_lane == NULL: all lanes
 * use luts[0]; otherwise lane l uses luts[table_of_lane[l]]. Returns the new pointer, or -1 when truncated. */
static int64_t step(uint32_t* x, const uint64_t* const* luts, const int32_t* table_of_lane, const uint16_t* words,
                    int64_t pointer, int32_t* out, int stride, int valid, int prob_bits) {
  const uint32_t size = 1u << prob_bits;
  int readers[ORC_NUM_STATES];
  int n = 0;
  for (int lane = 0; lane < valid; ++lane) {
    const uint32_t state = x[lane];
    const uint32_t slot = state & (size - 1u);
    const uint64_t entry = luts[table_of_lane ? table_of_lane[lane] : 0][slot];
    uint32_t f = (uint32_t)((entry >> 16) & 0xFFFFu);
    if (f == 0) f = size;
    out[(int64_t)lane * stride] = (int32_t)(entry & 0xFFFFu);
    x[lane] = f * (state >> prob_bits) + (slot - (uint32_t)(entry >> 32));
    if (x[lane] < ORC_STATE_MIN) readers[n++] = lane;
  }
  const int64_t first = pointer - n;
  if (first < 0) return -1;
  for (int i = 0; i < n; ++i) x[readers[i]] = (x[readers[i]] << 16) | words[first + i];
  return first;
}

/* Coset from stream 0, then field f from stream 1 + 2f + coset (rans.py:123-130). */
static int64_t group(uint32_t* x, const uint64_t* const* luts, const uint16_t* words, int64_t pointer,
                     int32_t* coset_out, int32_t* field_out, int valid, int prob_bits) {
  pointer = step(x, luts, NULL, words, pointer, coset_out, 1, valid, prob_bits);
  for (int f = 0; f < ORC_FIELDS && pointer >= 0; ++f) {
    const uint64_t* pair[2] = {luts[1 + 2 * f], luts[2 + 2 * f]};
    pointer = step(x, pair, coset_out, words, pointer, field_out + f, ORC_FIELDS, valid, prob_bits);
  }
  return pointer;
}

/* Entropy decode of every tile (rans.py:189-221). cosets: int32[V]; fields: int32[V][8] (still minus sym_min).
 * stream_meta: int32[17][4] = (n_symbols, sym_min, freq_offset, alphabet). Returns the first error met. */
int orc_decode_symbols(const uint16_t* payload, const uint32_t* offsets, const uint32_t* states,
                       const int32_t* stream_meta, const uint16_t* freq_tables, int prob_bits, int tile_vectors,
                       int64_t num_vectors, int32_t* cosets, int32_t* fields, int threads) {
  if (prob_bits < 9 || prob_bits > 15 || tile_vectors < 1 || num_vectors < 0) return ORC_BAD_ARGUMENT;
  const size_t size = (size_t)1 << prob_bits;
  uint64_t* storage = (uint64_t*)calloc(ORC_STREAMS * size, sizeof(uint64_t));
  const uint64_t* luts[ORC_STREAMS];
  if (!storage) return ORC_BAD_ARGUMENT;
  int status = ORC_OK;
  for (int s = 0; s < ORC_STREAMS; ++s) {
    const int alphabet = stream_meta[4 * s + 3];
    luts[s] = storage + s * size;
    if (alphabet > 0) {
      const int rc = orc_build_slot_table(freq_tables + stream_meta[4 * s + 2], alphabet, prob_bits, storage + s * size);
      if (rc != ORC_OK) status = rc;
    }
  }
  if (status != ORC_OK) { free(storage); return status; }
  int64_t tiles = (num_vectors + tile_vectors - 1) / tile_vectors;
  if (tiles < 1) tiles = 1;
#pragma omp parallel for schedule(dynamic, 4) num_threads(threads > 0 ? threads : 1)
  for (int64_t tile = 0; tile < tiles; ++tile) {
    const int64_t begin = tile * tile_vectors;
    const int count = (int)(num_vectors - begin < tile_vectors ? num_vectors - begin : tile_vectors);
    const uint16_t* words = payload + offsets[tile];
    int64_t pointer = (int64_t)offsets[tile + 1] - (int64_t)offsets[tile];
    uint32_t x[ORC_NUM_STATES];
    memcpy(x, states + tile * ORC_NUM_STATES, sizeof(x));
    const int rem = count % ORC_NUM_STATES;
    int off = count - rem;
    int rc = ORC_OK;
    if (rem) {
      pointer = group(x, luts, words, pointer, cosets + begin + off, fields + (begin + off) * ORC_FIELDS, rem, prob_bits);
    }
    while (pointer >= 0 && off > 0) {
      off -= ORC_NUM_STATES;
      pointer = group(x, luts, words, pointer, cosets + begin + off, fields + (begin + off) * ORC_FIELDS,
                      ORC_NUM_STATES, prob_bits);
    }
    if (pointer < 0) {
      rc = ORC_TRUNCATED;
    } else if (pointer != 0) {
      rc = ORC_NOT_CONSUMED;
    } else {
      for (int lane = 0; lane < ORC_NUM_STATES; ++lane) if (x[lane] != ORC_STATE_MIN) rc = ORC_NOT_CONSUMED;
    }
    if (rc != ORC_OK) {
#pragma omp critical
      if (status == ORC_OK) status = rc;
    }
  }
  free(storage);
  return status;
}

static uint16_t bf16_bits(float v) {
  uint32_t bits;
  memcpy(&bits, &v, 4);
  if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((bits >> 16) | 0x40u);
  return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

static uint16_t f16_bits(float v) {   /* round to nearest even; input already clamped to +-65504 */
  uint32_t bits;
  memcpy(&bits, &v, 4);
  const uint32_t sign = (bits >> 16) & 0x8000u;
  const uint32_t mag = bits & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
  if (mag >= 0x38800000u) {            /* normal half */
    const uint32_t r = mag - 0x38000000u;
    return (uint16_t)(sign | ((r + 0xFFFu + ((r >> 13) & 1u)) >> 13));
  }
  if (mag < 0x33000000u) return (uint16_t)sign;   /* below half the smallest subnormal -> 0 */
  const int shift = 126 - (int)(mag >> 23);        /* 14..24 */
  const uint32_t m = (mag & 0x7FFFFFu) | 0x800000u;
  const uint32_t q = m >> shift;
  const uint32_t rest = m & ((1u << shift) - 1u);
  const uint32_t half = 1u << (shift - 1);
  return (uint16_t)(sign | (q + ((rest > half) || (rest == half && (q & 1u)))));
}

static float snap_int(float v, float low, float high_exclusive) {   /* format.py:165-166 */
  const float high = nextafterf(high_exclusive, 0.0f);
  const float r = rintf(v);                                          /* half to even */
  return fminf(fmaxf(r, low), high);
}

/* Field minima, E8 point, row scale, container cast (eager.py:361-376, 54-58; format.py:153-168).
 * out: [rows][cols] of the container type. */
int orc_reconstruct(const int32_t* cosets, const int32_t* fields, const int32_t* stream_meta, const float* scales,
                    int64_t rows, int cols, int kind, void* out, int threads) {
  if (cols <= 0 || cols % 8) return ORC_BAD_ARGUMENT;
  const int vpr = cols / 8;
  const int64_t vectors = rows * vpr;
  int bad = 0;
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
  for (int64_t v = 0; v < vectors; ++v) {
    const int c = cosets[v];
    int32_t z[8];
    int32_t sum = 0;
    for (int f = 0; f < 8; ++f) z[f] = fields[v * 8 + f] + stream_meta[4 * (1 + 2 * f + c) + 1];
    for (int f = 0; f < 7; ++f) sum += z[f];
    z[7] = 2 * z[7] + (sum & 1);               /* two's complement & 1 == non-negative remainder */
    const float half = c ? 0.5f : 0.0f;
    const float scale = scales[v / vpr];
    for (int f = 0; f < 8; ++f) {
      const float point = (float)z[f] + half;
      const float w = point * scale;            /* -ffp-contract=off: one rounded multiply */
      const int64_t at = v * 8 + f;
      switch (kind) {
        case ORC_F32: ((float*)out)[at] = w; break;
        case ORC_BF16: ((uint16_t*)out)[at] = bf16_bits(fminf(fmaxf(w, -3.3895313892515355e38f), 3.3895313892515355e38f)); break;
        case ORC_F16: ((uint16_t*)out)[at] = f16_bits(fminf(fmaxf(w, -65504.0f), 65504.0f)); break;
        case ORC_I8: ((int8_t*)out)[at] = (int8_t)snap_int(w, -128.0f, 128.0f); break;
        case ORC_I16: ((int16_t*)out)[at] = (int16_t)snap_int(w, -32768.0f, 32768.0f); break;
        case ORC_I32: ((int32_t*)out)[at] = (int32_t)snap_int(w, -2147483648.0f, 2147483648.0f); break;
        case ORC_I64: ((int64_t*)out)[at] = (int64_t)snap_int(w, -9223372036854775808.0f, 9223372036854775808.0f); break;
        case ORC_U8: ((uint8_t*)out)[at] = (uint8_t)snap_int(w, 0.0f, 256.0f); break;
        case ORC_U16: ((uint16_t*)out)[at] = (uint16_t)snap_int(w, 0.0f, 65536.0f); break;
        case ORC_U32: ((uint32_t*)out)[at] = (uint32_t)snap_int(w, 0.0f, 4294967296.0f); break;
        case ORC_U64: ((uint64_t*)out)[at] = (uint64_t)snap_int(w, 0.0f, 18446744073709551616.0f); break;
        case ORC_BOOL: ((uint8_t*)out)[at] = rintf(w) != 0.0f; break;
        default: bad = 1; break;
      }
    }
  }
  return bad ? ORC_BAD_ARGUMENT : ORC_OK;
}

/* Whole decode of one container (eager.py:379-396). Allocates the symbol planes internally. */
int orc_decode(const uint16_t* payload, const uint32_t* offsets, const uint32_t* states, const int32_t* stream_meta,
               const uint16_t* freq_tables, const float* scales, int64_t rows, int cols, int prob_bits,
               int tile_elements, int kind, void* out, int threads) {
  if (rows <= 0 || cols <= 0 || cols % 8 || tile_elements <= 0) return ORC_BAD_ARGUMENT;
  const int tile_vectors = tile_elements / 9 > 32 ? tile_elements / 9 : 32;   /* format.py:171-172 */
  const int64_t vectors = rows * (cols / 8);
  int32_t* cosets = (int32_t*)malloc((size_t)vectors * sizeof(int32_t));
  int32_t* fields = (int32_t*)malloc((size_t)vectors * 8 * sizeof(int32_t));
  int rc = ORC_BAD_ARGUMENT;
  if (cosets && fields) {
    rc = orc_decode_symbols(payload, offsets, states, stream_meta, freq_tables, prob_bits, tile_vectors, vectors,
                            cosets, fields, threads);
    if (rc == ORC_OK) rc = orc_reconstruct(cosets, fields, stream_meta, scales, rows, cols, kind, out, threads);
  }
  free(cosets);
  free(fields);
  return rc;
}
