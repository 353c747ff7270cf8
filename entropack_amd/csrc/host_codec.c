/* libentropack_host.so: CPU encoder kernels of the lattice_rans scheme (plain C + OpenMP, no GPU).
 *
 * Tensors on the CPU are encoded on the CPU: the package carries its own
 * CPU restatement of the reference encoder; the heavy loops live here and the orchestration (scale search,
 * Hamilton normalisation, row-scale refit) in schemes/lattice_rans/eager.py. Algorithms followed, in the
 * reference tree:
 *   hc_quantize      entropack/schemes/lattice_rans/eager.py:18-51  (nearest E8 point, point -> coset + fields)
 *   hc_levels        entropack/schemes/lattice_rans/eager.py:54-58  (fields -> point)
 *   hc_rans_encode   entropack/schemes/lattice_rans/rans.py:133-186 (tiled 32-way interleaved rANS encode)
 *   hc_tile_ans_encode  entropack/schemes/tile_ans/eager.py:145-228 (byte-lane streams: raw words or 32-way rANS)
 * Built with -ffp-contract=off: every float operation below is a single IEEE operation, as in the reference.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define HC_STATES 32
#define HC_STATE_MIN (1u << 15)
#define HC_STREAMS 17

static void nearest_dn(const float* y, float* out) {
  float r[8];
  float total = 0.0f;
  for (int j = 0; j < 8; ++j) {
    out[j] = rintf(y[j]);            /* round half to even */
    r[j] = y[j] - out[j];
    total += out[j];                 /* small integers: exact in any order */
  }
  int at = 0;
  float best = -1.0f;
  for (int j = 0; j < 8; ++j) {
    const float a = fabsf(r[j]);
    if (a > best) { best = a; at = j; }   /* first maximum wins */
  }
  if (fmodf(total, 2.0f) != 0.0f) out[at] += (r[at] < 0.0f) ? -1.0f : 1.0f;   /* a zero residual steps up */
}

/* Sum of squared differences in float64, paired as (0+4)+(2+6) and (1+5)+(3+7): the order the reference's
 * per-row float64 reduction uses, which decides exact ties between the two cosets. */
static double distance2(const float* y, const float* p) {
  double s[8];
  for (int j = 0; j < 8; ++j) {
    const double d = (double)y[j] - (double)p[j];
    s[j] = d * d;
  }
  return ((s[0] + s[4]) + (s[2] + s[6])) + ((s[1] + s[5]) + (s[3] + s[7]));
}

/* Quantises rows `row_index[0..n_sel)` (or rows 0..n_sel when row_index is NULL) of x[rows][cols]:
 * y = (x / rms[row]) / scale, nearest E8 point, split into coset bit and the 8 fields (z0..z6, m).
 * coset: int8[n_sel * cols / 8]; fields: int32[n_sel * cols / 8][8]. */
void hc_quantize(const float* x, const float* rms, int64_t cols, float scale, const int64_t* row_index, int64_t n_sel,
                 int8_t* coset, int32_t* fields, int threads) {
  const int64_t vpr = cols / 8;
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
  for (int64_t i = 0; i < n_sel; ++i) {
    const int64_t row = row_index ? row_index[i] : i;
    const float* src = x + row * cols;
    const float norm = rms[row];
    for (int64_t v = 0; v < vpr; ++v) {
      float y[8], shifted[8], c0[8], c1[8];
      for (int j = 0; j < 8; ++j) {
        y[j] = (src[v * 8 + j] / norm) / scale;
        shifted[j] = y[j] - 0.5f;
      }
      nearest_dn(y, c0);
      nearest_dn(shifted, c1);
      for (int j = 0; j < 8; ++j) c1[j] += 0.5f;
      const int c = !(distance2(y, c0) <= distance2(y, c1));
      const float* p = c ? c1 : c0;
      int32_t z[8];
      int32_t sum = 0;
      for (int j = 0; j < 8; ++j) z[j] = (int32_t)rintf(p[j] - (c ? 0.5f : 0.0f));
      for (int j = 0; j < 7; ++j) sum += z[j];
      const int32_t parity = sum & 1;
      const int32_t top = z[7] - parity;          /* even by construction of E8; floor-divide anyway */
      z[7] = (top >= 0) ? top / 2 : -((-top + 1) / 2);
      const int64_t at = i * vpr + v;
      coset[at] = (int8_t)c;
      memcpy(fields + at * 8, z, sizeof(z));
    }
  }
}

/* Lattice point of each vector as float32[V][8]: z0..z6, 2 m + parity, plus c / 2. */
void hc_levels(const int8_t* coset, const int32_t* fields, int64_t vectors, float* levels, int threads) {
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
  for (int64_t v = 0; v < vectors; ++v) {
    const int32_t* z = fields + v * 8;
    int32_t sum = 0;
    for (int j = 0; j < 7; ++j) sum += z[j];
    const float half = coset[v] ? 0.5f : 0.0f;
    for (int j = 0; j < 7; ++j) levels[v * 8 + j] = (float)z[j] + half;
    levels[v * 8 + 7] = (float)(2 * z[7] + (sum & 1)) + half;
  }
}

/* Per stream (0 = coset, 1 + 2f + c = field f of coset-c vectors): symbol count, minimum and maximum.
 * stats: int64[17][3] = (n, min, max); min/max are 0 for empty streams. */
void hc_stream_stats(const int8_t* coset, const int32_t* fields, int64_t vectors, int64_t* stats) {
  int64_t n[HC_STREAMS] = {0}, lo[HC_STREAMS], hi[HC_STREAMS];
  for (int s = 0; s < HC_STREAMS; ++s) { lo[s] = INT64_MAX; hi[s] = INT64_MIN; }
  for (int64_t v = 0; v < vectors; ++v) {
    const int c = coset[v];
    n[0]++;
    if (c < lo[0]) lo[0] = c;
    if (c > hi[0]) hi[0] = c;
    for (int f = 0; f < 8; ++f) {
      const int s = 1 + 2 * f + c;
      const int64_t z = fields[v * 8 + f];
      n[s]++;
      if (z < lo[s]) lo[s] = z;
      if (z > hi[s]) hi[s] = z;
    }
  }
  for (int s = 0; s < HC_STREAMS; ++s) {
    stats[3 * s] = n[s];
    stats[3 * s + 1] = n[s] ? lo[s] : 0;
    stats[3 * s + 2] = n[s] ? hi[s] : 0;
  }
}

/* Histogram of every stream. counts is the concatenation of the 17 histograms; stream s starts at
 * count_offset[s] and bins (value - sym_min[s]). */
void hc_stream_counts(const int8_t* coset, const int32_t* fields, int64_t vectors, const int64_t* sym_min,
                      const int64_t* count_offset, int64_t* counts) {
  for (int64_t v = 0; v < vectors; ++v) {
    const int c = coset[v];
    counts[count_offset[0] + c - sym_min[0]]++;
    for (int f = 0; f < 8; ++f) {
      const int s = 1 + 2 * f + c;
      counts[count_offset[s] + fields[v * 8 + f] - sym_min[s]]++;
    }
  }
}

/* Largest-remainder (Hamilton) allocation of table_size slots over the symbols of a histogram, every present symbol
 * getting at least one (entropack/schemes/lattice_rans/rans.py:12-71 of the reference): ideal = count * (table_size /
 * total) in float64, floor, at least 1 where the count is not 0; a shortfall goes one slot at a time to the present
 * symbols in order of descending residual ideal - freq, a surplus comes one slot at a time from the symbols still above
 * 1 in order of ascending residual; equal residuals go by symbol, and a pass over the order repeats until the gap is
 * closed. Returns 0, -1 for an empty histogram, -2 when a surplus cannot be taken back, -3 out of memory. */
typedef struct {
  double key;
  int64_t symbol;
} ranked_symbol;

static int by_key_then_symbol(const void* a, const void* b) {
  const ranked_symbol* x = (const ranked_symbol*)a;
  const ranked_symbol* y = (const ranked_symbol*)b;
  if (x->key < y->key) return -1;
  if (x->key > y->key) return 1;
  return (x->symbol > y->symbol) - (x->symbol < y->symbol);
}

int hc_normalize_counts(const int64_t* counts, int64_t n, int64_t table_size, uint16_t* freq_out) {
  int64_t total = 0;
  for (int64_t i = 0; i < n; ++i) total += counts[i];
  if (n <= 0 || total == 0) return -1;
  int64_t* freq = (int64_t*)malloc((size_t)n * sizeof(int64_t));
  double* residual = (double*)malloc((size_t)n * sizeof(double));
  ranked_symbol* order = (ranked_symbol*)malloc((size_t)n * sizeof(ranked_symbol));
  if (!freq || !residual || !order) { free(freq); free(residual); free(order); return -3; }
  const double scale = (double)table_size / (double)total;
  int64_t given = 0;
  for (int64_t i = 0; i < n; ++i) {
    const double ideal = (double)counts[i] * scale;
    freq[i] = (int64_t)floor(ideal);
    if (counts[i] != 0 && freq[i] < 1) freq[i] = 1;
    residual[i] = ideal - (double)freq[i];
    given += freq[i];
  }
  int64_t gap = table_size - given;
  int status = 0;
  if (gap > 0) {
    int64_t present = 0;
    for (int64_t i = 0; i < n; ++i)
      if (counts[i] != 0) { order[present].key = -residual[i]; order[present].symbol = i; ++present; }
    qsort(order, (size_t)present, sizeof(ranked_symbol), by_key_then_symbol);
    while (gap > 0) {
      const int64_t take = gap < present ? gap : present;
      for (int64_t k = 0; k < take; ++k) freq[order[k].symbol] += 1;
      gap -= take;
    }
  } else if (gap < 0) {
    int64_t pool = 0;
    for (int64_t i = 0; i < n; ++i)
      if (counts[i] != 0 && freq[i] > 1) { order[pool].key = residual[i]; order[pool].symbol = i; ++pool; }
    if (pool == 0) status = -2;
    else qsort(order, (size_t)pool, sizeof(ranked_symbol), by_key_then_symbol);
    while (status == 0 && gap < 0) {
      int64_t taken = 0;
      for (int64_t k = 0; k < pool && taken < -gap; ++k)
        if (freq[order[k].symbol] > 1) { freq[order[k].symbol] -= 1; ++taken; }
      if (taken == 0) status = -2;
      gap += taken;
    }
  }
  if (status == 0)
    for (int64_t i = 0; i < n; ++i) freq_out[i] = (uint16_t)freq[i];
  free(freq);
  free(residual);
  free(order);
  return status;
}

/* hc_normalize_counts for several histograms laid end to end: histogram s is counts[starts[s] .. starts[s + 1]), its
 * frequencies go to the same positions of freq_out. Returns 0, or the first histogram's error code. */
int hc_normalize_streams(const int64_t* counts, const int64_t* starts, int64_t n_streams, int64_t table_size, uint16_t* freq_out) {
  for (int64_t s = 0; s < n_streams; ++s) {
    const int status = hc_normalize_counts(counts + starts[s], starts[s + 1] - starts[s], table_size, freq_out + starts[s]);
    if (status != 0) return status;
  }
  return 0;
}

/* The lossless scheme's allocation of table_size slots (entropack/schemes/tile_ans/eager.py:17-60 of the reference):
 * floor of the exact float64 share, at least 1 for a present symbol; then one slot at a time, a shortfall to the symbol
 * with the largest remainder (its remainder drops by one when it is served), a surplus from the symbol with the
 * smallest remainder among those above one slot (its remainder rises by one; at one slot it leaves the pool); the
 * smallest symbol among equals. Returns 0, -1 for an empty histogram, -2 when a surplus cannot be taken back, -3 out of
 * memory. */
int hc_tile_ans_normalize_counts(const int64_t* counts, int64_t n, int64_t table_size, uint16_t* freq_out) {
  int64_t total = 0;
  for (int64_t i = 0; i < n; ++i) total += counts[i];
  if (n <= 0 || total == 0) return -1;
  int64_t* freq = (int64_t*)malloc((size_t)n * sizeof(int64_t));
  double* key = (double*)malloc((size_t)n * sizeof(double));
  if (!freq || !key) { free(freq); free(key); return -3; }
  const double scale = (double)table_size / (double)total;
  int64_t given = 0;
  for (int64_t i = 0; i < n; ++i) {
    const double share = (double)counts[i] * scale;
    freq[i] = (int64_t)floor(share);
    if (counts[i] != 0 && freq[i] < 1) freq[i] = 1;
    key[i] = share - (double)freq[i];           /* the remainder, for now */
    given += freq[i];
  }
  const int64_t gap = table_size - given;
  int status = 0;
  if (gap > 0) {
    for (int64_t i = 0; i < n; ++i) key[i] = counts[i] != 0 ? -key[i] : INFINITY;
    for (int64_t step = 0; step < gap; ++step) {
      int64_t best = 0;
      for (int64_t i = 1; i < n; ++i)
        if (key[i] < key[best]) best = i;       /* first minimum */
      freq[best] += 1;
      key[best] += 1.0;
    }
  } else if (gap < 0) {
    int64_t pool = 0;
    for (int64_t i = 0; i < n; ++i) {
      if (counts[i] != 0 && freq[i] > 1) ++pool;
      else key[i] = INFINITY;
    }
    if (pool == 0) status = -2;
    for (int64_t step = 0; status == 0 && step < -gap; ++step) {
      int64_t best = 0;
      for (int64_t i = 1; i < n; ++i)
        if (key[i] < key[best]) best = i;
      if (isinf(key[best])) { status = -2; break; }
      freq[best] -= 1;
      key[best] = freq[best] > 1 ? key[best] + 1.0 : INFINITY;
    }
  }
  if (status == 0)
    for (int64_t i = 0; i < n; ++i) freq_out[i] = (uint16_t)freq[i];
  free(freq);
  free(key);
  return status;
}

typedef struct {
  uint16_t* words;
  size_t size, capacity;
} word_list;

static int push_word(word_list* list, uint16_t w) {
  if (list->size == list->capacity) {
    const size_t grown = list->capacity ? list->capacity * 2 : 4096;
    uint16_t* moved = (uint16_t*)realloc(list->words, grown * sizeof(uint16_t));
    if (!moved) return -1;
    list->words = moved;
    list->capacity = grown;
  }
  list->words[list->size++] = w;
  return 0;
}

static inline int put(uint32_t* state, uint32_t freq, uint32_t cdf, int prob_bits, word_list* out) {
  uint32_t x = *state;
  if (x >= (freq << (31 - prob_bits))) {          /* rans.py:168-170 */
    if (push_word(out, (uint16_t)(x & 0xFFFFu))) return -1;
    x >>= 16;
  }
  *state = (x / freq) * (1u << prob_bits) + (x % freq) + cdf;
  return 0;
}

/* Tiled 32-way interleaved rANS encode of all vectors. freq / cdf: per stream, indexed by (value - sym_min[s]),
 * concatenated with stream s starting at table_offset[s]. states: u32[tiles][32]; offsets: u32[tiles + 1];
 * *payload receives a malloc'd array of offsets[tiles] words (free it with hc_free). Returns 0, or -1 when out of
 * memory, or -2 when the payload would not fit 32-bit offsets. */
int hc_rans_encode(const int8_t* coset, const int32_t* fields, int64_t vectors, const int64_t* sym_min,
                   const int64_t* table_offset, const uint32_t* freq, const uint32_t* cdf, int prob_bits,
                   int tile_vectors, uint32_t* states, uint32_t* offsets, uint16_t** payload, int threads) {
  int64_t tiles = (vectors + tile_vectors - 1) / tile_vectors;
  if (tiles < 1) tiles = 1;
  word_list* lists = (word_list*)calloc((size_t)tiles, sizeof(word_list));
  if (!lists) return -1;
  int failed = 0;
#pragma omp parallel for schedule(dynamic, 8) num_threads(threads > 0 ? threads : 1)
  for (int64_t tile = 0; tile < tiles; ++tile) {
    const int64_t begin = tile * tile_vectors;
    const int64_t end = begin + tile_vectors < vectors ? begin + tile_vectors : vectors;
    uint32_t x[HC_STATES];
    for (int l = 0; l < HC_STATES; ++l) x[l] = HC_STATE_MIN;
    word_list* out = &lists[tile];
    int bad = 0;
    for (int64_t base = begin; base < end && !bad; base += HC_STATES) {
      const int lanes = (int)(end - base < HC_STATES ? end - base : HC_STATES);
      for (int f = 7; f >= 0 && !bad; --f) {                     /* fields last to first, then the coset */
        for (int l = 0; l < lanes; ++l) {
          const int64_t v = base + l;
          const int s = 1 + 2 * f + coset[v];
          const int64_t at = table_offset[s] + fields[v * 8 + f] - sym_min[s];
          if (put(&x[l], freq[at], cdf[at], prob_bits, out)) { bad = 1; break; }
        }
      }
      for (int l = 0; l < lanes && !bad; ++l) {
        const int64_t at = table_offset[0] + coset[base + l] - sym_min[0];
        if (put(&x[l], freq[at], cdf[at], prob_bits, out)) bad = 1;
      }
    }
    memcpy(states + tile * HC_STATES, x, sizeof(x));
    if (bad) {
#pragma omp atomic write
      failed = 1;
    }
  }
  uint64_t total = 0;
  offsets[0] = 0;
  for (int64_t tile = 0; tile < tiles; ++tile) {
    total += lists[tile].size;
    if (total > 0xFFFFFFFFull) failed = 2;
    offsets[tile + 1] = (uint32_t)total;
  }
  uint16_t* joined = NULL;
  if (!failed) {
    joined = (uint16_t*)malloc((total ? total : 1) * sizeof(uint16_t));
    if (!joined) failed = 1;
  }
  if (!failed) {
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
    for (int64_t tile = 0; tile < tiles; ++tile) {
      if (lists[tile].size) memcpy(joined + offsets[tile], lists[tile].words, lists[tile].size * sizeof(uint16_t));
    }
  }
  for (int64_t tile = 0; tile < tiles; ++tile) free(lists[tile].words);
  free(lists);
  *payload = joined;
  return failed == 0 ? 0 : (failed == 2 ? -2 : -1);
}

/* Lossless byte-lane coder. `bytes` is the tensor's storage, num_elements x num_lanes bytes; stream (lane, tile)
 * covers byte `lane` of elements [tile * tile_elements, ...). A raw lane stores its bytes two per word (even element in
 * the low byte); a coded lane runs 32 interleaved rANS states over its symbols in order, group after group of 32.
 * freq / cdf: u16[num_lanes][256]. states: u32[tiles * coded lanes][32], coded lanes in lane order; offsets:
 * u32[num_lanes * tiles + 1]; *payload: malloc'd (hc_free). Returns 0, -1 out of memory, -2 payload beyond 32-bit offsets. */
int hc_tile_ans_encode(const uint8_t* bytes, int64_t num_elements, int num_lanes, int64_t tile_elements, int prob_bits,
                       const uint16_t* freq, const uint16_t* cdf, const uint8_t* lane_raw, uint32_t* states,
                       uint32_t* offsets, uint16_t** payload, int threads) {
  const int64_t tiles = (num_elements + tile_elements - 1) / tile_elements;
  const int64_t streams = tiles * num_lanes;
  word_list* lists = (word_list*)calloc((size_t)streams, sizeof(word_list));
  int* coded_before = (int*)calloc((size_t)num_lanes + 1, sizeof(int));
  if (!lists || !coded_before) { free(lists); free(coded_before); return -1; }
  for (int lane = 0; lane < num_lanes; ++lane) coded_before[lane + 1] = coded_before[lane] + (lane_raw[lane] ? 0 : 1);
  int failed = 0;
#pragma omp parallel for schedule(dynamic, 8) num_threads(threads > 0 ? threads : 1)
  for (int64_t stream = 0; stream < streams; ++stream) {
    const int lane = (int)(stream / tiles);
    const int64_t tile = stream % tiles;
    const int64_t begin = tile * tile_elements;
    const int64_t end = begin + tile_elements < num_elements ? begin + tile_elements : num_elements;
    word_list* out = &lists[stream];
    int bad = 0;
    if (lane_raw[lane]) {
      for (int64_t e = begin; e < end && !bad; e += 2) {
        uint16_t word = bytes[e * num_lanes + lane];
        if (e + 1 < end) word |= (uint16_t)(bytes[(e + 1) * num_lanes + lane] << 8);
        if (push_word(out, word)) bad = 1;
      }
    } else {
      uint32_t x[HC_STATES];
      for (int l = 0; l < HC_STATES; ++l) x[l] = HC_STATE_MIN;
      const uint16_t* f = freq + lane * 256;
      const uint16_t* c = cdf + lane * 256;
      for (int64_t base = begin; base < end && !bad; base += HC_STATES) {
        const int lanes = (int)(end - base < HC_STATES ? end - base : HC_STATES);
        for (int l = 0; l < lanes; ++l) {
          const uint8_t symbol = bytes[(base + l) * num_lanes + lane];
          if (put(&x[l], f[symbol], c[symbol], prob_bits, out)) { bad = 1; break; }
        }
      }
      memcpy(states + ((int64_t)coded_before[lane] * tiles + tile) * HC_STATES, x, sizeof(x));
    }
    if (bad) {
#pragma omp atomic write
      failed = 1;
    }
  }
  uint64_t total = 0;
  offsets[0] = 0;
  for (int64_t stream = 0; stream < streams; ++stream) {
    total += lists[stream].size;
    if (total > 0xFFFFFFFFull) failed = 2;
    offsets[stream + 1] = (uint32_t)total;
  }
  uint16_t* joined = NULL;
  if (!failed) {
    joined = (uint16_t*)malloc((total ? total : 1) * sizeof(uint16_t));
    if (!joined) failed = 1;
  }
  if (!failed) {
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
    for (int64_t stream = 0; stream < streams; ++stream) {
      if (lists[stream].size) memcpy(joined + offsets[stream], lists[stream].words, lists[stream].size * sizeof(uint16_t));
    }
  }
  for (int64_t stream = 0; stream < streams; ++stream) free(lists[stream].words);
  free(lists);
  free(coded_before);
  *payload = joined;
  return failed == 0 ? 0 : (failed == 2 ? -2 : -1);
}

void hc_free(void* p) { free(p); }
