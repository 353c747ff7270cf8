/* entropack_hip.h -- C ABI of libentropack_hip.so: the MI355X (gfx950) lane of the lattice_rans decode path.
 *
 * Every pointer named *_dev is a device pointer (e.g. torch `tensor.data_ptr()`), every *_host pointer is host
 * memory. No entry point allocates or frees device memory and none synchronises the stream unless it says so;
 * work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the default stream). All functions return
 * 0 (EP_HIP_OK) or one of the EP_HIP_E* codes below; ep_hip_error_string() names them.
 *
 * The reference has no C ABI: its CUDA lane hands raw pointers and numpy scalars to CuPy-compiled kernels. Each
 * entry point below cites the reference interface it stands in for (paths relative to the reference root).
 */
#ifndef ENTROPACK_HIP_H
#define ENTROPACK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EP_HIP_ABI_VERSION 2

enum ep_hip_status {
  EP_HIP_OK = 0,
  EP_HIP_EINVAL = 1,        /* a size, alignment or enum argument is out of range */
  EP_HIP_EUNSUPPORTED = 2,  /* valid request this build has no kernel for */
  EP_HIP_ERUNTIME = 3,      /* a HIP runtime call failed; ep_hip_last_runtime_error() has the hipError_t */
  EP_HIP_ENODEVICE = 4,     /* no gfx950 device visible */
  EP_HIP_ETOOLARGE = 5      /* the request needs more scratch memory than the library's fixed, statically allocated buffer holds */
};

/* Output container kinds. 0..12 keep the numbering of the reference's store kinds
 * (entropack/schemes/lattice_rans/cuda.py:65-68, lattice_rans.cu:525-539); bf16 is its own kind here instead of
 * a separate kernel family. */
enum ep_hip_store_kind {
  EP_STORE_F32 = 0, EP_STORE_F16 = 1, EP_STORE_F8E4M3FN = 2, EP_STORE_F8E5M2 = 3,
  EP_STORE_I8 = 4, EP_STORE_I16 = 5, EP_STORE_I32 = 6, EP_STORE_I64 = 7,
  EP_STORE_U8 = 8, EP_STORE_U16 = 9, EP_STORE_U32 = 10, EP_STORE_U64 = 11,
  EP_STORE_BOOL = 12, EP_STORE_BF16 = 13
};

/* How a plan holds the slot -> (symbol, frequency, slot - cdf) map. The reference chooses among "shared",
 * "packed" and "wide" tables (entropack/schemes/lattice_rans/cuda.py:600-610,697-741); all decode to identical
 * output, and so do these. */
enum ep_hip_table_kind {
  EP_TABLE_GLOBAL64 = 0,    /* u64 per slot in HBM/L2, any prob_bits 9..15, any alphabet */
  EP_TABLE_LDS_BYTE = 1,    /* u32 per slot, LDS-resident; prob_bits <= 11, every field value in [-128, 127] */
  EP_TABLE_LDS_WIDE = 2,    /* u32 per slot, LDS-resident; prob_bits <= 11, alphabets <= 1024, frequencies < 2048 */
  EP_TABLE_LDS_RANK = 3,    /* LDS-resident rank/select form: per 32 slots a bitmap of symbol ends + running symbol count,
                               per present symbol freq | cdf << 16 and an int16 value; any prob_bits whose tables fit LDS */
  EP_TABLE_LDS_SYM = 4      /* two-level, LDS-resident: u8 per slot (the value + 128) and, per value, one 8-byte entry: freq plus a
                               parity mark, and cdf plus the value as a half-precision number (the kernel multiplies it with
                               the row scale without an integer conversion); a quarter of LDS_BYTE's size, so two workgroups
                               share a CU. Same conditions as LDS_BYTE. LDS_BYTE plans at prob_bits 11 carry it as a second
                               section (sym_offset) that large launches use; as a plan's own kind (force_kind only) every
                               launch uses it */
};

/* Device-side error flag values written (first one wins) to *error_dev by the decode kernels; same meaning as the
 * reference's set_error codes (lattice_rans.cu:51-53,777,799). */
enum ep_hip_decode_error {
  EP_DECODE_OK = 0,
  EP_DECODE_OVERREAD = 2,      /* renormalisation would read below the tile's first payload word */
  EP_DECODE_NOT_CONSUMED = 3,  /* tile ended with unread words or a lane state != 2^15 */
  EP_DECODE_BAD_OFFSETS = 4    /* offsets[t] > offsets[t+1] or offsets[t+1] > payload_words */
};

typedef struct ep_hip_device_info {
  int device;                 /* HIP device ordinal */
  int compute_units;
  int lds_bytes_per_block;    /* largest LDS allocation one workgroup may make */
  int wavefront_size;
  int is_gfx950;              /* 1 when gcnArchName starts with "gfx950" */
  char arch[64];
} ep_hip_device_info;

typedef struct ep_hip_plan_desc {
  int table_kind;             /* enum ep_hip_table_kind chosen for this container */
  int prob_bits;
  size_t table_bytes;         /* size of the device buffer ep_hip_plan_build fills (256-byte aligned start needed) */
  int lds_bytes;              /* dynamic LDS the decode kernel will request (0 for GLOBAL64) */
  int max_alphabet;
  int alphabet_sum;
  int sym_offset;             /* byte offset of the LDS_SYM section inside the plan buffer, 0 = none */
  int present_offset[18];     /* LDS_RANK: symbols with non-zero frequency in field streams before stream s (index s),
                                 [17] = their total; zero for the other kinds */
  int rank_values_half;       /* LDS_RANK: 1 = the value table holds lattice coordinates in half precision (every value is
                                 small enough to be exact there), 0 = 16-bit integers */
} ep_hip_plan_desc;

/* Library / device ------------------------------------------------------------------------------------------ */

int ep_hip_abi_version(void);
const char* ep_hip_error_string(int status);
int ep_hip_last_runtime_error(void);   /* hipError_t of the last failed runtime call on this thread, 0 if none */

/* Stands in for the reference's probe() + caps() (entropack/backends/cuda/__init__.py:4-12,
 * entropack/backends/cuda/device.py:66-81). `device` < 0 = current device. */
int ep_hip_device_query(int device, ep_hip_device_info* info);

/* Plan ------------------------------------------------------------------------------------------------------ */

/* Chooses the table representation from host copies of the container's stream_meta (int32[17][4] =
 * n_symbols, sym_min, freq_offset, alphabet) and freq_tables (u16[n_freq]), and validates them (offsets
 * contiguous, every stream's frequencies sum to 2^prob_bits). Pure host code, no GPU needed. `tile_elements` is
 * the container's layout[2] (must be positive); tiles of more than 2^18 vectors (tile_elements above 2 359 296) get
 * EP_TABLE_GLOBAL64, the LDS forms do not address them.
 * Reference: _decode_plan's representation choice, entropack/schemes/lattice_rans/cuda.py:697-732.
 * `force_kind` < 0 lets the library choose; otherwise it must be a kind the container qualifies for. */
int ep_hip_plan_describe(const int32_t* stream_meta_host, const uint16_t* freq_tables_host, size_t n_freq,
                         int prob_bits, int tile_elements, int lds_limit_bytes, int force_kind,
                         ep_hip_plan_desc* desc);

/* Builds the decode tables on the device, from the container's own device buffers, into `tables_dev`
 * (desc->table_bytes bytes, caller-allocated, 256-byte aligned). Asynchronous on `stream`.
 * Reference: _shared_tables / _packed_tables / _wide_tables (host numpy + upload),
 * entropack/schemes/lattice_rans/cuda.py:647-679. */
int ep_hip_plan_build(const int32_t* stream_meta_dev, const uint16_t* freq_tables_dev, const ep_hip_plan_desc* desc,
                      void* tables_dev, void* stream);

/* Decode ---------------------------------------------------------------------------------------------------- */

/* Entropy-decodes every tile and reconstructs straight into `out_dev` ([rows][cols_padded] of `store_kind`,
 * row-major, 16-byte aligned): rANS symbol steps, shared renormalisation, field minima, E8 point, row scale and
 * container cast, in one kernel. payload_dev must be 4-byte aligned. `error_dev` (int32, caller-zeroed) receives
 * an ep_hip_decode_error; it is never read back here. EP_HIP_EUNSUPPORTED for an LDS plan with tiles of more than
 * 2^18 vectors (ep_hip_plan_describe never makes one unless forced).
 * Reference: decode() + _decode_launch() and the e8_decode_vector_* kernels they launch,
 * entropack/schemes/lattice_rans/cuda.py:744-805, lattice_rans.cu:732-1141. */
int ep_hip_decode_lattice(const uint16_t* payload_dev, uint64_t payload_words, const uint32_t* offsets_dev,
                          const uint32_t* states_dev, const float* scales_dev, const void* tables_dev,
                          const ep_hip_plan_desc* desc, void* out_dev, int store_kind, int64_t rows,
                          int64_t cols_padded, int tile_elements, int32_t* error_dev, void* stream);

/* The table form ep_hip_decode_lattice uses for a container of this geometry: desc->table_kind, except that
 * LDS_BYTE plans with a two-level section (sym_offset != 0) take EP_TABLE_LDS_SYM once the launch has more tile pairs
 * than 16 waves on every one of `compute_units` CUs can hold. Host only; -1 on bad arguments. */
int ep_hip_decode_table_kind(const ep_hip_plan_desc* desc, int store_kind, int64_t rows, int64_t cols_padded,
                             int tile_elements, int compute_units);

/* Lossless decode ----------------------------------------------------------------------------------------------- */

/* Decodes a tile_ans container (payload u16[W], offsets u32[lanes * tiles + 1], states u32[tiles * coded lanes][32],
 * decode_tables u32[lanes][2^prob_bits], layout = tile_elements, prob_bits, lanes, elements) into `out_dev`, the
 * tensor's storage (elements * lanes bytes, element-aligned). `lane_modes_host` is a host copy of the container's
 * lane_modes (0 = coded, 1 = raw); lanes is 1, 2, 4 or 8. `error_dev` as for ep_hip_decode_lattice (a stream that
 * ends with unread words reports 3, one that runs out 2, bad offsets / raw lengths 4).
 * Reference: decode() and the tile_ans_decode_* kernels it launches, entropack/schemes/tile_ans/cuda.py:117-170,
 * tile_ans.cu:175-470. */
int ep_hip_decode_tile_ans(const uint16_t* payload_dev, uint64_t payload_words, const uint32_t* offsets_dev,
                           const uint32_t* states_dev, const uint32_t* decode_tables_dev,
                           const uint8_t* lane_modes_host, int64_t tile_elements, int prob_bits, int num_lanes,
                           int64_t num_elements, void* out_dev, int32_t* error_dev, void* stream);

/* Batched decode --------------------------------------------------------------------------------------------- */

/* One container of a batch: the arguments of ep_hip_decode_lattice, with the output given as a byte offset
 * (a multiple of 16) into an arena the caller passes at launch time. */
typedef struct ep_hip_decode_job {
  const uint16_t* payload_dev;
  uint64_t payload_words;
  const uint32_t* offsets_dev;
  const uint32_t* states_dev;
  const float* scales_dev;
  const void* tables_dev;
  const ep_hip_plan_desc* desc;     /* host pointer, read only while planning */
  uint64_t out_offset;
  int store_kind;
  int tile_elements;
  int64_t rows;
  int64_t cols_padded;
  int32_t* error_dev;
} ep_hip_decode_job;

/* Plans one pass over many containers (a whole state_dict): containers that share a kernel variant are decoded
 * by one launch whose workgroups each take a slice of one container, so small layers fill the device together
 * instead of one under-filled launch each. Pure host code. With `blob_host` NULL only `*blob_bytes` is written
 * (the size to allocate); otherwise `*blob_bytes` is the capacity of `blob_host`, which receives the plan. The
 * caller uploads the same bytes to the device (256-byte aligned) and keeps both copies for every launch.
 * `compute_units` sizes the slices (ep_hip_device_info.compute_units).
 * Reference: the per-layer loop a caller of decode() writes, entropack/linear/linear.py:125-130 over a model;
 * the reference has no batched entry. */
int ep_hip_batch_plan(const ep_hip_decode_job* jobs, int n_jobs, int compute_units, void* blob_host, size_t* blob_bytes);

/* Launches a planned batch on `stream`: job i writes at out_arena_dev + jobs[i].out_offset. Asynchronous. */
int ep_hip_decode_lattice_batch(const void* blob_host, const void* blob_dev, void* out_arena_dev, void* stream);


/* Linear ---------------------------------------------------------------------------------------------------- */

/* Element kinds of GEMM outputs, biases and quantiser inputs. */
enum ep_hip_float_kind { EP_FLOAT_BF16 = 0, EP_FLOAT_F16 = 1, EP_FLOAT_F32 = 2 };

/* y[M][N] = x[M][K] . w[N][K]^T (+ bias[N]): bf16 operands (rows ldx / ldw elements apart, 16-byte aligned, K a
 * multiple of 8), f32 accumulation on the matrix cores, result and bias of kind `out_kind`.
 * Reference: the F.linear call of CompressedLinear.forward, entropack/linear/linear.py:163-165. */
int ep_hip_gemm_bf16(const void* x_dev, const void* w_dev, const void* bias_dev, void* y_dev, int64_t M, int64_t N,
                     int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int out_kind, void* stream);

/* The same products with K split over blocks, for products too small to occupy the device otherwise; partial sums (f32,
 * or exact int32 for the int8 product) go to `workspace_dev` (16-byte aligned, at least
 * ep_hip_gemm_skinny_workspace(M, N, bytes of one row of K, compute_units) bytes, contents irrelevant on entry) and a second
 * kernel adds them, applies the same epilogue as ep_hip_gemm_bf16 / ep_hip_gemm_i8 and rounds once.
 *  - M <= 128: reading W once bounds the time; blocks of 128 weight rows, K split so that every CU streams weights.
 *  - M > 128: 128 x 128 tiles (operand tiles loaded straight into LDS, four stages), K split over 2..8 blocks per tile when
 *    the tiles number at most half the CUs and each block keeps a whole number of four 128-byte K steps, at least eight.
 *    Where no such split exists ep_hip_gemm_skinny_workspace returns 0 and the entry points EP_HIP_EUNSUPPORTED: the
 *    product then belongs to ep_hip_gemm_bf16 / ep_hip_gemm_i8.
 * f32 sums are added in the order of the slices, so a bf16 product can differ from ep_hip_gemm_bf16's in the last bit of
 * the f32 sum; the int8 product is the same bits. Same operand rules as those entry points. Reference: the F.linear call
 * of CompressedLinear.forward and the int8 GEMM of CompressedINT8Linear at small batch, entropack/linear/linear.py:163-165,
 * 485-490. */
size_t ep_hip_gemm_skinny_workspace(int64_t M, int64_t N, int64_t k_bytes, int compute_units);

/* 1 when ep_hip_gemm_bf16 / ep_hip_gemm_i8 multiply this product with blocks of 64 x 64: its 128 x 128 tiles would occupy at
 * most half of `compute_units`, its 64 x 64 tiles fit them in one round, and a row of K (`k_bytes` bytes) is a whole number of
 * four 128-byte steps, at least eight. These are the products on which this library's kernel is ahead of the vendor
 * library's on an MI355X (256 x 3072 x 3072 bf16: 16.9 us against 19.4 us with the weight coming from memory), which is what
 * a caller that has both may want to know; 0 otherwise. Host only. No counterpart in the reference (it has one product,
 * F.linear, entropack/linear/linear.py:163-165). */
int ep_hip_gemm_takes_small_blocks(int64_t M, int64_t N, int64_t k_bytes, int compute_units);
int ep_hip_gemm_bf16_skinny(const void* x_dev, const void* w_dev, const void* bias_dev, void* y_dev, int64_t M, int64_t N,
                            int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int out_kind, int compute_units,
                            void* workspace_dev, size_t workspace_bytes, void* stream);
int ep_hip_gemm_i8_skinny(const int8_t* a_dev, const int8_t* b_dev, const float* scale_a_dev, const float* scale_b_dev,
                          const void* bias_dev, void* y_dev, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                          int64_t ldy, int out_kind, int compute_units, void* workspace_dev, size_t workspace_bytes,
                          void* stream);

/* y[M][N] = (a[M][K] . b[N][K]^T)_int32 -> f32 * scale_a[m] * scale_b[n] (+ bias[n]) -> out_kind. K a multiple of 16.
 * Reference: int8_gemm / _int8_gemm_kernel, entropack/linear/quant_kernels.py:15-54,81-93. */
int ep_hip_gemm_i8(const int8_t* a_dev, const int8_t* b_dev, const float* scale_a_dev, const float* scale_b_dev,
                   const void* bias_dev, void* y_dev, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                   int64_t ldy, int out_kind, void* stream);

/* Per-row symmetric int8 quantisation of activations: scale = max(absmax / 127, FLT_EPSILON),
 * code = clamp(rint(x / scale), -127, 127). codes_dev is [rows][K] contiguous.
 * Reference: quantize_rows / _quantize_rows_kernel, entropack/linear/quant_kernels.py:56-79,95-106. */
int ep_hip_quantize_rows(const void* x_dev, int in_kind, int64_t rows, int64_t K, int64_t ldx, int8_t* codes_dev,
                         float* scales_dev, void* stream);

/* The same on block-rotated activations: every `group` consecutive elements of a row (group = 4, 16, 64 or 256,
 * dividing K) are multiplied with the symmetric orthogonal matrix kron^k([[1,1,1,-1],[1,1,-1,1],[1,-1,1,1],[-1,1,1,1]])
 * / sqrt(group), the product is rounded to the activation dtype, and the rotated row is quantised as above. Sums are
 * formed in float32 by radix-4 stages, not in the order of a matrix product, so a code can differ by one from a
 * library product's where a value sits on a rounding boundary. Needs K and ldx multiples of 4 and x_dev aligned to
 * four elements; EP_HIP_EUNSUPPORTED for groups above 256 or unaligned rows (rotate with a library product, then
 * ep_hip_quantize_rows).
 * Reference: rotate_activation followed by quantize_rows in CompressedINT8Linear._forward8,
 * entropack/linear/convrot.py:34-53, entropack/linear/linear.py:463-466,338-341. */
int ep_hip_rotate_quantize_rows(const void* x_dev, int in_kind, int64_t rows, int64_t K, int64_t ldx, int group,
                                int8_t* codes_dev, float* scales_dev, void* stream);

/* y[m_rows][rows] = x[m_rows][cols_padded] * W^T (+ bias) for one to four activation rows, W given as a compressed
 * container (`weight`: the arguments of ep_hip_decode_lattice; out_offset is ignored, store_kind must be
 * EP_STORE_BF16): every decoded vector is rounded to bf16 as the store would, multiplied with the matching
 * activations in registers and reduced into `workspace_dev` (m_rows * rows floats, zeroed here), so the dense weight is
 * never written or re-read. x is bf16 with row stride `ldx` elements (a multiple of 8, 16-byte aligned base); bias
 * (may be NULL) and y have type `out_kind` (ep_hip_float_kind), y with row stride `ldy`. Returns EP_HIP_EUNSUPPORTED
 * for more than four rows, fewer than 256 columns, non-bf16 weights or a GLOBAL64 plan: the caller then decodes and
 * multiplies separately. Sums are accumulated with floating-point atomics, so the last bits can vary from run to run.
 * Reference: the memory-bound use of CompressedLinear.forward, entropack/linear/linear.py:163-165 (decode, then
 * F.linear); the reference has no fused form. */
int ep_hip_linear_fused_bf16(const ep_hip_decode_job* weight, const void* x_dev, int64_t m_rows, int64_t ldx,
                             const void* bias_dev, void* y_dev, int64_t ldy, int out_kind, float* workspace_dev,
                             void* stream);

/* ep_hip_linear_fused_bf16 for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc): same arguments, results and errors, but the f32 accumulator is a fixed array inside
 * the library's device image (EP_HIP_STATIC_ACCUMULATOR_FLOATS floats = 1 MiB on every GPU the library runs on, held
 * until the process ends) instead of a caller's workspace. Nothing is allocated or freed, here or in any routine it
 * calls. m_rows * weight->rows above EP_HIP_STATIC_ACCUMULATOR_FLOATS returns EP_HIP_ETOOLARGE. Every call on a GPU
 * uses that GPU's one array (cleared by a kernel at the start of each call): calls that overlap on one GPU, from
 * different streams or threads, race; calls on one stream, or otherwise ordered, are safe. The array's address on a
 * device is looked up by ep_hip_device_query (when that device is current) or by the first call on the device: one of
 * the two must have happened before a call is captured into a HIP graph.
 * No counterpart in the reference, whose lane allocates its outputs with torch.empty
 * (entropack/schemes/lattice_rans/cuda.py:794). */
#define EP_HIP_STATIC_ACCUMULATOR_FLOATS (1 << 18)
int ep_hip_linear_fused_bf16_static(const ep_hip_decode_job* weight, const void* x_dev, int64_t m_rows, int64_t ldx,
                                    const void* bias_dev, void* y_dev, int64_t ldy, int out_kind, void* stream);

/* Decode-to-GEMM through LDS ------------------------------------------------------------------------------------ *
 *
 * y[m_rows][rows] = x[m_rows][cols_padded] * W^T (+ bias) for any number of activation rows, W a compressed container,
 * with the decoded weight handed from the rANS lanes to the matrix cores through LDS: the dense weight is never written
 * to memory. A workgroup decodes up to EP_HIP_FUSED_SLOTS tiles whose first vectors lie at (nearly) the same position
 * inside a weight row, because only such tiles supply many weight rows at one k, which is what a matrix-core operand is;
 * ep_hip_fused_plan groups a container's tiles that way (host only, pure arithmetic on the geometry), the caller copies
 * the batches to the device once per container and passes them to every product.
 * Reference: CompressedLinear.forward / _reconstruct, entropack/linear/linear.py:125-130,163-165 (decode the whole weight,
 * then F.linear); the reference has no fused form (its lattice_rans.cu:21-23 fuses decode, reconstruction and cast only). */
#define EP_HIP_FUSED_SLOTS 32        /* tiles per batch: one per 32-lane half of sixteen waves */
#define EP_HIP_FUSED_MAX_SKEW 31     /* largest distance, in vectors, between the in-row positions of a batch's tiles */

typedef struct ep_hip_fused_batch {
  int32_t base;                          /* in-row vector position (a multiple of 4) that aligned index 0 of this batch stands for */
  int32_t reserved[3];
  int32_t tile[EP_HIP_FUSED_SLOTS];      /* tile index, or -1 for an unused slot */
  int32_t delta[EP_HIP_FUSED_SLOTS];     /* (tile * tile_vectors) mod vectors_per_row - base, 0 .. EP_HIP_FUSED_MAX_SKEW */
} ep_hip_fused_batch;

/* Groups the tiles of a rows x cols_padded container with `tile_elements` symbols per tile into batches. With
 * batches_host NULL only counts them (*n_batches); else fills at most `capacity` batches. EP_HIP_EUNSUPPORTED for rows of
 * fewer than 32 vectors or whose number of vectors is no multiple of four (cols_padded not a multiple of 32). */
int ep_hip_fused_plan(int64_t rows, int64_t cols_padded, int tile_elements, ep_hip_fused_batch* batches_host, int capacity,
                      int* n_batches);

/* The product. `weight` as for ep_hip_linear_fused_bf16 (store_kind EP_STORE_BF16; the decoded values are rounded to
 * bf16 exactly as ep_hip_decode_lattice stores them); `batches_dev` = the device copy of ep_hip_fused_plan's output for
 * the same geometry. x is bf16 with row stride `ldx` elements (a multiple of 8, 16-byte aligned base); bias (may be NULL)
 * and y have type `out_kind`; `workspace_dev` (256-byte aligned) holds ep_hip_linear_fused_mfma_workspace(..., 0) bytes
 * and need not be cleared: the kernel writes every partial sum of an output (one per tile the weight row touches and half
 * of the k steps) into a plane of its own with plain stores, and a second kernel adds them in a fixed order, then the
 * bias, and rounds once, so results are the same from run to run. EP_HIP_EUNSUPPORTED unless the plan has the two-level
 * tables of prob_bits 11 (byte-valued symbols), which is what the default encoder settings give up to 7 bpp, and
 * cols_padded is a multiple of 32: the caller then decodes and multiplies separately. */
int ep_hip_linear_fused_mfma_bf16(const ep_hip_decode_job* weight, const ep_hip_fused_batch* batches_dev, int n_batches,
                                  const void* x_dev, int64_t m_rows, int64_t ldx, const void* bias_dev, void* y_dev, int64_t ldy,
                                  int out_kind, void* workspace_dev, void* stream);

/* The same for W8A8: `weight` is a container of int8 codes (store_kind EP_STORE_I8, decoded with the rounding and clamp of
 * the int8 store), a_dev the int8 activation codes of ep_hip_quantize_rows with row stride `lda` bytes (a multiple of 16),
 * scale_a_dev[m_rows] / scale_b_dev[rows] the activation and weight row scales:
 *   y[m][n] = cast(f32(sum_k a[m][k] * w[n][k]) * scale_a[m] * scale_b[n] + bias[n]),
 * the int32 sums exact (partial sums are added as integers), the epilogue three single-rounded float operations: the same
 * bits as ep_hip_gemm_i8 on the decoded codes. Workspace: ep_hip_linear_fused_mfma_workspace(..., 1) bytes.
 * Reference: CompressedINT8Linear._forward8 / _gemm, entropack/linear/linear.py:362-385,485-490 (decode the codes, then the
 * Triton int8 GEMM of entropack/linear/quant_kernels.py:15-54). */
int ep_hip_linear_fused_mfma_i8(const ep_hip_decode_job* weight, const ep_hip_fused_batch* batches_dev, int n_batches,
                                const int8_t* a_dev, int64_t m_rows, int64_t lda, const float* scale_a_dev, const float* scale_b_dev,
                                const void* bias_dev, void* y_dev, int64_t ldy, int out_kind, void* workspace_dev, void* stream);
size_t ep_hip_linear_fused_mfma_workspace(int64_t rows, int64_t cols_padded, int tile_elements, int64_t m_rows, int int8);

/* Encoder (the step before the path) -------------------------------------------------------------------------- *
 *
 * The device form of the lattice_rans encoder, one entry point per kernel of the reference's CUDA lane. All pointers are
 * device pointers; nothing is allocated, nothing synchronises, every launch goes to `stream`. From the same inputs
 * the integer outputs (coset bits, fields, summary, bins, states, offsets, payload) are bit-identical to the CPU
 * encoder's (entropack/schemes/lattice_rans/eager.py:18-58, rans.py:133-186), as the reference states of its own
 * kernels (lattice_rans.cu:3-18); the refitted row scales are float32 sums added in a fixed order of this library's own.
 * A coset bit is 0 (point of D8) or 1 (point of D8 + 1/2); the fields of a vector are z0..z6 and m, where the point is
 * (z0..z6, 2 m + parity(z0 + .. + z6)) + coset / 2. Stream 0 carries the coset bits, stream 1 + 2 f + c field f of the
 * vectors of coset c. */

#define EP_HIP_ENCODE_SUMMARY_WORDS 33

/* Quantises `rows` rows of x[.][cols] (float32, 16-byte aligned, cols a multiple of 8): row i of the output is row
 * row_index_dev[i] of x (row i when row_index_dev is NULL); y = (x / rms[row]) / scale, nearest E8 point, the first of
 * equally near ones in the order D8, D8 + 1/2. coset_dev: int8[rows * cols / 8]; fields_dev: int32[rows * cols / 8][8]
 * (16-byte aligned). summary_dev: int64[EP_HIP_ENCODE_SUMMARY_WORDS], set by the call: [2 k], [2 k + 1] = least and
 * greatest value of field stream k = 2 f + c (INT64_MAX, INT64_MIN for a stream without symbols), [32] = number of
 * vectors of coset 1. Replaces the quantise launch and the min/max pass of the reference's CUDA lane
 * (entropack/schemes/lattice_rans/cuda.py:115-139, lattice_rans.cu:224,334). */
int ep_hip_encode_quantize(const float* x_dev, const float* rms_dev, int64_t cols, float scale, const int64_t* row_index_dev,
                           int64_t rows, int8_t* coset_dev, int32_t* fields_dev, int64_t* summary_dev, void* stream);

/* Counts the symbols of all 17 streams into bins_dev (uint64[total_bins], cleared by the call): a symbol of value z of
 * stream s is counted in bin bin_rel_dev[s] + z, i.e. bin_rel_dev[s] = first bin of the stream - its least value
 * (int32[17]). Values whose bin falls outside [0, total_bins) are not counted. Replaces cuda.py:181-221
 * (e8_histogram_kernel, lattice_rans.cu:376). */
int ep_hip_encode_histogram(const int8_t* coset_dev, const int32_t* fields_dev, int64_t vectors, const int32_t* bin_rel_dev,
                            int32_t total_bins, uint64_t* bins_dev, void* stream);

/* Least-squares row scales against the chosen points: scales_dev[r] = max(sum(x p) / sum(p p), 1e-12) in float32, or
 * scale * rms[r] for a row whose points are all zero; row_sse_dev (may be NULL) receives the squared error of every row
 * at that scale, max(sum(x x) - sum(x p)^2 / sum(p p), 0), or sum(x x) for such a row. Replaces cuda.py:142-158 (the
 * refit kernels, lattice_rans.cu:313). */
int ep_hip_encode_row_scales(const float* x_dev, const float* rms_dev, int64_t cols, float scale, int64_t rows,
                             const int8_t* coset_dev, const int32_t* fields_dev, float* scales_dev, float* row_sse_dev,
                             void* stream);

/* Tiled 32-way interleaved rANS encode of `vectors` vectors in tiles of `tile_vectors` (>= 32). entries_dev:
 * uint64[total_entries], for every table position frequency | cumulative frequency << 16 in the low half and
 * min(floor(2^32 / frequency), 2^32 - 1) in the high half; table_rel_dev: int32[17], first position of stream s - its
 * least value. states_dev: uint32[tiles][32]; tile_words_dev: uint32[tiles], the number of
 * payload words of each tile, which the tile leaves at scratch_dev[tile * tile_vectors * 9 ..) (uint16[tiles *
 * tile_vectors * 9]). *error_dev (int32, cleared by the caller) becomes 1 when a symbol lies outside the tables or has
 * frequency 0; the outputs are then not a valid container. Replaces cuda.py:520-541 (e8_rans_encode_vector_kernel,
 * lattice_rans.cu:400). */
int ep_hip_encode_rans(const int8_t* coset_dev, const int32_t* fields_dev, int64_t vectors, const uint64_t* entries_dev,
                       const int32_t* table_rel_dev, int32_t total_entries, int prob_bits, int tile_vectors, uint32_t* states_dev,
                       uint32_t* tile_words_dev, uint16_t* scratch_dev, int32_t* error_dev, void* stream);

/* offsets_dev[0] = 0, offsets_dev[t + 1] = tile_words_dev[0] + .. + tile_words_dev[t] modulo 2^32 (uint32[tiles + 1]);
 * *total_words_dev (uint64, 8-byte aligned) = the sum itself, which the caller compares with 2^32 and sizes the payload
 * by. Replaces the cumulative sum of cuda.py:542-551. */
int ep_hip_encode_offsets(const uint32_t* tile_words_dev, int64_t tiles, uint32_t* offsets_dev, uint64_t* total_words_dev, void* stream);

/* payload_dev[offsets_dev[t] ..) = the words stream t left at scratch_dev[t * stride_words ..): stride_words =
 * tile_vectors * 9 after ep_hip_encode_rans, the scratch stride after ep_hip_tile_ans_encode; payload_dev 4-byte
 * aligned (EP_HIP_EINVAL otherwise: words are stored in pairs). Replaces cuda.py:552-557
 * (e8_compact_kernel, lattice_rans.cu:467) and tile_ans/cuda.py:110-115 (tile_ans_compact_kernel, tile_ans.cu:157). */
int ep_hip_encode_gather(const uint16_t* scratch_dev, const uint32_t* offsets_dev, int64_t tiles, int64_t stride_words,
                         uint16_t* payload_dev, void* stream);

/* The lossless tile_ans encoder. An element is num_lanes (1, 2, 4 or 8) bytes; byte b of elements [t * tile_elements, ..)
 * is stream b * tiles + t. All integer work: the streams are bit-identical to the CPU encoder's
 * (entropack/schemes/tile_ans/eager.py:145-228).
 *
 * ep_hip_tile_ans_histogram: counts_dev[b][s] (uint64[num_lanes][256], cleared by the call) = number of elements whose
 * byte b is s; bytes_dev 16-byte aligned. Replaces tile_ans/cuda.py:31-47 (tile_ans_histogram_kernel, tile_ans.cu:27).
 *
 * ep_hip_tile_ans_encode: entries_dev uint64[num_lanes][256] = frequency | cumulative frequency << 16 in the low half,
 * min(floor(2^32 / frequency), 2^32 - 1) in the high half (anything for symbols that do not occur); lane_raw_host
 * (host memory, num_lanes bytes): non-zero = the lane is stored raw, two bytes per word. states_dev: uint32[coded lanes *
 * tiles][32], coded lanes in lane order (may be NULL when every lane is raw); stream_words_dev: uint32[num_lanes * tiles];
 * stream s leaves its words at scratch_dev[s * scratch_stride_words ..), scratch_stride_words >= tile_elements.
 * *error_dev (cleared by the caller) becomes 1 when a coded symbol has frequency 0. Follow with ep_hip_encode_offsets and
 * ep_hip_encode_gather. Replaces tile_ans/cuda.py:84-100 (tile_ans_encode_kernel, tile_ans.cu:67). */
int ep_hip_tile_ans_histogram(const uint8_t* bytes_dev, int64_t num_elements, int num_lanes, uint64_t* counts_dev, void* stream);
int ep_hip_tile_ans_encode(const uint8_t* bytes_dev, int64_t num_elements, int num_lanes, int64_t tile_elements, int prob_bits,
                           const uint64_t* entries_dev, const uint8_t* lane_raw_host, uint32_t* states_dev, uint32_t* stream_words_dev,
                           uint16_t* scratch_dev, int64_t scratch_stride_words, int32_t* error_dev, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ENTROPACK_HIP_H */
