/*
 * sptmm.h -- C ABI of the MI355X (gfx950) SpTMM engine.
 *
 * Multiplication-free ternary-weight sparse matrix multiply
 *     C[m][n] = sum_{k in pos(n)} X[m][k] - sum_{k in neg(n)} X[m][k]
 * with three encodings of the same ternary K x N matrix W:
 *   u16    row-index lists per column (reference "SpTMM",       -row_split3_small)
 *   delta  8/16-bit gaps of the sorted lists (reference "SpTMM-delta", -row_split_delta2)
 *   i2s    2-bit packed dense ternary, 16 weights per 32-bit word (reference -i2s)
 *
 * Plain pointers and sizes only; no HIP or torch types.  `stream` arguments are
 * a hipStream_t passed as void* (NULL = the default stream).  Every function
 * returns SPTMM_OK (0) or a negative sptmm_status; sptmm_last_error() gives the
 * text of the last failure on the calling thread.  The library never exits or
 * aborts.  Calls on one sptmm_weights object from several threads are safe as
 * long as each uses its own X/C buffers (the object is immutable after upload).
 *
 * The reference has no library boundary of its own: its only interface is the
 * `rcr` command line plus the kernels' argument lists.  Each entry point below
 * names the reference code (file:line under the reference checkout) it stands
 * in for.
 */
#ifndef SPTMM_H
#define SPTMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum sptmm_status {
    SPTMM_OK = 0,
    SPTMM_ERR_INVALID = -1,     /* argument or shape violates a documented rule   */
    SPTMM_ERR_UNSUPPORTED = -2, /* valid request this build cannot serve          */
    SPTMM_ERR_HIP = -3,         /* a HIP runtime call failed (see last_error)     */
    SPTMM_ERR_NOMEM = -4
} sptmm_status;

typedef enum sptmm_kind { SPTMM_KIND_U16 = 1, SPTMM_KIND_DELTA = 2, SPTMM_KIND_I2S = 3 } sptmm_kind;

typedef struct sptmm_devinfo {
    char name[128];
    char arch[64];
    int compute_units;
    int wave_size;
    int lds_bytes_per_workgroup; /* largest LDS allocation one workgroup may make */
    int l2_bytes;
    uint64_t hbm_bytes;
    double peak_hbm_gbps;        /* published peak used for roofline lines (8000 on MI355X) */
} sptmm_devinfo;

typedef struct sptmm_winfo {
    int kind;        /* sptmm_kind */
    int K, N, S;     /* S = nonzeros per column (0 for i2s) */
    int split_k;     /* lanes cooperating on one column (0 for i2s) */
    int delta_bits;  /* 8 or 16 for SPTMM_KIND_DELTA, else 0 */
    uint64_t stream_bytes; /* bytes of the weight stream one GEMV reads */
    int ragged;      /* 1: built from a matrix whose columns differ in nonzeros (S is 0 then) */
    uint64_t nnz;    /* nonzeros of the whole matrix */
    int k_tile;      /* wide streams: rows per K-tile (0 for every other stream) */
    int row_bytes;   /* 8-bit gap streams: bytes per row of the activation tile the visiting order was scheduled for,
                      * 1 (sptmm_*_rows with rows = 1) or 4; 0 for every other stream */
    int stones;      /* 1: 8-bit gap stream of a matrix too sparse for byte gaps throughout -- the activation tile keeps 16 zero
                      * slots behind every 96 rows, the stream holds tile positions, and a gap of more than 127 positions
                      * is walked over zero slots (entries that add nothing); 0 for every other stream */
} sptmm_winfo;

typedef struct sptmm_weights sptmm_weights; /* opaque; owns its device buffer */

const char *sptmm_last_error(void);
const char *sptmm_version(void);

/* ------------------------------------------------------------------ host side
 * Weight generator and format builders.  Pure host code (no GPU needed). */

/* Seeded ternary matrix of the benchmark: main.cu:246-276 (generator + sorted
 * +1/-1 row lists) with the RNG of macro.cuh:69-76.  pos/neg are [N][S/2];
 * W_colmajor (K*N bytes, column n at W + n*K) may be NULL.
 * Rules of main.cu:85-91: K,N multiples of 16, K < 65536, S even, K > S. */
int sptmm_generate_ternary(int K, int N, int S, int8_t *W_colmajor, uint16_t *pos, uint16_t *neg);

/* Row lists of an arbitrary balanced ternary matrix (exactly S/2 of each sign
 * per column, as main.cu:276 asserts). */
int sptmm_lists_from_dense(const int8_t *W_colmajor, int K, int N, int S, uint16_t *pos, uint16_t *neg);

/* Seeded int8 activations, uniform on [-127,127] (stands in for make_X,
 * main.cu:784-797, which is unseeded): xorshift32 stream, r % 255 - 127. */
int sptmm_make_x_i8(uint32_t seed, size_t count, int8_t *X);
/* Seeded ~N(0,1) activations for the float variants (the reference has none: its X is `char` everywhere,
 * main.cu:784-797): Box-Muller over the same xorshift32 stream, two values per pair of draws
 * (u1 = (r + 1) / (2^32 + 1), u2 = r / 2^32).  Either output may be NULL: X32 receives the floats, X16 their IEEE
 * half bits (round to nearest even). */
int sptmm_make_x_normal(uint32_t seed, size_t count, float *X32, uint16_t *X16);

/* The split_k this library would pick for a balanced matrix (kind: SPTMM_KIND_U16 or
 * SPTMM_KIND_DELTA) on a device with `compute_units` CUs (0: 256) -- what the upload calls use when
 * they are handed split_k = 0.  The reference leaves the choice to the command line
 * (main.cu:998, 1042, 1059); the result does not depend on it.  Negative status when no split
 * in 8..256 (gap streams: 8..64) divides S/2. */
int sptmm_choose_split_k(int kind, int N, int S, int compute_units);

/* Wave64 stream of the u16 lists; replaces the W_map_{8,16,32}_div layouts of
 * main.cu:343-374.  split_k in {8,16,32,64,128,256}; (S/2) % split_k == 0
 * (main.cu:564). */
size_t sptmm_pack_u16_bytes(int N, int S, int split_k);
int sptmm_pack_u16(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, void *out);
int sptmm_unpack_u16(const void *packed, int K, int N, int S, int split_k, uint16_t *pos, uint16_t *neg);

/* Gap streams; replaces W_map_delta2_d / W_map_delta2_div256 of main.cu:376-413.
 * Each lane owns a contiguous run of the sorted list: a 16-bit first row
 * followed by its gaps.  16-bit gaps are unsigned and ascending.  8-bit gaps are
 * SIGNED: a lane visits its run in an order chosen by the packer (steps within
 * -128..127) so that the 32 lanes of a half-wavefront gather from different LDS
 * banks.  sptmm_delta_bits() returns 8 when every in-run gap of the sorted lists
 * is at most 127, else 16 (the reference narrows silently, main.cu:380-383).
 * split_k in {8,16,32,64}. */
int sptmm_delta_bits(const uint16_t *pos, const uint16_t *neg, int N, int S, int split_k);
size_t sptmm_pack_delta_bytes(int N, int S, int split_k, int bits);
int sptmm_pack_delta(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int bits, void *out);
int sptmm_unpack_delta(const void *packed, int K, int N, int S, int split_k, int bits, uint16_t *pos, uint16_t *neg);
/* The same stream with the visiting order of the 8-bit gaps chosen for calls with `rows` activation
 * rows.  rows = 1: for an activation tile of ONE BYTE per row (int8, a single row: the GEMV of
 * main.cu:556-594 at M = 1), where the gather address is the running row itself and the LDS bank of a
 * row is (row / 4) mod 32; any other value: as sptmm_pack_delta (4-byte slots, bank = row mod 32).
 * Size, layout and sptmm_unpack_delta are the same either way; every GEMV entry point serves either
 * stream at any M, fastest at the M it was scheduled for.  No counterpart in the reference. */
int sptmm_pack_delta_rows(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int bits, int rows, void *out);

/* Ragged matrices: any K x N matrix over {-1,0,+1} (column n at W + n*K), columns
 * free to differ in nonzeros and in their +1/-1 split -- what a quantised model
 * tensor looks like.  No counterpart in the reference, whose generator and
 * kernels fix S/2 entries per sign and column (main.cu:90, 276, 564); its unused
 * "VCSC" arrays (main.cu:461-488) sketch per-column counts.  kind is
 * SPTMM_KIND_U16 (split_k 8..256) or SPTMM_KIND_DELTA (split_k 8..64).  The
 * stream opens with one entry count per wavefront task; a task pads its shorter
 * lists with entries on the zero rows K..K+63 that the activation tile keeps;
 * K + 64 must fit 16 bits.  *bits (gap streams): in 0 = pick, 8 or 16 = exactly that; out the
 * width used.  Byte gaps are signed (+-127 rows).  Where some gap of a lane's run is longer --
 * the reference's delta layout narrows every gap to u8 unchecked, main.cu:376-394 -- an 8-bit
 * stream holds positions in a tile that keeps 16 zero slots behind every 96 rows (preamble
 * magic "SPTS" instead of "SPTR", sptmm_winfo.stones) and walks the gap over zero slots: entries
 * that add nothing, at most one per 97 positions.  bits = 0 takes that stream when it is
 * smaller than 16-bit gaps throughout, else 16.  _bytes returns the stream size (0 on error);
 * *read_bytes is what one GEMV reads of it (tasks sit at a fixed stride). */
size_t sptmm_pack_ragged_bytes(const int8_t *W_colmajor, int K, int N, int kind, int split_k, int *bits, size_t *read_bytes,
                               int *n_min, int *n_max, uint64_t *nnz);
int sptmm_pack_ragged(const int8_t *W_colmajor, int K, int N, int kind, int split_k, int bits, void *out);
int sptmm_unpack_ragged(const void *packed, int K, int N, int kind, int split_k, int bits, int8_t *W_colmajor);
/* As sptmm_pack_ragged, gap streams scheduled for `rows` activation rows per call (see sptmm_pack_delta_rows). */
int sptmm_pack_ragged_rows(const int8_t *W_colmajor, int K, int N, int kind, int split_k, int bits, int rows, void *out);
/* Seeded matrix with independent entries: +1 with probability p_pos, -1 with
 * p_neg (xorshift32 of macro.cuh:69-76 per column, state seed ^ 0x9E3779B9*(n+1);
 * entry = top 24 bits of the next state against the two thresholds). */
int sptmm_generate_ternary_iid(int K, int N, uint32_t seed, double p_pos, double p_neg, int8_t *W_colmajor);
/* Dense matrix from 2-bit words in the reference's own order: word g of column n
 * at words[n*(K/16) + g] holds rows 16g..16g+15 (main.cu:176-196). */
int sptmm_dense_from_i2s_words(const uint32_t *words, int K, int N, int8_t *W_colmajor);

/* Wide streams: u16 lists or gap streams for activation tiles of 16 int8 rows (8 fp16 rows), cut
 * into K-tiles of k_tile rows so that such a tile fits the LDS: the stream is read ONCE for up to
 * 16 rows whatever K is (the reference reads its lists once per row, main.cu:567, and this
 * library's other streams once per 8 rows when a 16-row tile does not fit).  Any K x N matrix over
 * {-1,0,+1}; split_k in {8,16,32,64}; k_tile a multiple of 16 (sptmm_wide_k_tile gives the largest
 * that fits an LDS of the given size).  *bits as in the ragged packer.  The stream is
 * self-describing (a 512-byte header with the K-tile table; at most 16 K-tiles). */
int sptmm_wide_k_tile(int K, int lds_bytes);
size_t sptmm_pack_wide_bytes(const int8_t *W_colmajor, int K, int N, int kind, int split_k, int k_tile, int *bits, size_t *read_bytes,
                             uint64_t *nnz);
int sptmm_pack_wide(const int8_t *W_colmajor, int K, int N, int kind, int split_k, int k_tile, int bits, void *out);
int sptmm_unpack_wide(const void *packed, int K, int N, int8_t *W_colmajor);

/* i2s: 16 weights per word, code = w + 2, element e at bit 8*(e%4) + 2*(e/4)
 * (main.cu:176-192, decode bitnet_kernels.cuh:52-72).  Word order is this
 * library's own wave64 tiling, not the reference's (whose prepared matrix,
 * main.cu:194-196, does not match its kernel's addressing anyway). */
uint32_t sptmm_i2s_pack_word(const int8_t w16[16]);
void sptmm_i2s_decode_word(uint32_t word, int8_t w16[16]);
size_t sptmm_pack_i2s_bytes(int K, int N);
int sptmm_pack_i2s(const int8_t *W_colmajor, int K, int N, void *out);
int sptmm_unpack_i2s(const void *packed, int K, int N, int8_t *W_colmajor);

/* ---------------------------------------------------------------- device side */

/* Selects the device and reports what the roofline lines need. */
int sptmm_device_init(int device, sptmm_devinfo *out);

/* Host lists / dense matrix -> device stream.  Stand in for the cudaMalloc +
 * prepareW_map / prepareW_i2s sequence of main.cu:914-989 and 1851-1859.
 * split_k = 0 (here, in _upload_dense and in _upload_wide): sptmm_choose_split_k for the
 * current device (ragged matrices: from the mean nonzeros per column). */
int sptmm_weights_upload_u16(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, sptmm_weights **out);
int sptmm_weights_upload_delta(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, sptmm_weights **out);
/* The _rows forms say how many activation rows the calls on this stream will bring, and the stream is built for
 * that: rows > 8 gives a WIDE stream (sptmm_weights_upload_wide: the lists read once for up to 16 int8 rows, where an
 * ordinary stream serves such a call in passes of eight rows and reads the lists once per pass; info.k_tile != 0
 * says so; u16: only for split_k <= 64 or 0); rows = 0: no preference.  Any stream still serves any M. */
int sptmm_weights_upload_u16_rows(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int rows, sptmm_weights **out);
/* Gap stream scheduled for calls with `rows` activation rows (sptmm_pack_delta_rows): rows = 1 is
 * the stream for GEMVs (int8, M = 1); 0 = no preference (as sptmm_weights_upload_delta).
 * Byte gaps where every gap fits; else the smaller of 16-bit gaps and the 8-bit stream that
 * walks long gaps over zero slots of the tile (sptmm_pack_ragged; info.ragged and info.stones
 * are 1 then, info.S stays S). */
int sptmm_weights_upload_delta_rows(const uint16_t *pos, const uint16_t *neg, int K, int N, int S, int split_k, int rows, sptmm_weights **out);
int sptmm_weights_upload_i2s(const int8_t *W_colmajor, int K, int N, sptmm_weights **out);
/* Any ternary matrix -> device stream of the given kind (ragged u16 lists,
 * ragged gap stream, or i2s).  The GEMV entry points below serve it like any
 * other weights object. */
int sptmm_weights_upload_dense(const int8_t *W_colmajor, int K, int N, int kind, int split_k, sptmm_weights **out);
/* The same with a gap stream scheduled for `rows` activation rows per call (see sptmm_weights_upload_delta_rows). */
int sptmm_weights_upload_dense_rows(const int8_t *W_colmajor, int K, int N, int kind, int split_k, int rows, sptmm_weights **out);
/* Any ternary matrix -> wide device stream (u16 lists or gap stream), K-tiled for this device's
 * LDS.  sptmm_gemv_i8 and sptmm_gemv_f16 (and the batched call) serve it with 16-row (8-row) tiles:
 * meant for M > 8 (M > 4 with fp16 rows); correct for any M.  No counterpart in the reference. */
int sptmm_weights_upload_wide(const int8_t *W_colmajor, int K, int N, int kind, int split_k, sptmm_weights **out);
/* Second device copy of the same stream (used to rotate over more bytes than
 * the last-level cache holds when timing cold reads).  The copy is complete on
 * return: a launch on any stream may follow at once. */
int sptmm_weights_clone(const sptmm_weights *w, sptmm_weights **out);
void sptmm_weights_free(sptmm_weights *w);
/* Weight files, so that the host-side preparation (prepareW_map,
 * main.cu:242-509, repeated by every run of the reference) happens once: a
 * fixed header (shape, encoding, checksum) followed by the device stream as it
 * is.  load checks the header against the stream size, the checksum and, for
 * ragged and wide streams, the count tables (wide: every K-tile's offset, stride
 * and counts, and that its K-tile fits this device's LDS: SPTMM_ERR_UNSUPPORTED
 * otherwise), before anything reaches the device. */
int sptmm_weights_save(const sptmm_weights *w, const char *path);
int sptmm_weights_load(const char *path, sptmm_weights **out);
int sptmm_weights_info(const sptmm_weights *w, sptmm_winfo *out);
size_t sptmm_weights_bytes(const sptmm_weights *w);

/* Launch plans.  The shape of a launch (wavefronts per workgroup, workgroups per compute unit, tasks per wavefront, ...)
 * comes from a model inside the library; a stream may carry its own choice per kind of call -- by activation rows
 * (1, 2-4, 5-8, more) and by lone or batched launch, whatever the activation type: tune with the type the stream will
 * meet -- which then replaces the model's for that stream.  Every field
 * 0 = the model's choice; a value the kernels cannot take is ignored, never an error, and no plan changes a result.
 * The reference fixes its launch shapes at compile time (grid and block per instantiation, main.cu:996-1455).
 *   sptmm_weights_tune: a bounded search on the device -- a few dozen candidate plans, each timed over launches that
 *   rotate over enough device copies of the stream to exceed the last-level cache (`batch` = 0 times lone launches, else launches of `batch`
 *   GEMVs; act as in sptmm_gemv_batched, or 3 / 4 for lone sptmm_gemv_q8 calls on fp16 / bf16 rows; the rows are zeros) -- which stores the fastest as the stream's
 *   plan for that kind of call and reports microseconds per GEMV under the model's shape and under the plan kept (the
 *   model's shape is kept unless a candidate is at least 2 % faster, and still is when both are timed again one
 *   after the other).  Synchronous; allocates and frees its own buffers.
 * Plans travel with sptmm_weights_save / _load and are copied by sptmm_weights_clone. */
typedef struct sptmm_plan {
    int waves_per_wg;    /* wavefronts per workgroup */
    int wgs_per_cu;      /* workgroups per compute unit, lone list launches */
    int tasks_per_wave;  /* tasks per wavefront, batched list launches */
    int share_log;       /* lone GEMV of one int8 row on u16 lists: 1 << share_log wavefronts per task; -1: never shared */
    int i2s_ct;          /* i2s: column tiles per wavefront (1, 2, 4, 8) */
    int reserved[3];
} sptmm_plan;
int sptmm_weights_set_plan(sptmm_weights *w, int M, int batched, const sptmm_plan *plan);
int sptmm_weights_get_plan(const sptmm_weights *w, int M, int batched, sptmm_plan *out);
int sptmm_weights_tune(sptmm_weights *w, int M, int batch, int act, double *us_model, double *us_tuned);

/* C[M][N] = X[M][K] . W, X and C row-major device pointers (main.cu:575,592).
 * Asynchronous on `stream`.  The device that held the weights at upload must be
 * the current one (SPTMM_ERR_INVALID otherwise).
 *   sptmm_gemv_i8  int8 activations, exact int32 sums: rowWiseSplit3Small4
 *                  (main.cu:556-594), rowWiseSplit2DeltaSmallAsync2/3
 *                  (main.cu:599-764) or ladder_int8xint2_kernel
 *                  (bitnet_kernels.cuh:75-111), by the kind of `w`.
 *   sptmm_gemv_f16 fp16 activations (raw bits), fp32 sums; u16 and delta kinds.
 *   sptmm_gemv_f32 fp32 activations, fp32 sums; u16 and delta kinds.
 * Non-finite activations (fp16 / fp32): an Inf or NaN at X[m][k] reaches exactly
 * the outputs C[m][n] of the columns n whose lists hold row k, as the IEEE sums of
 * the gathered values give them (Inf, or NaN where +Inf meets -Inf).  Every other
 * row of the batch and every column that does not gather k is computed as if the
 * value were not there.  (A workgroup whose activation tile holds a non-finite
 * value sums on the vector unit instead of the matrix unit -- same result, several
 * times slower, so that one sequence's overflow never spoils another's.) */
int sptmm_gemv_i8(const sptmm_weights *w, const int8_t *X_dev, int M, int32_t *C_dev, void *stream);
int sptmm_gemv_f16(const sptmm_weights *w, const uint16_t *X_dev, int M, float *C_dev, void *stream);
int sptmm_gemv_f32(const sptmm_weights *w, const float *X_dev, int M, float *C_dev, void *stream);

/* The GEMV with its BitNet wrapper fused in: fp16 or bf16 activation rows are
 * quantised to int8 while the tile is staged (per row s = 127 / max(|x|, 1e-5),
 * q = clamp(rint(x*s), -127, 127), round-half-even), the sums run exactly as in
 * sptmm_gemv_i8, and the output is Y[m][n] = (float)C[m][n] * (1/s_m) * w_scale
 * in fp32 (evaluated in this order).  One launch where the unfused sequence takes
 * three (quantise, GEMV, rescale).  The reference has the GEMV only; it passes
 * an unused scale to its i2s kernel (main.cu:1862).  u16 and gap streams. */
typedef enum sptmm_xtype { SPTMM_X_F16 = 1, SPTMM_X_BF16 = 2 } sptmm_xtype;
int sptmm_gemv_q8(const sptmm_weights *w, const uint16_t *X_dev, int x_type, int M, float w_scale, float *Y_dev, void *stream);
/* The rescale alone, for callers whose activations are int8 already (quantised by the operator in front, which also
 * left the rows' 1/s_m -- a_m / 127 -- in device memory): the sums of sptmm_gemv_i8 written as
 * Y[m][n] = (float)C[m][n] * inv_scale[m] * w_scale, in this order, by the GEMV's own launch.  u16 and gap streams. */
int sptmm_gemv_i8_scaled(const sptmm_weights *w, const int8_t *Xq_dev, const float *inv_scale_dev, int M, float w_scale, float *Y_dev, void *stream);
/* sptmm_gemv_q8 with a workspace in device memory (sptmm_gemv_q8_workspace_bytes(w, M) bytes, 256-byte aligned, the
 * caller's, reusable from call to call on one stream).  With more than four rows, or more than 32 K activation values
 * in two to four rows, it runs as two launches -- the rows quantised once into the workspace (int8 rows, then their
 * 1/s), then the int8 GEMV scaling its sums on the way out -- where the fused launch quantises all rows again in every
 * workgroup (K=6912 N=2560, 8 rows: 19.0 us fused, 11.8 us this way; 16 rows: 35.4 and 13.4); otherwise it is the
 * fused launch and leaves the workspace alone.  Same arithmetic, same results bit for bit. */
size_t sptmm_gemv_q8_workspace_bytes(const sptmm_weights *w, int M);
int sptmm_gemv_q8_ws(const sptmm_weights *w, const uint16_t *X_dev, int x_type, int M, float w_scale, float *Y_dev, void *workspace_dev,
                     size_t workspace_bytes, void *stream);
/* sptmm_gemv_q8_ws without a workspace of the caller's and without any allocation, for callers that cannot allocate:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * The workspace is a static array in the library's device image (528,384 bytes on every GPU the library runs on, until
 * the process ends; its address is looked up per device in sptmm_device_init, or at the first call on a device):
 * calls whose workspace would be larger (sptmm_gemv_q8_workspace_bytes: M x K int8 values and M floats, each rounded
 * up to 256 bytes -- 38 rows at K = 13824 still fit) return SPTMM_ERR_UNSUPPORTED.  All calls on one GPU share the one array:
 * calls that overlap on a GPU (different streams, or threads) race on it -- serialise them, or use sptmm_gemv_q8_ws.
 * Nothing in it has to start at zero (every call rewrites the rows and scales it reads).  Same floats as
 * sptmm_gemv_q8_ws and sptmm_gemv_q8, bit for bit. */
int sptmm_gemv_q8_static(const sptmm_weights *w, const uint16_t *X_dev, int x_type, int M, float w_scale, float *Y_dev, void *stream);

/* `count` independent GEMVs of one shape in ONE launch: C[i] = X[i] . ws[i]
 * (int8 activations; streams of one kind that agree in K, N, S, split_k).  What a
 * decoder does with projections that share a shape; the reference launches its
 * kernels one at a time (main.cu:994-1459), so every launch there pays the
 * dispatch latency that this call pays once.  The pointer arrays are host
 * arrays of device pointers. */
int sptmm_gemv_i8_batched(const sptmm_weights *const *ws, const int8_t *const *X_dev, int32_t *const *C_dev, int count,
                          int M, void *stream);
/* The same for any activation type: act 0 int8 (int32 out), 1 fp16 or 2 fp32
 * (float out; u16 and gap streams only). */
int sptmm_gemv_batched(const sptmm_weights *const *ws, const void *const *X_dev, void *const *C_dev, int count, int M,
                       int act, void *stream);

/* Thin device-memory / stream / event helpers so callers need no HIP headers
 * (the cudaMalloc/cudaMemcpy/cudaEvent* calls of main.cu:767-782, 804-815). */
int sptmm_malloc(void **dev_ptr, size_t bytes);
int sptmm_free(void *dev_ptr);
int sptmm_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes);
int sptmm_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes);
int sptmm_memset(void *dst_dev, int value, size_t bytes); /* complete on return, like the two copies */
int sptmm_stream_create(void **stream);
int sptmm_stream_destroy(void *stream);
int sptmm_stream_sync(void *stream);
int sptmm_device_sync(void);
int sptmm_event_create(void **event);
int sptmm_event_destroy(void *event);
int sptmm_event_record(void *event, void *stream);
int sptmm_event_sync(void *event);
int sptmm_event_elapsed_us(void *start, void *stop, double *us);
/* Work issued on `stream` after this call waits for what `event` had recorded.  Between
 * sptmm_graph_begin and _end it is also how a second stream joins the capture and leaves it
 * again: record an event on the capturing stream and let the side stream wait for it (fork),
 * launch on both, record an event on the side stream and let the capturing stream wait for it
 * (join) -- independent projections then sit on parallel branches of the graph. */
int sptmm_stream_wait_event(void *stream, void *event);
/* Stream capture: the launches issued on `stream` between _begin and _end (any of
 * the sptmm_gemv_* calls, in any mix) become one executable HIP graph that
 * _launch replays -- a decoder layer's fixed sequence of projections as one
 * submission.  The reference issues its kernels one by one with a device
 * synchronize after each (main.cu:767-782).  Pointers and shapes are frozen at
 * capture; the contents of X may change between replays.  `stream` must come
 * from sptmm_stream_create; capture is thread-local, and a failed call between
 * _begin and _end still has to be followed by _end, which then reports the
 * failure.  The graph holds kernel launches only (no memset or copy nodes). */
int sptmm_graph_begin(void *stream);
int sptmm_graph_end(void *stream, void **graph);
int sptmm_graph_launch(void *graph, void *stream);
int sptmm_graph_destroy(void *graph);

/* The timing loop of measureKernel (main.cu:767-782) around `iters` GEMV
 * launches, kept native so that no interpreter sits between launches.  Launch i
 * uses ws[i % n_ws] (several device copies of one matrix defeat the last-level
 * cache).  act: 0 int8, 1 fp16, 2 fp32, 3 / 4 sptmm_gemv_q8 on fp16 / bf16 rows.  mode: 0 = back-to-back launches on one
 * stream between two events; 1 = stream synchronize after every launch, as the
 * reference does (main.cu:1456); 2 = one rotation captured into a HIP graph and
 * replayed; 3 = every rotation is ONE sptmm_gemv_i8_batched launch of all n_ws
 * GEMVs (C_dev must then hold n_ws * M * N outputs); 4 = one GEMV per launch as in mode 0, launch i on the i % 4-th of
 * four streams the call makes for itself (C_dev holds 4 * M * N outputs), timed from an event all four wait for to an
 * event that waits for all four.  `stream` must come from sptmm_stream_create; the call returns after
 * the stream has drained.  Reports mean microseconds per launch, taken from two
 * events recorded on that stream. */
int sptmm_measure_gemv(const sptmm_weights *const *ws, int n_ws, int act, const void *X_dev, int M, void *C_dev,
                       int iters, int mode, void *stream, double *us_per_call);
/* The same loop around a SEQUENCE of GEMVs -- a decoder layer's projections in their order
 * (the per-shape loops of main.cu:994-1459 time each projection on its own).  steps[i] is one
 * GEMV (act: 0 int8, 1 fp16, 2 fp32); `stage` is non-decreasing over the array, stages run in
 * order, and the steps of one stage do not depend on each other (q, k, v of one input).  One
 * pass over all n_steps is one sequence; it is issued `reps` times between two events on
 * `stream` (made by sptmm_stream_create), after one untimed pass.  mode:
 *   0  every step its own launch, in array order, on `stream`
 *   1  one pass captured into a HIP graph as a chain, replayed `reps` times
 *   2  captured with the steps of a stage on parallel branches of the graph (fork / join)
 *   3  no graph; the steps of a stage issued on side streams that fork from and join `stream`
 *   4  as 0, but neighbouring steps of one stage whose streams agree in kind and shape (and in M
 *      and act) go out as ONE batched launch (sptmm_gemv_batched)
 * Reports mean microseconds per sequence.  Weights of several layers in one array (stages
 * numbered through) keep the pass larger than the last-level cache. */
typedef struct sptmm_step {
    const sptmm_weights *w;
    const void *X_dev;
    void *C_dev;
    int M;
    int act;
    int stage;
} sptmm_step;
int sptmm_measure_sequence(const sptmm_step *steps, int n_steps, int reps, int mode, void *stream, double *us_per_sequence);
/* Reads `bytes` of a scratch buffer and writes them back (a plain copy kernel):
 * evicts cached weight streams between cold-read timings and calibrates the
 * traffic counters. */
int sptmm_copy_kernel(void *dst_dev, const void *src_dev, size_t bytes, void *stream);
/* Streams `bytes` of device memory through the GEMV kernels' own load
 * instruction and throws the data away (sink_dev: 4 bytes of device memory):
 * `launches` timed launches after one untimed, mean microseconds per launch.
 * Launch i reads the region at src_dev + (i % regions) * stride_bytes, so that
 * enough regions defeat the last-level cache.  What this reaches is the
 * practical ceiling below the 8 TB/s datasheet figure -- for one large read,
 * and for one launch per GEMV-sized read.  workgroups <= 0 picks 4 per compute
 * unit. */
int sptmm_read_kernel(const void *src_dev, size_t bytes, size_t stride_bytes, int regions, void *sink_dev, int workgroups,
                      int launches, void *stream, double *us_per_launch);

#ifdef __cplusplus
}
#endif
#endif /* SPTMM_H */
