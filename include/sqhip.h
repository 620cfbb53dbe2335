/* sqhip: C ABI of the MI355X (gfx950) codebook-linear kernels.
 *
 * One shared library, libsqhip.so, replaces every GPU launch site of the reference's
 * codebook linear layer.  All pointers inside sq_matrix and all x / y / out / workspace
 * pointers are DEVICE pointers owned by the caller; nothing here allocates or frees
 * device memory and nothing synchronises the host: every call only enqueues kernels on
 * `stream` (a hipStream_t passed as void*; NULL = the default stream), so calls can be
 * recorded into a HIP graph.  Functions return SQ_OK or a negative SQ_E* code and keep a
 * message for sq_last_error() (thread local).
 *
 * Data layout is the packed file's own (reference shapequant/packed.py:1-42): per matrix
 * an int32 [R, W] little-endian bit stream of log2(K)-bit tags (W = ceil(C/d * bits / 32)),
 * an fp16 [G*K, d] table, an fp16 [R] row scale, optional uint8 [R] row_book (G > 1) and
 * uint8 [R] row_mask (M > 1).  Column orders are int32 [M, C] (regenerated from the seed by
 * the host, reference shapequant/masks.py:334-342).  Row r decodes as
 *     u[r, j*d + k] = f32(table[row_book[r]*K + tag[r, j]][k]) * f32(row_scale[r])
 *     w[r, perms[row_mask[r]][c]] = u[r, c]
 * and the layer computes Y[t, y_off + r] = sum_c X[t, c] * w[r, c] with fp32 accumulation.
 */
#ifndef SQHIP_H
#define SQHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { SQ_OK = 0, SQ_EINVAL = -1, SQ_EUNSUPPORTED = -2, SQ_EWORKSPACE = -3, SQ_ELAUNCH = -4 };
enum { SQ_F32 = 0, SQ_F16 = 1, SQ_BF16 = 2 };

/* One packed matrix resident in device memory (the tensors the reference keeps in
 * kernels/gemv.py:107-131 PackedLinear, same meaning, file layout unchanged). */
typedef struct sq_matrix {
    const int32_t*  tags;       /* [R, W]; may be NULL for a matrix that keeps only its slice stream (below): every entry
                                 * point then works from the stream (one resident copy, the reference's `compact`) */
    const uint16_t* table;      /* fp16 bits [G*K, d] */
    const uint16_t* row_scale;  /* fp16 bits [R] */
    const uint8_t*  row_book;   /* [R] or NULL when G == 1 */
    const uint8_t*  row_mask;   /* [R] or NULL when M == 1 */
    const int32_t*  perms;      /* [M, C] or NULL when M == 1 */
    const int32_t*  row_order;  /* optional [R]: row ids sorted by row_mask (stable); NULL = natural */
    int32_t R, C, d, bits, G, M, W;
    int32_t y_off;              /* first output column of this piece in the stacked Y */
    const void*     stream;     /* optional: device copy of the buffer sq_stream_build wrote for `tags`; NULL = none */
    int32_t stream_runs;        /* runs_out of sq_stream_build for that buffer (opaque: run count, longest run, column orders per run, flags) */
    int32_t stream_groups;      /* groups_out of sq_stream_build for that buffer */
} sq_matrix;

/* Library / device identification.  sq_version: ABI version (major*100 + minor). */
int sq_version(void);
const char* sq_last_error(void);

/* Dense weight rows [r0, r1) of one matrix into out[(r - r0) * ld_out + c], original column
 * order, out_dtype SQ_F32 (exact product), SQ_F16 or SQ_BF16 (one round-to-nearest-even).
 * Replaces cuda_dequant.dequant(rl, out, rows) (reference shapequant/kernels/cuda_dequant.py:79-103)
 * and batched_runs.dequant_tile (reference shapequant/kernels/batched_runs.py:935-961); unlike
 * those it also applies column orders, i.e. it is packed.decode_tensors (reference
 * shapequant/packed.py:259-270) on the device. */
int sq_dequant(const sq_matrix* m, void* out, int out_dtype, int64_t ld_out, int32_t r0, int32_t r1,
               void* stream);

/* Decode-time product for B = 1..SQ_SMALL_BMAX activation rows over n_mats stacked pieces that
 * share C: Y[b, y_off + r] for every piece, X [B, C] with row stride ldx, Y row stride ldy
 * (elements).  x_dtype / y_dtype: SQ_F16 or SQ_BF16 (y may also be SQ_F32).
 * Replaces proto_runs.gemv (reference shapequant/kernels/proto_runs.py:505-571), cuda_gemv.gemv
 * (cuda_gemv.py:148-172), PackedLinear.gemv (gemv.py:142-156) and RunsBatch.run
 * (batched_runs.py:745-771).  Pieces with M > 1 and pieces with a slice stream need a workspace (see
 * sq_workspace_bytes; the latter keep their partial sums in its header); from 11 activation
 * rows on, a stack that has column orders (and C % 64 == 0, 16-byte aligned x, ldx % 8 == 0) is decoded to
 * fp16 in the workspace and multiplied by the tile GEMM, which is faster than its decode-time kernel there. */
#define SQ_SMALL_BMAX 32
int sq_linear_small(const sq_matrix* mats, int32_t n_mats, const void* x, int x_dtype, int64_t ldx,
                    void* y, int y_dtype, int64_t ldy, int32_t B, void* workspace, size_t ws_bytes,
                    void* stream);

/* sq_linear_small without a workspace argument, for callers that cannot allocate device memory (code under HIP graph
 * capture that has not grown a workspace beforehand, tight serving loops, harnesses that forbid hipMalloc): same
 * arguments, same kernels and bit-identical results, with the workspace (header included) kept in a device array
 * of SQ_NOALLOC_SCRATCH_BYTES that the library itself holds on every GPU it runs on until the process ends.  It has no
 * counterpart in the reference (whose launchers grow torch buffers on demand).  Pieces and row counts whose workspace
 * (sq_workspace_bytes(mats, n_mats, B, 0)) exceeds the array are refused with SQ_EWORKSPACE; nothing is allocated or freed,
 * here or in anything it calls.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (two streams, two threads) race; calls on one stream are safe. */
#define SQ_NOALLOC_SCRATCH_BYTES (48u << 20)
int sq_linear_small_noalloc(const sq_matrix* mats, int32_t n_mats, const void* x, int x_dtype, int64_t ldx,
                            void* y, int y_dtype, int64_t ldy, int32_t B, void* stream);

/* Prefill product for T activation rows: dequantise-into-LDS tile GEMM on fp16 MFMA with fp32
 * accumulation, row scale applied to the accumulator.  Same argument meaning as sq_linear_small.
 * Replaces runs_gemm.gemm (reference shapequant/kernels/runs_gemm.py:471-514).  Pieces with
 * M > 1 are decoded with their column orders into workspace and multiplied from there.  Between
 * SQ_SMALL_BMAX + 1 and 224 rows (64 when the codebook does not fit LDS) pieces without column orders
 * run as passes of SQ_SMALL_BMAX rows through sq_linear_small's kernels, which is cheaper than decoding
 * the matrix first, and up to SQ_SMALL_BMAX rows the call is sq_linear_small; sq_workspace_bytes(which = 1)
 * accounts for whichever route T takes. */
int sq_linear_gemm(const sq_matrix* mats, int32_t n_mats, const void* x, int x_dtype, int64_t ldx,
                   void* y, int y_dtype, int64_t ldy, int32_t T, void* workspace, size_t ws_bytes,
                   void* stream);

/* Dense fp16/bf16 weight [R, C] (row stride ldw) times X: the GEMM half of the reference's
 * "dequant + GEMM" large-M route (reference shapequant/vllm_ext/core.py:396-406, where it is a
 * cuBLAS call).  w_dtype: SQ_F16 or SQ_BF16, independent of x_dtype (both are multiplied as fp16); y_dtype any of
 * the three, independent of both.  fp16 weights with fp16 activations (16-byte aligned, strides % 8 == 0,
 * C % 64 == 0) run on the 256 x 256 tile kernel from 33 activation rows on; other combinations on a 128 x 128 tile
 * kernel that converts while it loads. */
int sq_gemm_dense(const void* w, int w_dtype, int64_t ldw, int32_t R, int32_t C, const void* x, int x_dtype,
                  int64_t ldx, void* y, int y_dtype, int64_t ldy, int32_t T, void* stream);
/* The same product with a workspace (sq_gemm_dense_workspace_bytes(R, C, T) bytes, same rules as sq_workspace_bytes;
 * 0: none needed): the tiles of the last, partial round of the 256 x 256 kernel are then split along K over the idle
 * CUs (2048 x 18944 x 3584: 0.26 ms instead of 0.32 ms).  Results differ from sq_gemm_dense's only in the order of
 * fp32 additions inside those tiles. */
int sq_gemm_dense_ws(const void* w, int w_dtype, int64_t ldw, int32_t R, int32_t C, const void* x, int x_dtype,
                     int64_t ldx, void* y, int y_dtype, int64_t ldy, int32_t T, void* workspace, size_t ws_bytes,
                     void* stream);
size_t sq_gemm_dense_workspace_bytes(int32_t R, int32_t C, int32_t T);

/* Bytes of workspace sq_linear_small (which = 0) or sq_linear_gemm (which = 1) needs for these
 * pieces at `rows` activation rows (which = 2 / 3: the same for a workspace that serves these pieces only, see
 * below); the caller grows its buffer before any graph capture
 * (the reference grows its buffers the same way: batched_runs.py:628-640, runs_gemm.py:396-404).
 * A workspace must be 256-byte aligned.  One of at least SQ_WS_HEADER_BYTES begins with a header of that size,
 * which must be ZERO when the workspace is first handed to the library and which nobody else may write
 * afterwards: it holds the partial sums that the workgroups of the decode-time kernel for large codebooks
 * exchange, and in its last page the error word of that exchange.  A partial sum is its own arrival flag (a word
 * is zero until its sum has been written, each word is one atomic location, and the workgroup that adds a
 * word up puts zero back), so every call leaves the header zeroed again and no call ever clears it.
 * Everything else a call needs lies behind the header and may hold anything.  One workspace serves one stream
 * at a time.  A workspace smaller than SQ_WS_HEADER_BYTES has no header and is used from its first byte: it
 * serves pieces that keep no partial sums (which | 2 below asks for the size of such a private workspace;
 * pieces with a slice stream always need the header).
 *
 * When the exchange fails.  A workgroup waits for the partial sums of its rows a bounded number of polls
 * (2^18, about a third of a second; sq_stream_spin_limit changes it).  If it gives up, because the workgroups
 * it waits for were held up that long or because a launch was abandoned (a device reset), it writes NaN
 * for its rows and sets the error word; the missing sums may still arrive afterwards and stay in the header, so
 * from then on EVERY launch on that workspace writes NaN for all its rows (a dirty header never yields
 * finite numbers), and the next sq_linear_small* call on that device returns SQ_ELAUNCH without launching
 * anything (the workgroup also sets a word in pinned host memory, one 64-byte allocation per device made
 * by the first call that is given a workspace with a header, which calls read without synchronising).
 * sq_workspace_status(workspace, ws_bytes, stream) SYNCHRONISES the stream and returns SQ_ELAUNCH if the error
 * word of that workspace is set; sq_workspace_reset enqueues a kernel that zeroes the header and clears the
 * error (the caller makes sure no product is still running on the workspace: same stream, or synchronise
 * first); sq_noalloc_reset does the same for sq_linear_small_noalloc's built-in array. */
#define SQ_WS_HEADER_BYTES (32u << 20)
size_t sq_workspace_bytes(const sq_matrix* mats, int32_t n_mats, int32_t rows, int which);
int sq_workspace_status(const void* workspace, size_t ws_bytes, void* stream);
int sq_workspace_reset(void* workspace, size_t ws_bytes, void* stream);
int sq_noalloc_reset(void* stream);
/* Polls of a row's partial sums before a workgroup gives up (negative: the default, 2^18).  Process-wide; meant
 * for tests of the failure path (0: give up at once where a sum is missing, every kernel still ends normally). */
void sq_stream_spin_limit(int32_t polls);

/* Load-time regrouping of a matrix' tags for codebooks that do not fit LDS (d = 8, K = 8192..65,536, one
 * codebook; several: sq_stream_build_books below): the decode-time product (up to 4 activation rows, up to 8 of rows with at most 1024 chunks, any
 * B <= 32 with column orders) then gathers codewords from a 64 KB LDS slice instead of from L2.
 * HOST pointers: `tags_host` is the file's tag tensor in host memory, `row_mask_host` the file's row_mask
 * (NULL when the matrix has one column order), `out_host` receives sq_stream_bytes() bytes that the caller
 * copies to the device (16-byte aligned) and names in sq_matrix.stream, together with *runs_out and
 * *groups_out in sq_matrix.stream_runs / stream_groups (both opaque to the caller).  sq_stream_bytes returns 0 for
 * formats the stream does not cover.  `runs` asks for that many row runs; each run becomes
 * 2^(bits - 12) * ceil(C / 8 / 4064) workgroups of 1024 threads in the batch-1 launch, one per compute unit, so
 * pick it to give the pieces launched together about one workgroup per CU in total (0 = a good value for a matrix
 * launched alone on 256 CUs); rows with different column orders never share a run and no run is longer than 6144
 * rows, so the run count can exceed the request.  A matrix with column orders must be given to sq_linear_small with
 * the same row_mask and with perms on the device.  Once the stream is on the device the tags are optional: with
 * sq_matrix.tags == NULL sq_dequant, every row count of sq_linear_small and sq_linear_gemm work from the stream
 * alone (decode-time speed is kept, the other paths get slower; x must then be 16-byte aligned with ldx % 8 == 0).
 * This plays the part of the reference's load-time layouts (reference
 * shapequant/kernels/proto_runs.py:295-349 pack_lane_major / RunsLinear, batched_runs.py:213-373 tile_words),
 * with a layout chosen for LDS gathers.
 *
 * The same two calls serve the formats whose codebook lives in LDS (d = 4 with 8-, 10- or 12-bit tags, one column
 * order, rows of whole 128/160/96-bit units): for them the buffer is a tile-major copy of the tags (the units of
 * each 16-row tile stored unit by unit, as large as the tags rounded up to 16 rows) that lets the decode-time
 * kernel read with fully coalesced loads; `runs` is ignored, *runs_out = *groups_out = 0, and the caller passes
 * the device copy in sq_matrix.stream with stream_runs = stream_groups = 0.  It is optional like the slice
 * stream (the reference keeps such a copy too: shapequant/kernels/batched_runs.py tile_words); these formats
 * always need their tags. */
size_t sq_stream_bytes(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                       const uint8_t* row_mask_host, int32_t runs);
int sq_stream_build(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                    const uint8_t* row_mask_host, int32_t runs, void* out_host, size_t out_bytes,
                    int32_t* runs_out, int32_t* groups_out);

/* The same with the matrix' codebook at hand (`table_host`: fp16 [2^bits, d] in host memory; NULL = the two calls
 * above).  A workgroup of the decode-time kernel gathers from one slice of 4096 codewords, so its work is the number of
 * tags that point into its slice: tags that favour some codewords (a codebook whose first entries are its most used
 * ones, a few very common shapes) would leave most workgroups waiting for a few.  With the codebook the builder
 * relabels the codewords (most used first, each to the slice that carries the fewest tags so far), writes the
 * relabelled codebook into the buffer and the kernels read their slices from there, so every slice carries the same
 * share of the tags whatever their distribution; results are the same bits.  The buffer grows by the codebook and a
 * 2-byte back map per codeword (1.1 MiB at K = 65,536).  Formats the slice stream does not cover ignore `table_host`.
 * No counterpart in the reference, whose kernels gather from the whole codebook. */
size_t sq_stream_bytes_balanced(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                                const uint8_t* row_mask_host, int32_t runs, const void* table_host);
int sq_stream_build_balanced(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                             const uint8_t* row_mask_host, int32_t runs, const void* table_host, void* out_host,
                             size_t out_bytes, int32_t* runs_out, int32_t* groups_out);

/* The relabelling by itself, for callers that would rather keep ONE codebook: remap_out[k] (2^bits entries, host
 * memory) is the new label of the file's codeword k.  A caller that rewrites its tags through remap_out and moves row k
 * of its table to row remap_out[k] holds an equivalent packed matrix (every weight decodes to the same bits) whose
 * slices carry equal shares of the tags; the plain sq_stream_build of those tags then needs no codebook copy of its
 * own, and the relabelled table serves every other entry point too. */
int sq_codebook_balance(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                        uint16_t* remap_out);

/* The three calls above for a matrix with G codebooks (G a power of two, `row_book_host` [R] names each row's; the
 * file's row_book tensor, reference shapequant/packed.py:30-40).  The G codebooks lie behind each other in sq_matrix.table,
 * so a row's tags are labels of that one long codebook, book * 2^bits + tag, and the stream is cut into slices of 4096
 * of those labels: d = 8, more than 4096 and at most 64 * 4096 codewords over all codebooks (4 MiB).  A workgroup then
 * finds entries only in the rows of its slice's codebook, so the work is even when the codebooks have about the same
 * number of rows.  The buffer is handed to the library exactly like a single-codebook stream (sq_matrix.stream,
 * stream_runs, stream_groups, with G and row_book set as usual); each run becomes G * 2^bits / 4096 * ceil(C / 8 / 4064)
 * workgroups.  sq_codebook_balance_books writes remap_out[book * 2^bits + k] = the new label, within its codebook, of
 * the file's codeword k of that codebook (every codebook is balanced over its own slices; one of at most 4096 codewords
 * keeps its labels).  A stream with a relabelled codebook of its own (sq_stream_build_balanced) is for one codebook
 * only.  G == 1, and the d = 4 formats whose buffer is the tile-major copy of the tags (which does not depend on the
 * codebooks), forward to the calls above.  The reference groups its tiles by (codebook, column order) at load time
 * for the same purpose (shapequant/kernels/proto_runs.py:352-366 book_tiles). */
size_t sq_stream_bytes_books(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits, int32_t G,
                             const uint8_t* row_book_host, const uint8_t* row_mask_host, int32_t runs);
int sq_stream_build_books(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits, int32_t G,
                          const uint8_t* row_book_host, const uint8_t* row_mask_host, int32_t runs, void* out_host,
                          size_t out_bytes, int32_t* runs_out, int32_t* groups_out);
int sq_codebook_balance_books(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits, int32_t G,
                              const uint8_t* row_book_host, uint16_t* remap_out);

/* ---- The packed file's block-32 side formats (reference shapequant/packed.py:30-40): the 8-bit output head
 * `aux.lm_head` (q int8 [V, C], scale fp16 [V, C/32], w = q * scale of the row's 32-column block) and the 4-bit
 * embedding `aux.embed` (q uint8 [V, C/2] with column 2k in the low and 2k+1 in the high nibble of byte k, each
 * storing n + 8 for n in -8..7, scale fp16 [V, C/32]).  q, scale, x, y, out, ids, workspace: DEVICE pointers (q
 * and scale of sq_q4_embed may also be pinned host memory, which the GPU reads over the bus: the reference's
 * host = True embedding, shapequant/vllm_ext/core.py:605-616).  q 16-byte aligned, C a multiple of 32.
 *
 * sq_q8_linear: Y[b, v] = sum_c X[b, c] * w[v, c] for B activation rows, fp32 accumulation with the block scale
 * applied to each block's fp32 sum (the reference kernel's arithmetic, shapequant/kernels/batched_runs.py:376-440).
 * One or two rows (up to SQ_SMALL_BMAX when C % 256 != 0, 4 per pass) stream q through an exact-product kernel that
 * needs no workspace; otherwise 3 .. 320 rows run fp16 MFMA passes of up to 64 rows with the block scale
 * folded into the fp16 weight (one rounding) and need the workspace sq_q8_workspace_bytes names (an fp16 copy of
 * the activations).  It replaces gemv_q8_batched /
 * gemv_q8_tile (reference shapequant/kernels/batched_runs.py:826-861, called from vllm_ext/core.py:575-583) and
 * proto_formats.gemv_q8 (shapequant/kernels/proto_formats.py:474-482); it reads the file's natural layout, so
 * there is no counterpart of the reference's tile-major copy.  B > 320 (B > SQ_SMALL_BMAX when C % 256 != 0) decodes row chunks to fp16 in
 * the workspace (scale folded in, one rounding) and multiplies them with the tile GEMM, as the reference's chunked
 * route does (vllm_ext/core.py:584-591); sq_q8_workspace_bytes gives the size (0 for B <= 2), with the
 * same rules as sq_workspace_bytes.  x_dtype / y_dtype as in sq_linear_small. */
int sq_q8_linear(const int8_t* q, const uint16_t* scale, int32_t V, int32_t C, const void* x, int x_dtype, int64_t ldx,
                 void* y, int y_dtype, int64_t ldy, int32_t B, void* workspace, size_t ws_bytes, void* stream);
size_t sq_q8_workspace_bytes(int32_t V, int32_t C, int32_t B);

/* Dense rows [r0, r1) of the 8-bit matrix into out[(r - r0) * ld_out + c]: SQ_F32 is the exact product, SQ_F16 /
 * SQ_BF16 round it once.  Replaces Q8Head._rows (reference shapequant/vllm_ext/core.py:548-555) and
 * packed.q8_rows (shapequant/packed.py:155-158). */
int sq_q8_dequant(const int8_t* q, const uint16_t* scale, int32_t V, int32_t C, void* out, int out_dtype, int64_t ld_out,
                  int32_t r0, int32_t r1, void* stream);

/* Rows ids[0..n_ids) (int64) of the 4-bit embedding into out[i * ld_out + c], same rounding rule as above; an id
 * outside [0, V) gives a row of zeros.  Replaces q4_embed (reference shapequant/vllm_ext/core.py:594-602) and
 * packed.q4_embed_rows (shapequant/packed.py:148-152). */
int sq_q4_embed(const uint8_t* q, const uint16_t* scale, int32_t V, int32_t C, const int64_t* ids, int64_t n_ids, void* out,
                int out_dtype, int64_t ld_out, void* stream);

/* ---- The elementwise neighbours of the decode-time products ----
 *
 * sq_addnorm: residual add + RMS norm that writes the next product's input, for B activation rows:
 *     v[b, i]      = h_in[b * ld_h + i] + add[b * ld_add + i]            (fp32; add may be NULL)
 *     h_out[b, i]  = v[b, i]                                            (h_out may be NULL, or h_in when perms is NULL)
 *     act[b, i]    = round(v[b, i] * rsqrt(mean_i(v[b, i]^2) + eps) * w[i])   to out_dtype (SQ_F16 / SQ_BF16)
 *     out[(b * M + m) * C + i] = act[b, perms[m * C + i]]                (perms NULL: M = 1 and the identity)
 * It replaces addnorm_perm (reference shapequant/kernels/decode_e2e.py:84-108) and the EPI 1 epilogue of gemv_runs
 * (shapequant/kernels/proto_runs.py:223-268).  perms are a piece's column orders (sq_matrix.perms); the products of
 * this library read x through them themselves, so callers inside it pass NULL.  With perms C <= 32256.
 *
 * sq_silu_mul: out = silu(gate) * up, SiLU in fp32 rounded to `dtype`, the product rounded to `dtype` (the model
 * code's arithmetic), gate / up / out all of `dtype`, rows b at gate + b * ld and up + b * ld (gate | up of one
 * stacked product: up = gate + C, ld = 2 C), out[(b * M + m) * C + i] as above.  It replaces silu_mul_perm
 * (reference shapequant/kernels/decode_e2e.py:125-136) and the EPI 2 epilogue (proto_runs.py:269-276). */
int sq_addnorm(const float* h_in, float* h_out, int64_t ld_h, const void* add, int add_dtype, int64_t ld_add, const void* w,
               int w_dtype, const int32_t* perms, int32_t M, int32_t B, int32_t C, float eps, void* out, int out_dtype,
               void* stream);
int sq_silu_mul(const void* gate, const void* up, int dtype, int64_t ld, const int32_t* perms, int32_t M, int32_t B, int32_t C,
                void* out, void* stream);

/* sq_linear_small whose activations X [B, C] are produced by one of the two neighbours above instead of being read:
 * the same results, bit for bit, as sq_addnorm / sq_silu_mul (perms = NULL) into x_out followed by sq_linear_small
 * on x_out.  For one activation row of pieces that run on the tag-stream kernel (codebooks beyond LDS) and have no
 * column orders the add + norm producer is fused into that kernel: every workgroup computes its part of the row while
 * it stages it (the mean square of the whole row included, in the stand-alone kernel's summation order), so no launch
 * and no dependency bubble sit between the two; otherwise (with column orders every workgroup would gather the
 * producer's operands through each order of its run), and always for SiLU * up (whose exponentials every workgroup
 * would have to repeat for the whole row), both measured slower than the extra launch, the library launches the
 * stand-alone kernel first.  This is the
 * counterpart of the reference's epi argument (reference shapequant/kernels/proto_runs.py:505-571, EPI 1 / EPI 2 at
 * :223-287), turned round: there the producing kernel's last blocks write the next product's input, here the
 * consuming kernel's workgroups compute it, which needs no launch-wide ticket and no cross-die visibility.
 * mode SQ_FROM_ADDNORM: X = round(v * rsqrt(mean(v^2) + eps) * w), v = h_in + add (add NULL: v = h_in), h_out = v
 * if not NULL (h_out must not be h_in).  mode SQ_FROM_SILU_MUL: X = silu(add) * up.  add / up / w / x_out hold
 * x_dtype; rows b of h_in / h_out at b * ld_h, of add / up at b * ld_in, of x_out at b * C.  x_out is always
 * written (it must be 16-byte aligned and C % 8 == 0); x_out and h_out must not overlap h_in / add / up / w (the
 * reference lets its epilogue write into x's buffer because it runs after every block has read x; here workgroups
 * still read the operands while one of them writes). */
#define SQ_FROM_ADDNORM 1
#define SQ_FROM_SILU_MUL 2
typedef struct sq_producer {
    int32_t mode;
    float eps;
    const float* h_in;
    float* h_out;
    const void* add;
    const void* up;
    const void* w;
    void* x_out;
    int64_t ld_h, ld_in;
} sq_producer;
int sq_linear_small_from(const sq_matrix* mats, int32_t n_mats, const sq_producer* from, int x_dtype, void* y, int y_dtype,
                         int64_t ldy, int32_t B, void* workspace, size_t ws_bytes, void* stream);

/* The stacked gate | up product with SiLU * up on the way out: mats[0] = the gate piece, mats[1] = the up piece (same
 * R and C), out[b * ld_out + r] = silu(Y[b, r]) * Y[b, R + r] with Y the stacked product rounded to `dtype` (SQ_F16 /
 * SQ_BF16, also x's type): the same results, bit for bit, as sq_linear_small into a `dtype` y followed by sq_silu_mul
 * (gate = y, up = y + R, perms = NULL).  One launch: the workgroup that adds a row's partial sums up reads the gate
 * row's and the up row's and writes their product, so Y never goes to memory.  This is the reference's EPI 2 epilogue
 * (reference shapequant/kernels/proto_runs.py:223-237,269-287, the epi argument of gemv at :505-571) without its
 * launch-wide ticket: there the last blocks of the launch compute the whole next input once every block has written y,
 * here every row is finished where its sums meet.  `from` (NULL, or mode SQ_FROM_ADDNORM as in sq_linear_small_from,
 * one activation row; x and ldx are then ignored and from->x_out is the row the launch computes and reads) lets the
 * same launch produce its own input too.  For pieces on the tag-stream kernel without column orders whose streams are
 * cut into the same runs (sq_stream_build with the same `runs`), 1 to 8 activation rows; any other stack returns
 * SQ_EUNSUPPORTED and the caller makes the two calls.  Needs the workspace of sq_linear_small (its header). */
int sq_linear_small_silu(const sq_matrix* mats, int32_t n_mats, const sq_producer* from, const void* x, int dtype, int64_t ldx,
                         void* out, int64_t ld_out, int32_t B, void* workspace, size_t ws_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SQHIP_H */
