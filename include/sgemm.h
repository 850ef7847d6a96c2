/*
 * sgemm.h - C ABI of the MI355X (gfx950) FP8 skinny-GEMM library, libsgemm.so.
 *
 * Every entry point is enqueue-only: it validates its arguments on the host, launches
 * on the given HIP stream (a hipStream_t passed as void*; NULL is the default stream)
 * and returns without synchronising.  All data pointers are DEVICE pointers owned by
 * the caller.  Nothing here calls exit(); failures come back as SgReturnCode values.
 *
 * Formats: "fp8" is OCP E4M3 (one byte, 0x7f/0xff NaN, max 448) - the format gfx950
 * MFMA decodes - not the E4M3 FNUZ of gfx942.  "bf16" is the upper half of an IEEE
 * binary32, rounded to nearest even.  Weights B are N x K, K contiguous, row stride
 * b_stride bytes; activations A are M x K row-major; outputs D are M x N row-major.
 *
 * Differences from the reference launchers that a caller must know:
 *   - D is OVERWRITTEN (the reference accumulates with atomics into a pre-zeroed D);
 *   - D is bf16 (the reference writes fp16 or fp32);
 *   - split-K partial sums are reduced in fp32 in a fixed order, so results are
 *     bit-reproducible from run to run.  The order in which one output element's K
 *     products are summed is a property of the configuration that runs (which waves
 *     and workgroups share K, and at which K block each of them starts); two
 *     configurations may differ in the last bit of the fp32 sum before rounding.
 *
 * Reference citations are paths below the reference tree's projects/ directory.
 */
#ifndef SGEMM_H
#define SGEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Codes 0-6 are the reference's SkinnyGemmReturnCode verbatim
 * (skinny_gemm/skinny_gemm_caller.cu:9-17); codes >= 7 are additions. */
typedef enum SgReturnCode {
    SG_SUCCESS = 0,
    SG_M_ABOVE_WARPTILE_M = 1,             /* kept for numbering; never returned (unused in the reference too) */
    SG_N_NOT_EVEN = 2,
    SG_K_NOT_DIVISIBLE_BY_WARPTILE_K = 3,
    SG_TOO_MANY_WARPS = 4,
    SG_QSIZE_TOO_SMALL = 5,
    SG_INVALID_CONFIG = 6,
    SG_LAUNCH_FAILED = 7,                  /* the HIP runtime refused the launch */
    SG_BAD_ALIGNMENT = 8,                  /* pointer or stride not 16-byte aligned */
    SG_BAD_ARGUMENT = 9,                   /* null pointer, non-positive size, ... */
    SG_WORKSPACE_TOO_SMALL = 10,           /* split-K partials do not fit the workspace */
    SG_NO_DEVICE = 11                      /* no usable gfx950 device / HIP runtime error at set-up */
} SgReturnCode;

const char* sg_strerror(int code);

/* Library-owned split-K workspaces (fp32 partial fragments + one arrival counter per output tile), one per
 * device and stream: launches on one stream run in order and share a workspace, launches on different
 * streams may overlap and never share one.  A workspace is created, or grown, by the first launch on its
 * stream that needs it (split_k > 1, also when the library chooses the split itself); at most 512 MB of
 * partials per launch, beyond that SG_WORKSPACE_TOO_SMALL.  An outgrown buffer is kept until it is released
 * (below).  A launch recorded into a HIP graph keeps the workspace of the stream it was captured on: run no
 * other split-K work on that stream while the graph replays elsewhere.
 *   sg_init          sets up the current device and a 64 MB workspace for the default stream
 *   sg_init_stream   the same for `stream` with room for partial_bytes of partials, so that later launches
 *                    on it allocate nothing
 *   sg_workspace_bytes  device memory the workspaces of the current device hold */
int    sg_init(void);
int    sg_init_stream(void* stream, size_t partial_bytes);
size_t sg_workspace_bytes(void);

/* Giving the library-owned buffers back (split-K workspaces, buffers they have outgrown, the activation scratch of
 * sg_skinny_gemm_bf16act): sg_release_stream waits for `stream` and frees what the library holds for it on the
 * current device - call it before destroying a stream, whose handle the runtime may hand out again -;
 * sg_release_workspaces waits for the device and frees everything, after which sg_workspace_bytes() is 0.  Later
 * launches allocate afresh.  A HIP graph that recorded a launch keeps pointing at the workspace of its capture
 * stream: release only after such graphs are destroyed. */
int    sg_release_stream(void* stream);
int    sg_release_workspaces(void);

/* The fastpath on caller-owned memory: the reference launcher allocates nothing and keeps no state
 * (skinny_gemm/skinny_gemm_caller.cu:20-43; the caller owns even the one-word scale, skinny_gemm/test.cu:78-79), and
 * sg_skinny_gemm_auto_ws does the same - its split-K partials and arrival counters live in `workspace` and nowhere
 * else, nothing is allocated, and a launch that would need more than it is given returns SG_WORKSPACE_TOO_SMALL.
 *   sg_workspace_query  *bytes = what sg_skinny_gemm_auto_ws needs for the shape with the tuning table as it is now
 *                       (0 when the launch it would choose has no K split; then workspace may be NULL)
 *   sg_workspace_init   zeroes the counter region (the first 64 KB) of a workspace with a kernel in stream order:
 *                       once per buffer, before its first use; every launch that completes leaves it zero again
 * workspace: device memory, 256-byte aligned, [16384 arrival counters][fp32 partials]; one buffer serves launches of
 * different shapes in stream order (size it by the largest query); launches that overlap need a buffer each. */
int sg_workspace_query(int m, int n, int k, size_t* bytes);
int sg_workspace_init(void* workspace, size_t bytes, void* stream);
int sg_skinny_gemm_auto_ws(const uint8_t* A, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                           int m, int n, int k, int b_stride, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Dense FP8 skinny GEMM:  D[m,n] = bf16( scale[0] * sum_k A[m,k] * B[n,k] ).
 * Replaces  int skinny_gemm(const fp8*, const fp8*, half*, const float*, int m, int n,
 * int k, int b_stride, int split_k, int A_producers, int B_producers, int consumers,
 * int b_lanes, int qsize, int op_m, int ops, hipStream_t)
 * (skinny_gemm/skinny_gemm_caller.cu:20-43) - same parameter list, same validation
 * order and return codes (:55-75).  Meaning of the tunables in this library:
 *   op_m     8, 16 or 32: rows of A covered by one MFMA column block (8 and 16 use one
 *            16-wide block with unused rows masked, 32 uses two); m above op_m is
 *            covered by further row tiles, each re-streaming B, as in the reference
 *            (skinny_gemm/skinny_gemm_kernel.cu:44-46).
 *   ops      MFMA K-steps per pipeline stage: a stage is WARPTILE_K = (512/op_m)*ops
 *            bytes of K per weight row; k must be a multiple of it.
 *   b_lanes  16-row weight tiles that share one activation fragment (1..4).
 *   qsize    stages kept in flight per wave (register ring depth) / LDS ring slots.
 *   A_producers, B_producers, consumers
 *            wavefront roles of one workgroup, at most 16 in total.  With
 *            A_producers == 0 and B_producers == 0 every one of the `consumers` waves
 *            streams its own operands from global memory straight into MFMA registers
 *            (no LDS hop) and the waves of a workgroup split K among themselves; with
 *            producers > 0 the operands go through an LDS ring filled by the producer
 *            waves, as in the reference.
 *   split_k  K is also split across split_k workgroups; partials meet in the fp32
 *            workspace and the last workgroup to arrive reduces them in split order.
 *            Honoured with and without producers (with producers a persistent workgroup
 *            walks (tile, split) work items, as skinny_gemm/skinny_gemm_kernel.cu:44-64
 *            decodes them); split_k above k / WARPTILE_K is SG_INVALID_CONFIG.
 */
int sg_skinny_gemm(const uint8_t* A, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                   int m, int n, int k, int b_stride, int split_k,
                   int A_producers, int B_producers, int consumers,
                   int b_lanes, int qsize, int op_m, int ops, void* stream);

/* Replaces  int skinny_gemm_fastpath(const fp8* A, const fp8* B, half* D, const float*
 * scale_tensor, int m, int n, int k)  (skinny_gemm/skinny_gemm_caller.cu:343-405):
 * b_stride = k, default stream, tunables chosen by the library for the shape instead of
 * compiled-in #defines (skinny_gemm/core.cu:29-38).  Requires k % 16 == 0 and n even. */
int sg_skinny_gemm_fastpath(const uint8_t* A, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                            int m, int n, int k);

/* The fastpath with an explicit row stride and stream (what the torch binding passes,
 * skinny_gemm/skinny_gemm_binding.cu:36-60). */
int sg_skinny_gemm_auto(const uint8_t* A, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                        int m, int n, int k, int b_stride, void* stream);

/* The same GEMM with per-row and per-column scale factors in the epilogue:
 *     D[i][j] = bf16( ((sum_k A[i][k]*B[j][k]) * scale) * row_scales[i] * col_scales[j] )
 * with three separately rounded fp32 products in that order.  No counterpart in the reference (its
 * epilogue applies the one scalar, skinny_gemm/consumers/mfma_16x16x32_consumer.cu:111-118); this is
 * the step on either side of the GEMM in a decode layer: activations quantised per row with
 * sg_fp8_encode_rows (its `scales` output is row_scales), weights quantised per output channel.
 * scale_tensor, row_scales ([m] floats) and col_scales ([n] floats) may each be NULL (factor 1). */
int sg_skinny_gemm_rowcol(const uint8_t* A, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                          const float* row_scales, const float* col_scales, int m, int n, int k, int b_stride,
                          void* stream);

/* Library-native tuning record for sg_skinny_gemm_tuned - no counterpart in the reference,
 * whose tunables are compile-time #defines rewritten by its grid-search script
 * (grid.py:106-116); this is the run-time equivalent a tuning driver sweeps. */
typedef struct SgTuning {
    int engine;        /* 0 library's choice, 1 direct (global -> VGPR -> MFMA), 2 LDS ring (global -> LDS DMA -> MFMA),
                          4 mid-batch (32 < m: weights streamed once, both operands staged in LDS for 2x2 or 4x2 waves;
                          k a multiple of 128, or - for the tile and ring combinations the library itself chooses - any
                          multiple of 16 beyond 128, the last 128-byte stage then loaded from k - 128) */
    int split_k;       /* workgroups sharing one output tile along K */
    int waves;         /* wavefronts per workgroup, sharing the tile along K (1..16); mid-batch: 4 (2 along n x 2 along m),
                          8 (4 x 2) or 14 (7 x 2, row_tiles = 2: 224-row tiles), each owning row_tiles x m_blocks
                          fragments of the tile */
    int row_tiles;     /* 16-row weight tiles per wavefront (b_lanes); mid-batch: 2 or 4 */
    int m_blocks;      /* 16-row activation blocks per tile: 1 (m <= 16 per tile) or 2; mid-batch: 2, 4 or 8 per wavefront */
    int depth;         /* stages in flight per wavefront (register ring / LDS ring slots) */
    int k_chunks;      /* direct engine: 64-byte K chunks per stage (1, 2, 4, 8); LDS ring: fixed 256-byte stage (k a
                          multiple of 256; one workgroup per tile and wave_tiles = 1 also take any other k > 256: the last
                          stage is loaded from k - 256 and its new bytes used);
                          mid-batch: ring slots of the activations, 2 <= k_chunks < depth (anything else = depth) */
    int non_temporal;  /* LDS ring: stream weights with the non-temporal hint */
    int persistent_wgs_per_cu; /* LDS ring: 0 = one workgroup per tile; n > 0 = n persistent workgroups per CU */
    int wave_tiles;    /* LDS ring: 1 = every wavefront owns whole tiles over the full K range and the activations
                          stay resident in LDS; 2 = persistent K-split workgroups with resident activations
                          3 = the same with the activations in the wavefronts' registers (k = 256 * waves * 1, 2 or 4)
                          (all need persistent_wgs_per_cu >= 1, split_k = 1, m <= 16*m_blocks); + 4 = persistent
                          workgroups get one extra wavefront that streams nothing and does every reduction and store;
                          8 (alone, with row_tiles = 2, persistent_wgs_per_cu = 0) = 24-row tiles: the
                          second 16-row fragment carries 8 weight rows (6144 rows = 256 tiles instead of 384);
                          mid-batch: 0 = the last workgroup of a tile to arrive sums the tile's split_k partials, 1 = the
                          GEMM launch stores partials only and a second launch sums them, four 16 x 16 fragments per wave
                          over the whole device (same split order, same result bits); anything else is SG_INVALID_CONFIG */
} SgTuning;

int sg_skinny_gemm_tuned(const uint8_t* A, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                         int m, int n, int k, int b_stride, const SgTuning* tuning, void* stream);

/* sg_skinny_gemm_tuned for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  No counterpart in the reference.  Same arguments, same kernels,
 * same result bits; the split-K partials and arrival counters live in a fixed array inside the library's
 * device image (8 MB + 4096 counters per GPU, held until the process ends) instead of a workspace from
 * hipMalloc, and nothing is allocated or freed by the call.  A configuration whose partials need more
 * (tiles * split_k * fragment bytes > 8 MB, or more than 4096 output tiles with split_k > 1) is refused
 * with SG_WORKSPACE_TOO_SMALL; without a K split there is no limit.  With engine = 0 the library's own choice is made
 * to fit: a K split that does not fit the array is not taken (the result then differs from sg_skinny_gemm_tuned's in
 * summation order only).  The counters are cleared by a kernel with
 * the first call on a device; after that every launch that completes leaves them zero.  All calls on one GPU share the array:
 * calls that overlap on one GPU (two streams, unordered graph nodes) race, calls in stream order do not. */
int sg_skinny_gemm_tuned_noalloc(const uint8_t* A, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                                 int m, int n, int k, int b_stride, const SgTuning* tuning, void* stream);

/* The rowcol GEMM on bf16 activations: the per-row quantisation of sg_fp8_encode_rows happens inside the GEMM,
 * so a decode layer's "quantise activations, then project" is one launch instead of two.
 *     s[i]    = absmax(X[i,:]) / 448  (1 for an all-zero row);   A[i][k] = e4m3_rne_sat(fp32(X[i][k]) / s[i])
 *     D[i][j] = bf16( ((sum_k A[i][k]*B[j][k]) * scale) * s[i] * col_scales[j] )
 * - bit for bit what sg_fp8_encode_rows followed by sg_skinny_gemm_rowcol(row_scales = its scales) returns when
 * both run the same GEMM configuration.  No counterpart in the reference, whose A producer copies FP8 bytes
 * (skinny_gemm/producers/producers.cuh:5-25) and whose epilogue applies one scalar
 * (skinny_gemm/consumers/mfma_16x16x32_consumer.cu:111-118).  X is [m][k] bf16, 16-byte aligned; scale_tensor
 * and col_scales may be NULL (factor 1); row_scales_out, if not NULL, receives s[0..m).
 * The fused kernel applies where one activation tile covers m (m <= 32), k % 256 == 0 and the codes fit LDS beside
 * the weight rings of four waves: every workgroup quantises its own copy of the activations while its first weight
 * stages are in flight.  That repeats the quantisation in every workgroup, so the library uses it only where it
 * measured faster than the two launches - m <= 8 and at least three 16-row tiles per CU (8 x 28672 x 4096: 26.9
 * against 29.0 us) - and otherwise runs the two launches itself, with the codes in a per-stream scratch buffer it
 * keeps.  sg_skinny_gemm_bf16act_choice says which (*fused) and with which record.  sg_skinny_gemm_bf16act_tuned
 * always runs the fused kernel: with the given record (LDS ring, persistent_wgs_per_cu >= 1, wave_tiles 2 or 6,
 * row_tiles 1, depth 2; at most 8 streaming waves), or - engine 0 - the library's own for the shape;
 * SG_INVALID_CONFIG where the kernel does not apply. */
int sg_skinny_gemm_bf16act(const void* X_bf16, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                           const float* col_scales, float* row_scales_out, int m, int n, int k, int b_stride,
                           void* stream);
int sg_skinny_gemm_bf16act_tuned(const void* X_bf16, const uint8_t* B, void* D_bf16, const float* scale_tensor,
                                 const float* col_scales, float* row_scales_out, int m, int n, int k, int b_stride,
                                 const SgTuning* tuning, void* stream);
int sg_skinny_gemm_bf16act_choice(int m, int n, int k, SgTuning* out, int* fused);

/* The configuration sg_skinny_gemm_auto would use, in the eight integers of the reference's launcher
 * (skinny_gemm_caller.cu:55-75), for logging and for drivers written against those:
 * out[8] = {split_k, A_producers, B_producers, consumers, b_lanes, qsize, op_m, ops}.
 * The eight cannot say everything a launch here depends on (persistent workgroups, resident activations,
 * the epilogue wave, the mid-batch tiles): passed back through sg_skinny_gemm they select a kernel of the
 * same ring geometry, not necessarily the one sg_skinny_gemm_auto runs.  sg_skinny_gemm_choice below
 * returns the complete record, and sg_skinny_gemm_tuned replays exactly that. */
int sg_skinny_gemm_pick(int m, int n, int k, int out[8]);

/* The complete record sg_skinny_gemm_auto would launch for the shape: the tuning table's entry when
 * there is one (*from_table = 1), the built-in heuristics' otherwise (0).  from_table may be NULL. */
int sg_skinny_gemm_choice(int m, int n, int k, SgTuning* out, int* from_table);

/* Per-shape tuning table - the run-time form of what the reference's grid search produces: there the
 * best #define set found by grid.py (:84-145, search space :151-159) is pasted into core.cu and picked
 * by the 249-arm macro chain of skinny_gemm_caller.cu:86-334; here a tuning driver stores the best
 * SgTuning per (m, n, k) and sg_skinny_gemm_auto / _fastpath / _rowcol use it instead of the built-in
 * heuristics.  A record the kernels cannot run for the shape (no such instantiation, ring larger than
 * LDS, ...) is skipped at launch and the heuristics' choice runs.  The table is process-wide and may be
 * read and changed from any thread; a launch uses the table as it is when the launch is made.
 * The library ships the table its tuning driver found for the benchmark shapes on MI355X
 * (rocm_dev_amd/tuning/mi355x.tbl, looked for as ../tuning/mi355x.tbl from the directory of libsgemm.so) and merges
 * it into the table once, before the table is first read or changed - the counterpart of the reference committing
 * what its search found (skinny_gemm/core.cu:29-38).  The environment variable SGEMM_TUNING_TABLE names another file
 * to load instead; empty or "none" starts with an empty table.
 *   sg_tuning_set    stores a copy of *t for the shape (engine 1, 2 or 4); t == NULL removes the entry
 *   sg_tuning_get    SG_SUCCESS and *out, or SG_INVALID_CONFIG when the table has no entry
 *   sg_tuning_load   merges a file into the table; SG_BAD_ARGUMENT (table unchanged) if the file cannot be
 *                    read or any line is malformed.  Format: first line "sgemm-tuning 1", then one record
 *                    per line as thirteen integers "m n k engine split_k waves row_tiles m_blocks depth
 *                    k_chunks non_temporal persistent_wgs_per_cu wave_tiles"; '#' starts a comment
 *   sg_tuning_save   writes the whole table in that format */
int sg_tuning_set(int m, int n, int k, const SgTuning* t);
int sg_tuning_get(int m, int n, int k, SgTuning* out);
int sg_tuning_count(void);
int sg_tuning_clear(void);
int sg_tuning_load(const char* path);
int sg_tuning_save(const char* path);

/* Replaces  template<class out> void async_gemm(const fp8* A, const fp8* B, out* D, int m,
 * int n, int k)  (async_gemm_sparse/sparse_k.cu:45-69, async_gemm_blanes/sparse_k.cu,
 * async_gemm_16x16x64/src.cu:55-82): D = A * B^T without a scale, default stream, through
 * the LDS producer/consumer ring.  The reference prints and exits on a bad shape; these
 * return SG_K_NOT_DIVISIBLE_BY_WARPTILE_K / SG_BAD_ARGUMENT instead.  D is overwritten. */
int sg_async_gemm_f32(const uint8_t* A, const uint8_t* B, float* D, int m, int n, int k);
int sg_async_gemm_bf16(const uint8_t* A, const uint8_t* B, void* D_bf16, int m, int n, int k);

/* 2:4 structured-sparse FP8 skinny GEMM - no counterpart in the reference (its "sparse" kernels
 * run dense operands through the sparse instruction, skinny_gemm/consumers/
 * smfma_16x16x64_consumer.cu:86-92; 2:4-compressed WEIGHTS are new here).
 *   D[m,n] = bf16( scale[0] * sum_k A[m,k] * Bdense[n,k] ),  Bdense = decompress(B_vals, B_meta)
 * B_vals [n][k/2]: the two kept E4M3 codes of every group of four consecutive k, in k order.
 * B_meta [n][k/8]: one nibble per group - low two bits = position (0..3) of the first kept
 *                  code, high two bits = position of the second (first < second); the group
 *                  with the lower k sits in the low nibble of each byte.
 * k must be a multiple of 128 and at least 512 (a k that 512 does not divide costs one partly used stage), n even;
 * all pointers 16-byte aligned.  The weights are the
 * sparse operand of gfx950's v_smfmac_f32_16x16x64_fp8_fp8; HBM traffic is 0.625 bytes per
 * dense weight.  The _tuned form takes row_tiles, waves, depth, split_k and m_blocks from
 * the record (engine 0 = library's choice); wave_tiles = 1 with persistent_wgs_per_cu >= 1
 * selects the kernel that keeps the activation matrix resident in LDS and gives every wave
 * whole 16*row_tiles-row tiles (m <= 16, split_k = 1, row_tiles 1 or 2).  Where k is a multiple of 1024 (and
 * split_k <= k / 1024) the metadata is fetched by whole 128-byte lines, two K stages per row and request, as long as
 * the ring that takes (4 KB of LDS per wave and row tile more) fits; k_chunks = 1 in the record keeps the fetch by
 * 64-byte pieces per stage. */
int sg_sparse24_gemm(const uint8_t* A, const uint8_t* B_vals, const uint8_t* B_meta, void* D_bf16,
                     const float* scale_tensor, int m, int n, int k, void* stream);
int sg_sparse24_gemm_tuned(const uint8_t* A, const uint8_t* B_vals, const uint8_t* B_meta, void* D_bf16,
                           const float* scale_tensor, int m, int n, int k, const SgTuning* tuning, void* stream);

/* Producer of that format: prunes a dense E4M3 matrix B [n][k] (row stride b_stride) to 2:4 and
 * compresses it.  Per group of four consecutive k the two codes of largest magnitude are kept
 * (ties keep the lower position; an already-2:4 input is compressed unchanged, zeros padding with the
 * lowest free positions).  No counterpart in the reference.  k % 16 == 0; B 16-byte aligned with
 * b_stride % 16 == 0, B_vals 8-byte, B_meta 2-byte aligned. */
int sg_sparse24_compress(const uint8_t* B, uint8_t* B_vals, uint8_t* B_meta, int n, int k, int b_stride, void* stream);

/* Replaces  void tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m,
 * int n)  (tiled_sum_reduce/src.cu:52-73):  D[m,n] = sum_b (A[b,m,n] + B[b,m,n]), summed
 * in batch order per element.  Any m, n (the reference needs m % 8 == 0, n % 64 == 0). */
int sg_tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n, void* stream);

/* Replaces  void tiled_sum_reduce(const float* A, const float* B, float* D, int b, int m, int n)  of
 * tiled_sum_reduce_async/src.cu:179-200, the variant that stages the batches through a queue in LDS
 * (kernel :98-177, producers :13-48, consumers :50-96).  Same result bits as sg_tiled_sum_reduce; every
 * wave keeps its own queue of direct-to-LDS loads, two to four batches ahead, ordered by its load counter
 * instead of flag bytes.  Any b, m, n. */
int sg_tiled_sum_reduce_async(const float* A, const float* B, float* D, int b, int m, int n, void* stream);

/* Per-row FP8 codec - no counterpart in the reference; the local compute on either side
 * of an FP8 all-reduce exchange.
 *   encode: scales[r] = absmax(X[r,:]) / 448 (1 if the row is all zero; NaNs do not count towards the maximum),
 *           Q[r,c] = e4m3_rne_sat( X[r,c] / scales[r] )                  (bit exact)
 *           A NaN quotient (NaN input, or an infinite input in a row whose maximum is infinite) is 0x7f;
 *           a finite input in such a row is a zero of its sign.
 *   decode: Y[r,c] = bf16( dec(Q[r,c]) * scales[r] )
 *   reduce: Y[r,c] = bf16( sum_{i<nbuf} dec(Q_i[r,c]) * scales_i[r] ), fp32, buffer order;
 *           buffer i starts at Q + i*q_buf_stride bytes, scales at scales + i*rows.
 * cols must be a multiple of 16; X, Q, Y must be 16-byte aligned. */
int sg_fp8_encode_rows(const void* X_bf16, uint8_t* Q, float* scales, int rows, int cols, void* stream);
int sg_fp8_decode_rows(const uint8_t* Q, const float* scales, void* Y_bf16, int rows, int cols, void* stream);
int sg_fp8_reduce_rows(const uint8_t* Q, const float* scales, void* Y_bf16,
                       int nbuf, size_t q_buf_stride, int rows, int cols, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SGEMM_H */
