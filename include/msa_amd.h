/*
 * msa_amd — C ABI of the MI355X (gfx950) routing / sparse-attention hot path of MSA.
 *
 * The reference (EverMind-AI/MSA) is pure Python: its "FFI" for this path is a set of torch
 * op sequences inside three Python call sites.  Each entry point below replaces one of those
 * sequences and cites it (paths relative to the reference checkout).  A Python maintainer binds
 * these with ctypes (see msa_amd/_lib.py) and passes `tensor.data_ptr()`.
 *
 * Conventions
 *   - every function returns 0 (MSA_OK) or a negative MSA_E* code and never throws;
 *     msa_last_error() gives the message of the calling thread's last failure;
 *   - pointers are DEVICE pointers unless the name ends in `_host`;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all work is
 *     enqueued on it and nothing synchronises unless stated;
 *   - only msa_bank_create allocates device memory (three index tables); every other entry point
 *     takes its scratch as `workspace`, sized by the matching *_workspace_bytes() function;
 *   - activations are token-major [T, H, D]; pooled tensors and the bank are chunk-major
 *     [C, Hkv, D]; document indices are 0-based in bank order; D must be 128;
 *   - dtype: MSA_BF16 (storage bf16, fp32 accumulation) or MSA_F32.
 */
#ifndef MSA_AMD_H
#define MSA_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSA_OK 0
#define MSA_EINVAL (-1)   /* bad argument (shape, null pointer, unsupported value) */
#define MSA_EHIP (-2)     /* a HIP runtime call failed */
#define MSA_ESIZE (-3)    /* workspace or output capacity too small */
#define MSA_ESTATE (-4)   /* bank layer not set / handle misuse */

#define MSA_BF16 0
#define MSA_F32 1

#define MSA_MODE_COSINE 0      /* q L2-normalised per head here, K_r expected normalised, scale 1 */
#define MSA_MODE_SCALED_DOT 1  /* raw dot product times `scale` (head_dim^-0.5 in the reference) */

/* reductions of msa_route_topk_reduce (the reference's query_reduce_method / chunk_reduce_method strings) */
#define MSA_QUERY_MAX 0    /* max over the scored tokens (src/msa_service.py:749-750): what msa_route_topk does */
#define MSA_QUERY_MEAN 1   /* sum over the scored tokens / their number, at least 1 (:751-767) */
#define MSA_QUERY_LAST 2   /* the token at position (number of scored tokens - 1) (:768-780) */
#define MSA_CHUNK_MAX 0    /* max over a document's chunks (:787-792): what msa_route_topk does */
#define MSA_CHUNK_MEAN 1   /* mean over a document's chunks (:794-811) */

const char* msa_last_error(void);
int msa_abi_version(void);

/* ---------------------------------------------------------------------------------------------
 * Chunk table of a packed block.  Replaces the nonzero / unique_consecutive / cumsum /
 * repeat_interleave chain of src/msa/memory_sparse_attention.py:138-163 and the per-document
 * ceil(len / P) of src/prefill.py:225.
 *   doc_start[n_docs+1]: token offset of each document in the packed block (doc_start[0] may be
 *   > 0: template tokens in front belong to no chunk).  Document d has ceil(len_d / P) chunks.
 * Outputs (capacity `chunk_cap` entries each, writes beyond it are suppressed):
 *   doc_chunk_off[n_docs+1], chunk_start[C] (first token), chunk_len[C] (1..P),
 *   chunk_doc[C] (0-based document), n_chunks_out[1] (int64, total C for the caller to verify). */
int msa_chunk_table(const int32_t* doc_start, int32_t n_docs, int32_t P, int64_t chunk_cap,
                    int32_t* doc_chunk_off, int32_t* chunk_start, int32_t* chunk_len,
                    int32_t* chunk_doc, int64_t* n_chunks_out, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Chunk-mean pooling of K, V and K_r.  Replaces sequence_pooling_kv
 * (src/msa/memory_sparse_attention.py:467-486), the inline K_r pooling (:178-190) and the
 * optional normalise (:192-194); with `rope_cos` it also fuses the rotary of :133 into the K read.
 *   k, v, kr: [T, H, D] token-major, any of them may be NULL (skipped with its output).
 *   Sums are direct fp32 segment sums; a partial last chunk is divided by its true length.
 *   rope_cos / rope_sin: fp32 [rope_rows, D/2] tables or NULL.  When given, K is rotated
 *   (half-split layout) at position (token - first token of its document) before pooling and
 *   `max_doc_len` must not exceed rope_rows.  `doc_start` is only read in that case.
 *   normalize_kr != 0: pooled K_r is divided by max(||.||_2, 1e-12) per (chunk, head). */
int msa_pool_chunks(const void* k, const void* v, const void* kr, int32_t dtype, int64_t T,
                    int32_t H, int32_t D, const int32_t* chunk_start, const int32_t* chunk_len,
                    const int32_t* chunk_doc, int64_t C, const int32_t* doc_start,
                    const float* rope_cos, const float* rope_sin, int32_t rope_rows,
                    int32_t max_doc_len, int32_t normalize_kr, void* k_out, void* v_out,
                    void* kr_out, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Memory bank.  Replaces Memory._init_block_data / BlockDesc / _generate_slice
 * (src/msa_service.py:191-231, 481-492, 644-695): K_r resident in HBM, pooled K / V in pinned
 * host memory, documents as contiguous chunk ranges.  The handle copies the two tables; the
 * per-layer tensors stay owned by the caller and must outlive the handle's use of them.
 *   doc_chunk_off_host[n_docs+1] (int32, first entry 0, last entry C), doc_global_id_host[n_docs]. */
typedef struct msa_bank msa_bank;
int msa_bank_create(msa_bank** out, int32_t n_layers, int64_t C, int32_t Hkv, int32_t D,
                    int32_t dtype, const int32_t* doc_chunk_off_host,
                    const int64_t* doc_global_id_host, int64_t n_docs);
/* kr_dev: device [C, Hkv, D]; k_host / v_host: pinned host [C, Hkv, D] (may be NULL for a
 * scoring-only bank). */
int msa_bank_set_layer(msa_bank* bank, int32_t layer, const void* kr_dev, const void* k_host,
                       const void* v_host);
int msa_bank_destroy(msa_bank* bank);

/* ---------------------------------------------------------------------------------------------
 * Router scoring + top-k.  Replaces MSAService._gather_querys' scaling / regrouping
 * (src/msa_service.py:1095-1100) and Memory.prefill_stage2 (:703-828): matmul, pad-token mask,
 * mean over the Hq heads, max over query tokens, max over a document's chunks, top-k.
 *   q: [B, S, Hq, D] (token-major, NOT pre-scaled), qmask_u8: [B, S] (1 = scored token) or NULL.
 *   msa_chunk_scores writes chunk_scores[B, C] fp32 (-inf where a query has no scored token).
 *   msa_route_topk writes scores_out[B, topk] (descending; ties by lower document index),
 *   doc_out[B, topk] (0-based, -1 past the number of documents) and doc_global_out[B, topk]
 *   (doc_global_id[doc], -1 likewise).  topk <= 64.  The max over a document's chunks (:789-792,
 *   :817-820) is taken in the scoring kernel's epilogue, so routing never writes a per-chunk plane.
 *   msa_route_workspace_bytes covers both calls (it holds the [B, C] plane of msa_chunk_scores);
 *   msa_route_topk alone needs only msa_route_topk_workspace_bytes. */
size_t msa_route_workspace_bytes(int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D,
                                 int64_t C, int64_t n_docs, int32_t topk);
size_t msa_route_topk_workspace_bytes(int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D,
                                      int64_t n_docs, int32_t topk);
int msa_chunk_scores(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8,
                     int32_t B, int32_t S, int32_t Hq, int32_t mode, float scale,
                     float* chunk_scores, void* workspace, size_t workspace_bytes, void* stream);
int msa_route_topk(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8,
                   int32_t B, int32_t S, int32_t Hq, int32_t mode, float scale, int32_t topk,
                   float* scores_out, int32_t* doc_out, int64_t* doc_global_out, void* workspace,
                   size_t workspace_bytes, void* stream);

/* msa_route_topk for callers that cannot allocate or carry a workspace: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and results as
 * msa_route_topk (bit for bit: it runs the same kernels), but the scratch is a device array built into the library,
 * MSA_ROUTE_STATIC_SCRATCH_BYTES per device for the life of the process, and the call allocates nothing.  Sizes
 * whose scratch need (msa_route_topk_workspace_bytes) exceeds that are refused with MSA_ESIZE; 16 queries of 128
 * tokens over 87,000 documents need about 10 MiB.  The array's device address is looked up on the first call on
 * each device (make that call outside graph capture).  All calls on one device share the array: calls that overlap
 * in time on one device (different streams or threads) race and must be serialised by the caller. */
#define MSA_ROUTE_STATIC_SCRATCH_BYTES (16 << 20)
int msa_route_topk_static(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8,
                          int32_t B, int32_t S, int32_t Hq, int32_t mode, float scale, int32_t topk,
                          float* scores_out, int32_t* doc_out, int64_t* doc_global_out, void* stream);

/* msa_route_topk with the reference's other reductions over a query's tokens and over a document's chunks
 * (Memory.prefill_stage2, src/msa_service.py:749-811; the head reduction stays the mean).  query_reduce MEAN / LAST
 * collapse every query to one row before the scan (both are linear in the query row or pick one row), so the scan
 * reads the bank once for one row block per query.  A query without scored tokens gets -inf scores as in
 * msa_route_topk (LAST: also when the token at that position is not scored).  chunk_reduce MEAN scores every chunk
 * (the per-chunk plane of msa_chunk_scores), averages each document's chunks and selects from those means; it needs
 * the workspace of msa_route_workspace_bytes, the others that of msa_route_topk_workspace_bytes. */
int msa_route_topk_reduce(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                          int32_t S, int32_t Hq, int32_t mode, float scale, int32_t query_reduce, int32_t chunk_reduce,
                          int32_t topk, float* scores_out, int32_t* doc_out, int64_t* doc_global_out, void* workspace,
                          size_t workspace_bytes, void* stream);

/* Measurement hook (no counterpart in the reference): while enabled, every launch of the scoring
 * kernel inside msa_chunk_scores / msa_route_topk is bracketed by a HIP event pair on its own
 * stream, up to max_records launches (0 disables and frees the events).  msa_profile_collect waits
 * for the recorded launches, writes their durations in milliseconds to ms_host[0..*n_out) and
 * resets the record count.  Not thread-safe; meant for benchmarks. */
int msa_profile_enable(int32_t max_records);
int msa_profile_collect(float* ms_host, int32_t cap, int32_t* n_out);

/* Measurement aid (no counterpart in the reference): a register-only loop of v_mfma_f32_32x32x16_bf16, 8 wavefronts
 * per workgroup with a 4 x 2 grid of accumulators each (the scoring kernel's shape and occupancy), `iters`
 * iterations of 8 MFMAs per wavefront, enqueued on `stream`.  mode 0: zero operands; 1: operands of ones (every
 * sink[thread] then holds 128 * iters exactly); 2: operands whose signs and mantissas change every iteration, which is
 * what the shader clock under real data answers to.  sink: device float [workgroups * 512]; *flops_out (host, may be
 * null) receives the launch's floating-point operations.  The rate of mode 2 is the ceiling of this GPU's matrix
 * cores under load, below the published peak, which assumes the boost clock.
 * mode + 16 * extra adds other VALU work per iteration of 8 MFMAs, on registers of its own (sink is then not
 * defined): extra 1 / 2: 24 / 48 v_fma_f32; 3 / 4: 24 / 48 v_exp_f32; 5: 24 v_cvt_pk_bf16_f32; 6: 24 v_dot2c_f32_bf16;
 * 7: 24 v_max3_f32.  The rates tell what each instruction costs on the SIMD's issue port next to the products
 * (the budget of a kernel that does softmax arithmetic between them). */
int msa_diag_mfma_loop(int32_t workgroups, int32_t iters, int32_t mode, float* sink, double* flops_out, void* stream);

/* Measurement aid (no counterpart in the reference): loops that only read `bytes` of device memory at `src`, taken
 * as rows of 2 KB (8 heads x 128 bf16), in the access patterns of the library's HBM-bound kernels, enqueued on
 * `stream`; bytes is a multiple of 128 KB.  mode 0: 64 consecutive rows per workgroup, non-temporal 16-byte loads (the
 * pooling kernel's reads); dst (device, >= 16 bytes) is not written.  mode 1: the same plus pooling's writes, one
 * 2 KB row of dst per 128 KB read: 16-byte word t (t < 128) of dst row w is the xor of the words at byte
 * 4096 * i + 16 * t of workgroup w's 128 KB for i = 0 .. 31; dst holds bytes / 64.  mode 2: each
 * workgroup reads one head's 256-byte piece of every row of a range of rows (the decode attention's reads of a
 * [rows, 8, 128] cache); dst (>= 16 bytes) is not written.  bytes / time is the rate a kernel with that pattern can
 * be held to on this GPU, below the published HBM peak. */
int msa_diag_read_stream(const void* src, int64_t bytes, void* dst, int32_t mode, void* stream);

/* Test aid (no counterpart in the reference; runs on the host, no GPU needed): replays the tile order of the
 * persistent large-tile scan (more than 128 query rows) for a launch of `grid` workgroups over tiles_m x tiles_n
 * tiles of 256 x 256, with or without the workgroup that copies K / V rows instead of scoring, the last pool_n N
 * tiles handed out from the shared pool.  visits (host, [tiles_m * tiles_n], M-major) receives how often each tile is
 * scored: all ones for a correct order.  Fails if the kernel's incremental tile cursor and the closed form of the
 * order disagree anywhere. */
int msa_diag_scan_walk(int32_t tiles_m, int32_t tiles_n, int32_t grid, int32_t has_copy_workgroup, int32_t pool_n,
                       int32_t* visits);

/* Registers and bytes of scratch per lane of the loaded code object's asm-scheduled kernels (which = 0: the routing
 * scan score_scan4_kernel, 1: flash_wide_kernel).  Their statements keep state in physical registers across statements,
 * which only holds while the compiler spilled nothing: the library refuses to launch either with scratch (MSA_ESTATE),
 * and this call lets a test see the numbers.  A diagnostic: no counterpart in the reference. */
int msa_diag_asm_kernel_resources(int32_t which, int32_t* num_regs, int32_t* scratch_bytes);

/* Switch (no counterpart in the reference): the large-tile scan hands the last eighth of its tiles out dynamically,
 * from a counter in the workspace, to even out the ends of the eight XCDs.  enabled = 0 gives every tile a fixed
 * workgroup (a few percent slower on large banks; no atomics on the hand-out path); 1 is the default.  Process-wide,
 * takes effect at the next call. */
int msa_route_set_tile_pool(int32_t enabled);

/* Test aid (no counterpart in the reference): `workgroups` workgroups that each claim a compute unit's whole LDS
 * (160 KB) and fill it with `word`; check (device, [workgroups], may be null) receives one word read back per
 * workgroup.  LDS is not cleared between kernels, so a launch of a few workgroups per compute unit leaves every unit's
 * LDS holding `word` (a NaN pattern, say) for the next kernel to find: the tests use it to show that kernels whose
 * tiles end in rows they did not load (ragged tails) never let stale LDS contents reach their results. */
int msa_diag_fill_lds(uint32_t word, uint32_t* check, int32_t workgroups, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Gather of the selected documents' pooled K / V from pinned host memory.  Replaces the
 * index_select fetch and per-sample regroup of MSAService.doc_query
 * (src/msa_service.py:1203-1262, 1289-1312).
 *   doc_sel_host[B, k]: 0-based documents (-1 = none).  Per sample, documents are laid out in
 *   ascending bank order, each once.  msa_gather_plan fills cu_sel_host[B+1] (prefix sums of
 *   selected chunk counts).  msa_gather_kv enqueues one hipMemcpyAsync per contiguous document
 *   run and tensor on `copy_stream` into k_out / v_out [cu_sel[B], Hkv, D]; the caller orders
 *   consumers after the stream (event or synchronise).  A document selected by several samples is
 *   read from the host once (the batch-wide unique() of :1214); the other samples' rows are
 *   device-to-device copies of the first on the same stream. */
int msa_gather_plan(const msa_bank* bank, const int32_t* doc_sel_host, int32_t B, int32_t k,
                    int64_t* cu_sel_host);
int msa_gather_kv(const msa_bank* bank, int32_t layer, const int32_t* doc_sel_host, int32_t B,
                  int32_t k, void* k_out, void* v_out, int64_t out_capacity_chunks,
                  void* copy_stream);

/* Device-side variant of the same gather: the selection stays on the device (doc_sel[B, k] int32, e.g. msa_route_topk's
 * doc_out; -1 or out-of-range entries are skipped), a planning kernel sorts / de-duplicates it per sample and writes
 * cu_sel[B+1] (device int32), and a copy kernel reads the rows straight from the pinned host bank.  Nothing
 * synchronises and nothing is copied to the host; rows past out_capacity_chunks are dropped and cu_sel stops at that
 * capacity, so size the outputs for B * k * (largest document's chunks).  While B * k <= 2048 a document selected by
 * several samples is read from the host once and copied on the device for the others.  k <= 64. */
size_t msa_gather_device_workspace_bytes(int32_t B, int32_t k);
int msa_gather_kv_device(const msa_bank* bank, int32_t layer, const int32_t* doc_sel, int32_t B,
                         int32_t k, void* k_out, void* v_out, int64_t out_capacity_chunks,
                         int32_t* cu_sel, void* workspace, size_t workspace_bytes, void* stream);

/* msa_route_topk of one layer with the msa_gather_kv_device of an earlier selection inside the same launch (typically
 * the previous router layer's documents: the reference fetches a layer's K / V right after routing it,
 * src/msa_service.py:1203-1262; a pipelined caller can let that fetch ride under the next layer's scan).  One
 * workgroup of the scan copies the rows from the pinned host bank while the others score, so the copy takes a compute
 * unit of its own instead of slowing scoring workgroups that a separate copy kernel's wavefronts would sit beside.
 * Arguments and results are those of the two calls (gather_* name the gathered layer and its selection [gather_B,
 * gather_k]; gather_workspace is msa_gather_device_workspace_bytes(gather_B, gather_k)).  The large-tile form of the
 * scan (bf16, more than 128 padded query rows) carries the copy; for other shapes the gather's own kernels run on the
 * stream in front of the scan, with the same results. */
int msa_route_topk_gather(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B, int32_t S,
                          int32_t Hq, int32_t mode, float scale, int32_t topk, float* scores_out, int32_t* doc_out,
                          int64_t* doc_global_out, void* workspace, size_t workspace_bytes, int32_t gather_layer,
                          const int32_t* gather_doc_sel, int32_t gather_B, int32_t gather_k, void* k_out, void* v_out,
                          int64_t out_capacity_chunks, int32_t* cu_sel, void* gather_workspace,
                          size_t gather_workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Context assembly.  Replaces the ragged scatter of src/msa/memory_sparse_attention.py:282-329
 * and the compact cache of :344-351: for every sample b writes
 *   [ prefix (n_prefix rows) | mem rows cu_sel[b]..cu_sel[b+1] | local rows cu_local[b]..cu_local[b+1] ]
 * into kcache / vcache [B, Lcap, Hkv, D] starting at row 0 of the sample, and kv_len[b].
 * Rows are [Hkv, D]; cu_sel / cu_local are device int32 [B+1]. */
int msa_assemble_context(const void* prefix_k, const void* prefix_v, int32_t n_prefix,
                         const void* mem_k, const void* mem_v, const int32_t* cu_sel,
                         const void* local_k, const void* local_v, const int32_t* cu_local,
                         int32_t B, int32_t Hkv, int32_t D, int32_t dtype, void* kcache,
                         void* vcache, int32_t Lcap, int32_t* kv_len, void* stream);

/* Appends one new K / V row per sample at kv_len[b] and increments kv_len[b]
 * (the torch.cat of src/msa/memory_sparse_attention.py:372-373, done in place). */
int msa_cache_append(const void* k_new, const void* v_new, int32_t B, int32_t Hkv, int32_t D,
                     int32_t dtype, void* kcache, void* vcache, int32_t Lcap, int32_t* kv_len,
                     void* stream);

/* Ragged form for a block of new tokens per sample (the source-context injection of the Memory-Interleave
 * loop, src/msa/generate.py:190-259, which reaches the same torch.cat at memory_sparse_attention.py:372-373 with
 * S > 1): sample b appends rows cu_new[b] .. cu_new[b+1] of k_new / v_new [total_new, Hkv, D] (device int32
 * prefix sums, at most max_new rows per sample) at kv_len[b]; rows that do not fit in Lcap are dropped. */
int msa_cache_append_rows(const void* k_new, const void* v_new, const int32_t* cu_new, int32_t max_new,
                          int32_t B, int32_t Hkv, int32_t D, int32_t dtype, void* kcache, void* vcache,
                          int32_t Lcap, int32_t* kv_len, void* stream);

/* ---------------------------------------------------------------------------------------------
 * GQA attention of ragged query rows over per-sample KV ranges.  Replaces repeat_kv + SDPA of the
 * decode step (src/msa/memory_sparse_attention.py:389-399) and, with several query rows per
 * sample, the causal varlen attention of stage 2 (:334-339).
 *   q: [sum Sq, Hq, D] with cu_q[B+1] (NULL = one row per sample); k / v: rows [Hkv, D];
 *   sample b's keys are rows kv_off[b] .. kv_off[b] + kv_len[b].  causal != 0: query row i of a
 *   sample with Sq rows sees the first kv_len - Sq + i + 1 keys (bottom-right aligned).
 *   out: [sum Sq, Hq, D].  max_sq / max_kv bound the per-sample sizes (grid sizing only).
 *   q, k, v and out must be 16-byte aligned (MSA_EINVAL otherwise): rows move in 16-byte pieces. */
size_t msa_attn_workspace_bytes(int32_t total_q, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_kv);
int msa_sparse_attn(const void* q, const int32_t* cu_q, const void* k, const void* v,
                    const int64_t* kv_off, const int32_t* kv_len, int32_t B, int32_t total_q,
                    int32_t max_sq, int32_t max_kv, int32_t Hq, int32_t Hkv, int32_t D,
                    int32_t dtype, float scale, int32_t causal, void* out, void* workspace,
                    size_t workspace_bytes, void* stream);

/* Same contract as msa_sparse_attn for bf16, built for blocks of query rows (stage-1 document-wise attention,
 * src/msa/memory_sparse_attention.py:216-241, and the stage-2 query prefill, :334-339): an MFMA flash kernel, one
 * pass over the keys, no workspace.  Use msa_sparse_attn for decode (one row per sample) and for fp32. */
int msa_flash_attn(const void* q, const int32_t* cu_q, const void* k, const void* v,
                   const int64_t* kv_off, const int32_t* kv_len, int32_t B, int32_t total_q,
                   int32_t Hq, int32_t Hkv, int32_t D, float scale, int32_t causal, void* out,
                   void* stream);
/* The same with the longest query block of the batch named (the lengths themselves are on the device): a batch of
 * ragged samples (max_sq * B > 1.25 total_q) keeps to the 32-column form of the kernel, see below. */
int msa_flash_attn_hint(const void* q, const int32_t* cu_q, const void* k, const void* v,
                        const int64_t* kv_off, const int32_t* kv_len, int32_t B, int32_t total_q,
                        int32_t Hq, int32_t Hkv, int32_t D, float scale, int32_t causal, void* out,
                        int32_t max_sq, void* stream);
/* msa_flash_attn has two forms of its kernel: 32 (token, head) columns per wavefront, two workgroups per compute unit,
 * and a wide one (64 columns per wavefront, one wavefront per SIMD, the tile step written at the instruction level)
 * that it picks when the call has at least 4096 columns.  form 0: by size (the default), 1: always the first,
 * 2: always the wide one.  A test and measurement aid (no counterpart in the reference); process-wide. */
int msa_flash_set_form(int32_t form);

/* ---------------------------------------------------------------------------------------------
 * Fused helpers around the attention call.  msa_qk_norm_rope replaces q_norm / k_norm + apply_rotary_pos_emb
 * (src/msa/memory_sparse_attention.py:129-133; transformers Qwen3RMSNorm, rotate_half): per head RMSNorm over the
 * 128 dims in fp32 times the norm weight, then half-split rotary at positions[n] from fp32 tables
 * [rope_rows, D/2] (positions are clamped to the table).  q / k / v are rows of a (possibly fused) projection
 * output with the given row strides in elements; outputs are dense [N, H, D].  v may be NULL (no copy).
 * msa_rmsnorm: out = rmsnorm(x) * weight over rows of H elements; with `residual` it first does
 * residual += x in place and normalises the sum (the residual add + norm of a decoder layer).
 * msa_silu_mul: out[n, i] = silu(gate_up[n, i]) * gate_up[n, I + i] for a fused gate/up projection. */
int msa_qk_norm_rope(const void* q, const void* k, const void* v, int64_t q_row_stride,
                     int64_t k_row_stride, int64_t v_row_stride, const int64_t* positions,
                     const void* q_norm_w, const void* k_norm_w, float eps, const float* rope_cos,
                     const float* rope_sin, int32_t rope_rows, int32_t dtype, int64_t N, int32_t Hq,
                     int32_t Hkv, int32_t D, void* q_out, void* k_out, void* v_out, void* stream);
/* Fused projection of a block of tokens (the encode path of stage 1 and the query prefill of stage 2): one bf16 GEMM
 * x[T, K] . w[N, K]^T over the concatenated weights of q_proj / k_proj / v_proj and, on router layers, router_k_proj
 * or router_q_proj (src/msa/memory_sparse_attention.py:125-127, 178, 263), with q_norm / k_norm and
 * apply_rotary_pos_emb (:129-133) applied to the q and k heads in the GEMM's epilogue, exactly as msa_qk_norm_rope
 * would to the bf16 projection output.  Rows of w, 128 per head: Hr_front router heads | Hq q heads | Hkv k heads |
 * Hkv v heads | Hr_back router heads (so one [rk | q | k | v | rq] matrix serves stage 1 with Hr_front = Hkv, stage 2
 * with a pointer 1024 rows in and Hr_back = Hq, and the decode step's q | k | v slice).  K a multiple of 64.
 * Outputs are dense: q_out [T, Hq, 128], k_out / v_out [T, Hkv, 128], r_out [T, Hr_front + Hr_back, 128]
 * (router heads are stored as projected: no norm, no rotary).  All of x, w, the outputs and the norm weights are
 * bf16 (q_norm_w / k_norm_w: 128 values each, 16-byte aligned like x, w and the outputs); the rotary tables are fp32
 * [rope_rows, 64].  The element types cannot be checked through this interface: a caller with fp32 norm weights
 * converts them first (or uses msa_qk_norm_rope, which takes a dtype). */
int msa_qkv_proj(const void* x, int64_t T, int32_t K, const void* w, int32_t Hq, int32_t Hkv, int32_t Hr_front,
                 int32_t Hr_back, const int64_t* positions, const void* q_norm_w, const void* k_norm_w, float eps,
                 const float* rope_cos, const float* rope_sin, int32_t rope_rows, void* q_out, void* k_out,
                 void* v_out, void* r_out, void* stream);
/* msa_qk_norm_rope for a decode step (one new token per sample, N = B) fused with msa_cache_append: the
 * normalised, rotated k row and the v row of sample b are written to kcache / vcache [b][kv_len[b]] and
 * kv_len[b] is incremented (src/msa/memory_sparse_attention.py:129-133 followed by the cache update at
 * :372-379).  A full cache (kv_len[b] == Lcap) drops the row. */
int msa_qk_norm_rope_append(const void* q, const void* k, const void* v, int64_t q_row_stride,
                            int64_t k_row_stride, int64_t v_row_stride, const int64_t* positions,
                            const void* q_norm_w, const void* k_norm_w, float eps,
                            const float* rope_cos, const float* rope_sin, int32_t rope_rows,
                            int32_t dtype, int32_t B, int32_t Hq, int32_t Hkv, int32_t D, void* q_out,
                            void* kcache, void* vcache, int32_t Lcap, int32_t* kv_len, void* stream);
/* The decode step of src/msa/memory_sparse_attention.py:361-405 from the fused projection output to the attention
 * output in two launches: q / k RMSNorm + rotary (:129-133), the cache update (:372-379) and GQA attention over
 * [cache | new token] (:389-399) for one new token per sample.  qkv rows are [Hq q heads | Hkv k heads | Hkv v heads]
 * (bf16, row stride in elements); kcache / vcache are [B, Lcap, Hkv, D]; kv_len[b] rows are valid on entry and
 * kv_len[b] + 1 on return (a full cache drops the new row and the token attends to the cache only).  Groups of 4 or
 * 8 query heads per KV head.  Workspace: msa_attn_workspace_bytes(B, Hq, Hkv, D, Lcap).  Same results as
 * msa_qk_norm_rope_append followed by msa_sparse_attn up to the order of the fp32 sums. */
int msa_decode_attn_fused(const void* qkv, int64_t row_stride, const int64_t* positions, const void* q_norm_w,
                          const void* k_norm_w, float eps, const float* rope_cos, const float* rope_sin,
                          int32_t rope_rows, int32_t B, int32_t Hq, int32_t Hkv, int32_t D, void* kcache,
                          void* vcache, int32_t Lcap, int32_t* kv_len, float scale, void* out, void* workspace,
                          size_t workspace_bytes, void* stream);
int msa_rmsnorm(const void* x, void* residual, const void* weight, int32_t dtype, int64_t N,
                int32_t H, float eps, void* out, void* stream);
int msa_silu_mul(const void* gate_up, int32_t dtype, int64_t N, int32_t I, void* out, void* stream);

/* Greedy sampling of a decode step in place of `logits.argmax(-1)` and the token bookkeeping that follows it
 * in the generation loops (src/msa/generate.py:102-105, :190-259: next token = argmax of the last position, position
 * += 1, token appended to the output): tok[b] = index of the largest of logits[b, 0..V) (the smallest index among
 * equal values; a NaN with a clear sign bit ranks above +inf, as in torch.argmax); pos[b] += 1 if pos is given; if
 * out / col are given, out[b, col[b]] = tok[b] when 0 <= col[b] < max_new, then col[b] += 1.  `scratch` holds
 * B * 32 64-bit words.  Two launches, no host synchronisation, safe to capture in a HIP graph. */
#define MSA_GREEDY_SCRATCH_WORDS_PER_ROW 32
int msa_greedy_sample(const void* logits, int32_t dtype, int32_t B, int64_t V, void* scratch, int64_t* tok,
                      int64_t* pos, int64_t* out, int64_t out_stride, int64_t* col, int32_t max_new,
                      void* stream);

/* Linear layer for the few rows of a decode step: y[M, N] = x[M, K] . w[N, K]^T, bf16, M <= 16,
 * K a multiple of 128, w in torch.nn.Linear layout (the F.linear calls behind q/k/v/o_proj and the MLP at
 * src/msa/memory_sparse_attention.py:125-127, 405 when one token per sample is decoded).  The weight matrix is
 * streamed from HBM once.  epilogue 0: plain; 1: y = residual + bf16(x w^T) (residual [M, N]); 2: w holds
 * alternating 8-row groups of gate and up rows (rows 16 i .. 16 i + 7 are gate rows 8 i .. 8 i + 7, the next eight
 * the same up rows; N = 2 I, I a multiple of 8) and y[M, I] = silu(gate) * up, both products rounded
 * to bf16 first as the unfused sequence does.  With norm_w [K] the RMSNorm in front of the projection is folded
 * in: the operand is bf16(x * rsqrt(mean(x^2) + eps) * norm_w) (input_layernorm / post_attention_layernorm of
 * src/msa/model.py's decoder layer).  Partial sums are added in a fixed order: results are
 * reproducible run to run. */
#define MSA_EPI_PLAIN 0
#define MSA_EPI_RESIDUAL 1
#define MSA_EPI_SILU_MUL 2
int msa_skinny_linear(const void* x, const void* w, const void* residual, const void* norm_w, float eps,
                      int32_t epilogue, int32_t dtype, int32_t M, int32_t N, int32_t K, void* y,
                      void* stream);
/* The same call with a scratch buffer of msa_skinny_linear_workspace_bytes(M, N, K) bytes (0 when the shape has
 * no use for one): matrices with few rows and a long K (down_proj) are then cut into row blocks x K slices whose
 * fp32 partial sums meet in the workspace and are added in K order by a second launch, which cuts the activation
 * bytes every compute unit re-reads.  With a NULL or too small workspace it is msa_skinny_linear. */
size_t msa_skinny_linear_workspace_bytes(int32_t M, int32_t N, int32_t K);
int msa_skinny_linear_ws(const void* x, const void* w, const void* residual, const void* norm_w, float eps,
                         int32_t epilogue, int32_t dtype, int32_t M, int32_t N, int32_t K, void* y,
                         void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MSA_AMD_H */
