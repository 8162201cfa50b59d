/*
 * flagtree_smla.h -- C ABI of libflagtree_smla.so: sparse MLA forward for MI355X (gfx950).
 *
 * Plain pointers and sizes only.  Every pointer named "device" must be HIP device
 * memory of the current device; `stream` is a hipStream_t passed as void* (NULL =
 * the default stream).  All launches are asynchronous on `stream`.  q, kv, out, workspaces and
 * the GEMM operands must be 16-byte aligned, index lists and sequence lengths 4-byte aligned.  The library
 * never allocates or frees device memory and keeps no state between calls.
 * Functions return SMLA_OK (0) or a negative error code; they never abort.
 *
 * The reference ships this path as Triton/TLE kernels reached through a generated
 * per-kernel C launcher: launch(gridX, gridY, gridZ, stream, function, ..., *args)
 * with tensors passed by data_ptr()
 * (/root/reference/third_party/amd/backend/driver.py:385-434, pointer extraction
 * :344-383), and it loads closed backends as C-symbol plug-ins with dlopen/dlsym
 * (/root/reference/python/src/plugin.h:34-83).  The entry points below are what a
 * binding for the sparse-MLA operator would call instead of that launcher.
 */
#ifndef FLAGTREE_SMLA_H
#define FLAGTREE_SMLA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  SMLA_OK = 0,
  SMLA_EINVAL_NULLPTR = -1,   /* a required pointer is NULL */
  SMLA_EINVAL_SHAPE = -2,     /* a size is non-positive or unsupported (d_qk != 576, d_v != 512, ...) */
  SMLA_EINVAL_ALIGN = -3,     /* a pointer is not 16-byte aligned */
  SMLA_EINVAL_WORKSPACE = -4, /* workspace missing or too small for n_splits > 1 */
  SMLA_EINVAL_SPLITS = -5,    /* n_splits outside [1, SMLA_MAX_SPLITS] */
  SMLA_ENODEVICE = -6,        /* no gfx950 device / kernels not loadable */
  SMLA_EINVAL_SCALE = -7,     /* sm_scale is not a positive finite number, or logit_cap is negative / not finite */
  SMLA_EWORKSPACE_STATE = -8, /* smla_workspace_status: a launch flagged the workspace (see SMLA_WS_STATUS_*) */
  SMLA_EHIP_BASE = -100       /* HIP runtime error e is reported as SMLA_EHIP_BASE - e */
};

#define SMLA_D_QK 576          /* 512 NoPE + 64 RoPE */
#define SMLA_D_V 512
#define SMLA_FP8_RECORD_BYTES 656 /* 512 e4m3fn | 4 f32 block scales | 64 bf16 rope */
#define SMLA_MAX_SPLITS 32
#define SMLA_WS_COUNTER_BYTES 262144 /* head of the workspace: arrival words (zero between calls) + header */
/* The last 64 bytes of that head are the workspace header, four uint32 words written by
 * smla_workspace_init: [0] SMLA_WS_MAGIC, [1] status (SMLA_WS_STATUS_* bits, 0 = healthy),
 * [2] poll limit of the split merge's bounded wait, [3] reserved. */
#define SMLA_WS_HEADER_OFFSET (SMLA_WS_COUNTER_BYTES - 64)
#define SMLA_WS_MAGIC 0x414c4d53u          /* "SMLA" */
#define SMLA_WS_SPIN_LIMIT_DEFAULT 4000000u /* polls (each about a microsecond) before the split merge gives up */
#define SMLA_WS_STATUS_UNINITIALISED 1u    /* a launch found no magic word: smla_workspace_init was never run */
#define SMLA_WS_STATUS_STALE 2u            /* an arrival word was in an illegal state (overlapping launches?) */
#define SMLA_WS_STATUS_TIMEOUT 4u          /* the last split to arrive gave up waiting for the others */

/* KV row formats */
#define SMLA_KV_BF16 0         /* row = 576 bf16 (1152 B) */
#define SMLA_KV_FP8_B128 1     /* row = 656-byte record, one f32 scale per 128 NoPE values */
#define SMLA_KV_F32 2          /* row = 576 fp32 (2304 B); q/out fp32 as well (plumbing path) */

/* Human-readable text for a status code (static storage). */
const char* smla_strerror(int status);

/* ABI version (bumped when a signature changes). */
int smla_abi_version(void);

/*
 * Addressing shared by all forward entry points.
 *   n_tokens         number of query tokens T (= batch * tokens_per_seq)
 *   tokens_per_seq   token t belongs to sequence t / tokens_per_seq
 *   indices          device int32 [T, topk]; -1 (any negative) = padding; order is free
 *   block_table      device int32 [n_seqs, block_table_stride] physical page numbers, or NULL
 *   page_size        tokens per page (used only with block_table)
 *   kv_seq_stride    without block_table: physical row = seq * kv_seq_stride + index and
 *                    0 <= index < kv_seq_stride must hold; 0 = one shared pool
 *                    (row = index, 0 <= index < kv_rows)
 *   kv_rows          rows in the kv buffer; translated rows outside [0, kv_rows) are masked
 * Replaces the page lookup the reference's MLA decode kernels do in-kernel
 * (/root/reference/third_party/mthreads/python/test/wmma/test_accuracy_musa_vllm_mla.py:278-283).
 */

/*
 * Sparse MLA forward:  out[t,h,:] = sum_j softmax_j(sm_scale * <q[t,h,:], kv[I[t,j],:]>) * kv[I[t,j], :d_v]
 *                      lse[t,h]   = log sum_j exp(sm_scale * <q[t,h,:], kv[I[t,j],:]>)      (natural log)
 * over the valid entries of indices[t,:].  A token without valid entries gives out = 0, lse = -inf.
 *   kv_format   SMLA_KV_BF16: q bf16 [T,H,576], kv bf16 [kv_rows,576], out bf16 [T,H,512]
 *               SMLA_KV_FP8_B128: q bf16, kv [kv_rows,656] records, out bf16
 *               SMLA_KV_F32: q, kv, out fp32 (exact-fp32 scalar kernel; small shapes)
 *   lse         device f32 [T,H]
 *   n_splits    split the top-k list over this many workgroups per token (1 = no split);
 *               0 = choose (smla_plan_splits).  n_splits > 1 needs `workspace` of at least
 *               smla_workspace_bytes() bytes (device, 16-byte aligned) that went through
 *               smla_workspace_init() once; the split results are merged inside the same launch
 *               by the last workgroup to finish, which also leaves the workspace ready for the
 *               next call (or by a second launch on the same stream: smla_merge_in_launch).
 *               Calls that share a workspace must not overlap.
 *   sm_scale    positive and finite.
 * Stands where the reference's host wrapper launches its attention kernel
 * (/root/reference/python/triton/ops/flash_attention.py:387-408; MLA decode:
 * test_accuracy_musa_vllm_mla.py:340-423 stage 1 and :480-510 stage 2).
 */
int smla_fwd(int kv_format, const void* q, const void* kv, const int32_t* indices,
             const int32_t* block_table, void* out, float* lse,
             int32_t n_tokens, int32_t tokens_per_seq, int32_t n_heads, int32_t topk,
             int32_t d_qk, int32_t d_v, int32_t page_size, int32_t block_table_stride,
             int64_t kv_seq_stride, int64_t kv_rows, float sm_scale, int32_t n_splits,
             void* workspace, size_t workspace_bytes, void* stream);

/*
 * Dense MLA decode over the whole paged context (no index list): token t of sequence s attends to
 * logical positions 0 .. seq_lens[s]-1 (clipped to max_seq_len); everything else as smla_fwd,
 * same kernels, same split merge.  seq_lens device int32 [n_tokens / tokens_per_seq].
 * logit_cap > 0 squashes every scaled score s to logit_cap * tanh(s / logit_cap) before the
 * mask and the softmax (0 = off), as the reference's kernels do (:299-302).
 * The reference's decode_attention_fwd(q, k_buffer, v_buffer, o, req_to_token, b_seq_len,
 * attn_logits, num_kv_splits, sm_scale, page_size, logit_cap)
 * (/root/reference/third_party/mthreads/python/test/wmma/test_accuracy_musa_vllm_mla.py:571-620;
 * page lookup :278-283) for a latent cache whose values are the first d_v columns of its keys.
 */
int smla_decode_dense(int kv_format, const void* q, const void* kv, const int32_t* seq_lens,
                      const int32_t* block_table, void* out, float* lse,
                      int32_t n_tokens, int32_t tokens_per_seq, int32_t n_heads, int32_t max_seq_len,
                      int32_t d_qk, int32_t d_v, int32_t page_size, int32_t block_table_stride,
                      int64_t kv_seq_stride, int64_t kv_rows, float sm_scale, float logit_cap,
                      int32_t n_splits, void* workspace, size_t workspace_bytes, void* stream);

/* Same computation with the exact-fp32 scalar kernel regardless of shape; q/kv/out dtype
 * follows kv_format (bf16 inputs are widened to fp32, out is written in the q dtype).
 * A second, independent device implementation used to cross-check the MFMA kernels at
 * sizes a CPU check cannot reach. */
int smla_fwd_scalar(int kv_format, const void* q, const void* kv, const int32_t* indices,
                    const int32_t* block_table, void* out, float* lse,
                    int32_t n_tokens, int32_t tokens_per_seq, int32_t n_heads, int32_t topk,
                    int32_t d_qk, int32_t d_v, int32_t page_size, int32_t block_table_stride,
                    int64_t kv_seq_stride, int64_t kv_rows, float sm_scale, void* stream);

/* Split count smla_fwd picks for n_splits = 0 on the current device. */
int smla_plan_splits(int kv_format, int32_t n_tokens, int32_t n_heads, int32_t topk);

/*
 * How a split launch is merged on the current device: 1 = inside the launch, 0 = by a second
 * launch (the smla_merge_splits kernel) right behind it on the same stream.
 * The merge inside the launch hands partials from workgroup to workgroup through the L2 cache
 * without fences, so it needs every workgroup of a token behind one L2.  Assumption it rests on:
 * block ids are dealt round-robin to the device's XCDs, the kernels give a token's workgroups ids
 * 8 apart, and the XCD count divides 8.  That holds for a gfx950 device of 256, 128, 64 or at most
 * 32 compute units (a whole MI355X or one of its partitions); on any other compute-unit count, or
 * with FLAGTREE_SMLA_SEPARATE_MERGE=1 in the environment, the second launch is used.
 * No counterpart in the reference, whose stage 2 is always a second launch
 * (test_accuracy_musa_vllm_mla.py:426-477).
 */
int smla_merge_in_launch(void);

/* Bytes of workspace smla_fwd needs for the given split count (0 when n_splits <= 1). */
size_t smla_workspace_bytes(int32_t n_tokens, int32_t n_heads, int32_t d_v, int32_t n_splits);

/* Zero the arrival words at the head of a freshly allocated workspace and write its header (a
 * fill kernel on `stream`, so it may be captured in a graph).  Needed once per allocation, not
 * per call. */
int smla_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/*
 * Health of a workspace after the launches issued so far.  A split launch that finds the
 * workspace without its magic word, an arrival word in an illegal state, or whose last split
 * waits longer than the header's poll limit for the others does not hang and does not merge: it
 * sets a SMLA_WS_STATUS_* bit in the header, writes NaN to the LSE of the rows concerned and
 * ends normally.  A flagged workspace stays unusable until the host has dealt with it: every
 * later split launch on it gives up at once (NaN LSE, `out` rows zero or untouched), because a
 * launch that gave up may have left arrival words in a state the next one cannot tell from a
 * legal one.  This call waits for `stream`, copies the header back, stores the status bits in
 * *status_out (may be NULL) and returns SMLA_OK when they were zero; otherwise it initialises
 * the workspace again (as smla_workspace_init does, unless the magic word was missing) and
 * returns SMLA_EWORKSPACE_STATE.  It synchronises, so a serving loop calls it at the points where
 * it synchronises anyway (after a batch has been read back), or when it meets a NaN LSE.
 * No counterpart in the reference (its two-stage decode keeps no state between launches:
 * test_accuracy_musa_vllm_mla.py:426-477 is a second launch).
 */
int smla_workspace_status(void* workspace, size_t workspace_bytes, void* stream, uint32_t* status_out);

/*
 * Page translation + masking + gather alone (the first stage of smla_fwd, exposed so the
 * integer path can be checked bit for bit):
 *   phys_out  device int32 [T, topk]: physical row or -1
 *   rows_out  device bytes [T, topk, row_bytes]: copy of each selected row, zeros where masked
 *             (may be NULL to get the translation only)
 * row_bytes must be a multiple of 16.
 */
int smla_gather_rows(const void* kv, int32_t row_bytes, const int32_t* indices,
                     const int32_t* block_table, int32_t* phys_out, void* rows_out,
                     int32_t n_tokens, int32_t tokens_per_seq, int32_t topk, int32_t page_size,
                     int32_t block_table_stride, int64_t kv_seq_stride, int64_t kv_rows,
                     void* stream);

/*
 * Merge of split partials (second stage of smla_fwd with n_splits > 1):
 *   part_out f32 [T, n_splits, H, d_v] (each normalised by its own sum), part_lse f32 [T, n_splits, H]
 *   out bf16 [T,H,d_v], lse f32 [T,H];  w_i = exp(lse_i - max) / sum.
 * Counterpart of the reference's stage-2 reduce
 * (test_accuracy_musa_vllm_mla.py:426-477).
 */
int smla_merge_splits(const float* part_out, const float* part_lse, void* out, float* lse,
                      int32_t n_tokens, int32_t n_heads, int32_t d_v, int32_t n_splits,
                      void* stream);

/*
 * KV-cache writer for the fp8 format: quantise latent rows into 656-byte records.
 *   src bf16 [n_rows, 576]; slot device int64 [n_rows] destination row in `records`
 *   (negative = skip), or NULL for rows 0..n_rows-1.
 *   scale_b = max(absmax_b, 2^-126 * 448) / 448 ; code = rtne(x / scale_b), saturating.
 * Counterpart of the reference's cache writer
 * (/root/reference/third_party/cambricon/python/triton/ops/reshape_and_cache.py:1-75)
 * with the group-scale quantiser pattern of
 * /root/reference/third_party/hcu/python/test/unit/sglang/decode_attention_int4kv.py:862-931.
 */
int smla_kv_quantize_fp8(const void* src, const int64_t* slot, void* records,
                         int64_t n_rows, int64_t record_rows, void* stream);

/*
 * KV-cache writer, both formats: append latent rows to the paged pool.
 *   latent bf16 [n_tokens, 576]; slot_mapping device int64 [n_tokens]: destination row of the pool,
 *   slot = page * page_size + offset (negative or >= cache_rows = skip; NULL = rows 0..n_tokens-1);
 *   kv_cache: bf16 rows of 1152 bytes (SMLA_KV_BF16, a plain copy) or 656-byte fp8 records
 *   (SMLA_KV_FP8_B128, quantised as smla_kv_quantize_fp8 does).
 * Same operator as the reference's reshape_and_cache(key, value, key_cache, value_cache,
 * slot_mapping, ...) (/root/reference/third_party/cambricon/python/triton/ops/reshape_and_cache.py:48-75;
 * kernel :7-45, negative slots masked at :40) for a cache that holds one latent row per token.
 */
int smla_kv_write(int kv_format, const void* latent, const int64_t* slot_mapping, void* kv_cache,
                  int64_t n_tokens, int64_t cache_rows, void* stream);

/*
 * Top-k index producer (the step that feeds smla_fwd its `indices`):
 *   indices_out[r, :] = the indices of the k largest entries of scores[r, 0 : len_r), in ascending
 *   index order, padded with -1 when len_r < k;  len_r = context_lens[r] clipped to [0, n_cols]
 *   (NULL = n_cols).  Ties at the k-th value go to the lower index; NaN counts as -inf, -0 as +0.
 *   scores device f32 [n_rows, row_stride] (row_stride >= n_cols), indices_out device int32 [n_rows, k].
 * The reference has the selection only as a language-level primitive that returns the k largest
 * values (/root/reference/third_party/metax/python/triton/language/standard.py:443-444, bitonic
 * top-k :399-435); returning indices, their order and the tie rule are this library's decisions.
 *   workspace  optional device scratch (4-byte aligned) of at least smla_topk_workspace_bytes() bytes, or
 *   NULL.  With few long rows (fewer rows than half the device's compute units) and a workspace,
 *   a row is cut into parts that select their own k largest entries, one workgroup each, and a
 *   second launch on the same stream selects the row's answer from the parts' (same list, entry
 *   for entry, as without a workspace).  Without one, or when the shape does not call for it,
 *   one workgroup takes a row.  The workspace needs no initialisation and carries nothing from
 *   call to call.
 */
int smla_topk_indices(const float* scores, const int32_t* context_lens, int32_t* indices_out,
                      int32_t n_rows, int32_t n_cols, int64_t row_stride, int32_t k, void* workspace,
                      size_t workspace_bytes, void* stream);

/*
 * The same selection, written as physical rows of a paged cache: entry j of rows_out[r, :] is
 *   block_table[r / rows_per_seq, i / page_size] * page_size + i % page_size
 * for the j-th selected position i (in ascending order of i), or -1 where the table has no page for
 * it, the page number is negative or the row lies past kv_rows -- exactly what smla_fwd would make
 * of position i (smla_gather_rows exposes that translation).  A list produced here goes to
 * smla_fwd with block_table = NULL and kv_seq_stride = 0: the attention kernel then starts
 * fetching rows one dependent memory round trip earlier (no page-table look-up of its own).
 * block_table device int32 [n_rows / rows_per_seq, block_table_stride]; everything else as
 * smla_topk_indices.  The reference does the look-up inside its attention kernels
 * (/root/reference/third_party/mthreads/python/test/wmma/test_accuracy_musa_vllm_mla.py:278-283).
 */
int smla_topk_rows(const float* scores, const int32_t* context_lens, const int32_t* block_table,
                   int32_t* rows_out, int32_t n_rows, int32_t n_cols, int64_t row_stride, int32_t k,
                   int32_t rows_per_seq, int32_t page_size, int32_t block_table_stride, int64_t kv_rows,
                   void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of workspace with which smla_topk_indices / smla_topk_rows cut rows of this shape into parts on
 * the current device; 0 when they would not (many rows, short rows).  No counterpart in the reference. */
size_t smla_topk_workspace_bytes(int32_t n_rows, int32_t n_cols, int32_t k);

/*
 * Local GEMM of GEMM + reduce-scatter with chunked-output epilogue:
 *   out_chunk[r][i][n] = bf16_rne( sum_k X[r*M/n_chunks + i][k] * W[k][n] + partial[r*M/n_chunks + i][n] )
 *   X bf16 [M,K] row-major, W bf16 [K,N] row-major, partial f32 [M,N] (may be NULL = 0),
 *   out bf16; chunk r starts at out + r * chunk_stride elements (chunk_stride >= M/n_chunks*N).
 * M % 128 == 0, M % n_chunks == 0, N % 256 == 0, K % 64 == 0.
 * Stands where the reference launches its matmul kernel
 * (/root/reference/python/triton/ops/matmul.py:162-228; kernel :92-151).
 */
int smla_gemm_rs_local(const void* x, const void* w, const float* partial, void* out,
                       int32_t m, int32_t n, int32_t k, int32_t n_chunks, int64_t chunk_stride,
                       void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLAGTREE_SMLA_H */
