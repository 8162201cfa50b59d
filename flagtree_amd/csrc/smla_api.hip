// C ABI of libflagtree_smla.so: argument validation and kernel dispatch.
#include "smla_common.h"

#include <stdlib.h>

using namespace smla;

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_common(const void* q, const void* kv, const int32_t* indices, const void* out,
                 const float* lse, int32_t n_tokens, int32_t tokens_per_seq, int32_t n_heads,
                 int32_t topk, int32_t d_qk, int32_t d_v, int32_t page_size,
                 const int32_t* block_table, int32_t bt_stride, int64_t kv_seq_stride,
                 int64_t kv_rows) {
  if (!q || !kv || !indices || !out || !lse) return SMLA_EINVAL_NULLPTR;   // (`indices`: the list, or the sequence lengths of a dense call)
  if (n_tokens <= 0 || tokens_per_seq <= 0 || n_heads <= 0 || topk <= 0) return SMLA_EINVAL_SHAPE;
  if (n_tokens % tokens_per_seq != 0) return SMLA_EINVAL_SHAPE;
  if (d_qk != kDqk || d_v != kDv) return SMLA_EINVAL_SHAPE;
  if (kv_rows <= 0 || kv_rows > 0x7fffffffLL || kv_seq_stride < 0) return SMLA_EINVAL_SHAPE;
  if (block_table && (page_size <= 0 || bt_stride <= 0)) return SMLA_EINVAL_SHAPE;
  if (!aligned16(q) || !aligned16(kv) || !aligned16(out)) return SMLA_EINVAL_ALIGN;
  if ((reinterpret_cast<uintptr_t>(indices) & 3u) != 0) return SMLA_EINVAL_ALIGN;   // read 4 bytes at a time
  return SMLA_OK;
}

// Kernels that have passed the parity checks but whose speed has not been measured on hardware
// yet stay behind a switch until it has (read at every call): FLAGTREE_SMLA_FEW_FP8=1 sends few-heads launches over an
// fp8 cache to the two-workgroups-per-CU kernel (smla_mfma_few_fp8.hip).  Read at every call.
// FLAGTREE_SMLA_HEAD_GROUPS=1 sends many-heads launches (either cache format) to the kernel that
// takes 128 heads per workgroup, a wavefront per 32 heads (smla_mfma_group.hip).
bool head_groups_enabled() {
  const char* e = getenv("FLAGTREE_SMLA_HEAD_GROUPS");
  return e != nullptr && e[0] == '1';
}

bool few_fp8_enabled() {
  const char* e = getenv("FLAGTREE_SMLA_FEW_FP8");
  return e != nullptr && e[0] == '1';
}

// FLAGTREE_SMLA_FP8_MFMA=1 sends few-heads launches over an fp8 cache to the kernel that contracts
// the records' e4m3 codes on the matrix cores as they are (smla_mfma_few_f8.hip; also two
// workgroups per CU).  It wins over FLAGTREE_SMLA_FEW_FP8.
// FLAGTREE_SMLA_PERSIST=1: many-heads launches that do not split and have at least two items per
// compute unit (prefill, dense decode over many tokens) run one persistent workgroup per compute
// unit, which sends for the next item's indices and Q under the current item's epilogue.
bool persist_enabled() {
  const char* e = getenv("FLAGTREE_SMLA_PERSIST");
  return e != nullptr && e[0] == '1';
}

bool fp8_mfma_enabled() {
  const char* e = getenv("FLAGTREE_SMLA_FP8_MFMA");
  return e != nullptr && e[0] == '1';
}

// FLAGTREE_SMLA_TOKEN_BANDS=1 gives each XCD a contiguous band of tokens instead of every eighth
// token (for causal prefill; see token_of).
bool token_bands_enabled() {
  const char* e = getenv("FLAGTREE_SMLA_TOKEN_BANDS");
  return e != nullptr && e[0] == '1';
}

// Compute units of the current device (256 when there is none to ask: planning calls made on a
// machine without a GPU).  Asked at every call: the answer belongs to the device that is current
// now, the query is a table look-up in the runtime, and a cache would have to be keyed by device
// and guarded against concurrent callers for no measurable gain.
int device_cus() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
    return n;
  return 256;
}

// The merge inside the launch passes partials between workgroups through the L2 without fences,
// which is only correct when every workgroup of a token runs behind the same L2.  The kernels
// give those workgroups block ids 8 apart; the hardware deals block ids round-robin to the XCDs of
// the device, so ids 8 apart share an XCD whenever the XCD count divides 8.  On gfx950 an XCD has
// 32 compute units and a device (a whole GPU or a partition of it) has 1, 2, 4 or 8 of them; any
// other compute-unit count is a layout this code knows nothing about, and there, or when
// FLAGTREE_SMLA_SEPARATE_MERGE=1 asks for it, every split publishes its partial and a second
// launch merges them (a kernel boundary makes the partials visible everywhere).
bool merge_in_launch_ok() {
  const char* e = getenv("FLAGTREE_SMLA_SEPARATE_MERGE");
  if (e != nullptr && e[0] == '1') return false;
  const int n = device_cus();
  return n <= 32 || n == 64 || n == 128 || n == 256;
}

}  // namespace

extern "C" {

const char* smla_strerror(int status) {
  switch (status) {
    case SMLA_OK: return "ok";
    case SMLA_EINVAL_NULLPTR: return "a required pointer is NULL";
    case SMLA_EINVAL_SHAPE: return "unsupported or inconsistent shape";
    case SMLA_EINVAL_ALIGN: return "a pointer is not 16-byte aligned";
    case SMLA_EINVAL_WORKSPACE: return "workspace missing or too small";
    case SMLA_EINVAL_SPLITS: return "n_splits out of range for this top-k length";
    case SMLA_ENODEVICE: return "no usable gfx950 device";
    case SMLA_EINVAL_SCALE: return "sm_scale must be positive and finite, logit_cap non-negative and finite";
    case SMLA_EWORKSPACE_STATE: return "a split launch flagged its workspace (uninitialised, shared by overlapping launches, or a split never arrived)";
    default: break;
  }
  if (status <= SMLA_EHIP_BASE) return hipGetErrorString((hipError_t)(SMLA_EHIP_BASE - status));
  return "unknown status";
}

int smla_abi_version(void) { return 4; }

int smla_merge_in_launch(void) { return merge_in_launch_ok() ? 1 : 0; }

// Workspace layout: [0, SMLA_WS_HEADER_OFFSET) arrival words (zero between calls), the 64-byte
// header {magic, status, poll limit, -} up to SMLA_WS_COUNTER_BYTES, then the partial outputs [T, n_splits, H, d_v] f32 and the partial LSEs [T, n_splits, H] f32.
size_t smla_workspace_bytes(int32_t n_tokens, int32_t n_heads, int32_t d_v, int32_t n_splits) {
  if (n_splits <= 1 || n_tokens <= 0 || n_heads <= 0 || d_v <= 0) return 0;
  return SMLA_WS_COUNTER_BYTES + (size_t)n_tokens * n_splits * n_heads * ((size_t)d_v + 1) * sizeof(float);
}

int smla_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
  if (!workspace) return SMLA_EINVAL_NULLPTR;
  if (!aligned16(workspace)) return SMLA_EINVAL_ALIGN;
  if (workspace_bytes < SMLA_WS_COUNTER_BYTES) return SMLA_EINVAL_WORKSPACE;
  return launch_workspace_init(workspace, static_cast<hipStream_t>(stream));
}

int smla_workspace_status(void* workspace, size_t workspace_bytes, void* stream, uint32_t* status_out) {
  if (!workspace) return SMLA_EINVAL_NULLPTR;
  if (!aligned16(workspace)) return SMLA_EINVAL_ALIGN;
  if (workspace_bytes < SMLA_WS_COUNTER_BYTES) return SMLA_EINVAL_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint8_t* header = static_cast<uint8_t*>(workspace) + SMLA_WS_HEADER_OFFSET;
  uint32_t h[4] = {0, 0, 0, 0};
  hipError_t e = hipMemcpyAsync(h, header, sizeof(h), hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  if (e != hipSuccess) return hip_status(e);
  uint32_t status = h[1];
  if (h[0] != SMLA_WS_MAGIC) status |= SMLA_WS_STATUS_UNINITIALISED;
  if (status_out) *status_out = status;
  if (status == 0) return SMLA_OK;
  if (h[0] == SMLA_WS_MAGIC) {
    // A flagged launch may have left arrival words behind (a split that arrived after the word
    // was given up on): start over.  An uninitialised workspace stays as it is.
    const int rc = launch_workspace_init(workspace, s);
    if (rc != SMLA_OK) return rc;
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_status(e);
  }
  return SMLA_EWORKSPACE_STATE;
}

int smla_plan_splits(int kv_format, int32_t n_tokens, int32_t n_heads, int32_t topk) {
  if (n_tokens <= 0 || n_heads <= 0 || topk <= 0) return 1;
  if (kv_format == SMLA_KV_F32) return 1;
  // one 4-wave workgroup per CU is resident at a time; each covers 64 (or, for <= 32 heads, 16)
  // heads of one token
  // (the opt-in fp8 kernel keeps two workgroups per CU; every further split adds a partial to publish and fold)
  const bool few_fp8 = kv_format == SMLA_KV_FP8_B128 && n_heads <= 32 && (few_fp8_enabled() || fp8_mfma_enabled());
  const int slots = few_fp8 ? 2 * device_cus() : device_cus();
  const bool wide = n_heads > 32 && head_groups_enabled();
  const int per_wg = n_heads <= 32 ? 16 : (wide ? 128 : 64);
  const long long groups = (long long)n_tokens * ((n_heads + per_wg - 1) / per_wg);
  int want = (int)((slots + groups - 1) / groups);
  const int min_len = 256;                                 // keep at least 4 tiles per split
  int cap = topk / min_len;
  if (cap < 1) cap = 1;
  if (want > cap) want = cap;
  if (want > SMLA_MAX_SPLITS) want = SMLA_MAX_SPLITS;
  if (groups * 8 > SMLA_WS_HEADER_OFFSET) want = 1;        // more (token, head block) pairs than arrival words
  return want < 1 ? 1 : want;
}

static int fill_params(Params& p, const void* q, const void* kv, const int32_t* indices,
                       const int32_t* block_table, void* out, float* lse, int32_t n_tokens,
                       int32_t tokens_per_seq, int32_t n_heads, int32_t topk, int32_t page_size,
                       int32_t bt_stride, int64_t kv_seq_stride, int64_t kv_rows, float sm_scale) {
  p.q = q; p.kv = kv; p.indices = indices; p.seq_lens = nullptr; p.block_table = block_table; p.out = out; p.lse = lse;
  p.part_out = nullptr; p.part_lse = nullptr; p.counters = nullptr;
  p.ws_header = nullptr;                                        // (only a split launch has a workspace, and only it reads the header)
  p.n_tokens = n_tokens; p.tokens_per_seq = tokens_per_seq; p.n_heads = n_heads; p.topk = topk;
  p.page_size = block_table ? page_size : 1; p.bt_stride = block_table ? bt_stride : 0;
  p.n_splits = 1; p.split_len = topk;
  p.kv_seq_stride = kv_seq_stride; p.kv_rows = kv_rows; p.sm_scale = sm_scale; p.logit_cap = 0.f;
  p.token_band = token_bands_enabled() ? (n_tokens + 7) / 8 : 0;
  p.merge_in_launch = 0;
  p.persist_workgroups = 0;
  return SMLA_OK;
}

// Shared body of the forward entry points.  `dense`: `indices` holds the per-sequence context
// lengths instead of an index list and every token attends to positions 0 .. length-1 (< topk).
static int fwd_impl(bool dense, int kv_format, const void* q, const void* kv, const int32_t* indices,
                    const int32_t* block_table, void* out, float* lse, int32_t n_tokens,
                    int32_t tokens_per_seq, int32_t n_heads, int32_t topk, int32_t d_qk, int32_t d_v,
                    int32_t page_size, int32_t block_table_stride, int64_t kv_seq_stride, int64_t kv_rows,
                    float sm_scale, float logit_cap, int32_t n_splits, void* workspace, size_t workspace_bytes,
                    void* stream) {
  int rc = check_common(q, kv, indices, out, lse, n_tokens, tokens_per_seq, n_heads, topk, d_qk, d_v,
                        page_size, block_table, block_table_stride, kv_seq_stride, kv_rows);
  if (rc != SMLA_OK) return rc;
  if (kv_format != SMLA_KV_BF16 && kv_format != SMLA_KV_FP8_B128 && kv_format != SMLA_KV_F32)
    return SMLA_EINVAL_SHAPE;
  if (n_splits < 0 || n_splits > SMLA_MAX_SPLITS) return SMLA_EINVAL_SPLITS;
  if (!(sm_scale > 0.f) || !(sm_scale < INFINITY)) return SMLA_EINVAL_SCALE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  Params p;
  fill_params(p, q, kv, indices, block_table, out, lse, n_tokens, tokens_per_seq, n_heads, topk,
              page_size, block_table_stride, kv_seq_stride, kv_rows, sm_scale);
  if (dense) { p.seq_lens = indices; p.indices = nullptr; }
  if (!(logit_cap >= 0.f) || !(logit_cap < INFINITY)) return SMLA_EINVAL_SCALE;
  p.logit_cap = logit_cap;
  if (kv_format == SMLA_KV_F32) return launch_fwd_scalar(kv_format, p, s);

  if (n_splits == 0) {
    n_splits = smla_plan_splits(kv_format, n_tokens, n_heads, topk);
    // without a big enough workspace fall back to the smallest legal split count
    if (n_splits > 1 && (!workspace || workspace_bytes < smla_workspace_bytes(n_tokens, n_heads, d_v, n_splits)))
      n_splits = 1;
  }
  if (n_splits > topk) n_splits = topk;
  const int split_len = ((topk + n_splits - 1) / n_splits + 31) / 32 * 32;   // whole tiles per split
  n_splits = (topk + split_len - 1) / split_len;
  p.n_splits = n_splits;
  p.split_len = split_len;
  if (n_splits > 1) {
    const size_t need = smla_workspace_bytes(n_tokens, n_heads, d_v, n_splits);
    if (!workspace || workspace_bytes < need || !aligned16(workspace)) return SMLA_EINVAL_WORKSPACE;
    if ((size_t)n_tokens * ((n_heads + 15) / 16) * 8 > SMLA_WS_HEADER_OFFSET) return SMLA_EINVAL_SPLITS;
    p.counters = static_cast<unsigned long long*>(workspace);
    p.ws_header = reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(workspace) + SMLA_WS_HEADER_OFFSET);
    p.part_out = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + SMLA_WS_COUNTER_BYTES);
    p.part_lse = p.part_out + (size_t)n_tokens * n_splits * n_heads * d_v;
    p.merge_in_launch = merge_in_launch_ok() ? 1 : 0;
  }
  if (persist_enabled() && device_cus() % 8 == 0) p.persist_workgroups = device_cus();
  const bool head_groups = n_heads > 32 && head_groups_enabled();    // (that kernel keeps its partial sums as bf16)
  if (head_groups) rc = launch_fwd_group(kv_format, p, s);
  else if (n_heads > 32) rc = launch_fwd_tall(kv_format, p, s);
  else if (kv_format == SMLA_KV_FP8_B128 && fp8_mfma_enabled()) rc = launch_fwd_few_f8(p, s);
  else if (kv_format == SMLA_KV_FP8_B128 && few_fp8_enabled()) rc = launch_fwd_few_fp8(p, s);
  else rc = launch_fwd_short(kv_format, p, s);
  if (rc != SMLA_OK || n_splits == 1 || p.merge_in_launch) return rc;
  return launch_merge(p.part_out, p.part_lse, out, lse, n_tokens, n_heads, d_v, n_splits, head_groups, s);
}

int smla_fwd(int kv_format, const void* q, const void* kv, const int32_t* indices,
             const int32_t* block_table, void* out, float* lse, int32_t n_tokens,
             int32_t tokens_per_seq, int32_t n_heads, int32_t topk, int32_t d_qk, int32_t d_v,
             int32_t page_size, int32_t block_table_stride, int64_t kv_seq_stride, int64_t kv_rows,
             float sm_scale, int32_t n_splits, void* workspace, size_t workspace_bytes,
             void* stream) {
  return fwd_impl(false, kv_format, q, kv, indices, block_table, out, lse, n_tokens, tokens_per_seq, n_heads,
                  topk, d_qk, d_v, page_size, block_table_stride, kv_seq_stride, kv_rows, sm_scale, 0.f, n_splits,
                  workspace, workspace_bytes, stream);
}

int smla_decode_dense(int kv_format, const void* q, const void* kv, const int32_t* seq_lens,
                      const int32_t* block_table, void* out, float* lse, int32_t n_tokens,
                      int32_t tokens_per_seq, int32_t n_heads, int32_t max_seq_len, int32_t d_qk,
                      int32_t d_v, int32_t page_size, int32_t block_table_stride, int64_t kv_seq_stride,
                      int64_t kv_rows, float sm_scale, float logit_cap, int32_t n_splits, void* workspace,
                      size_t workspace_bytes, void* stream) {
  return fwd_impl(true, kv_format, q, kv, seq_lens, block_table, out, lse, n_tokens, tokens_per_seq, n_heads,
                  max_seq_len, d_qk, d_v, page_size, block_table_stride, kv_seq_stride, kv_rows, sm_scale, logit_cap,
                  n_splits, workspace, workspace_bytes, stream);
}

int smla_fwd_scalar(int kv_format, const void* q, const void* kv, const int32_t* indices,
                    const int32_t* block_table, void* out, float* lse, int32_t n_tokens,
                    int32_t tokens_per_seq, int32_t n_heads, int32_t topk, int32_t d_qk,
                    int32_t d_v, int32_t page_size, int32_t block_table_stride,
                    int64_t kv_seq_stride, int64_t kv_rows, float sm_scale, void* stream) {
  int rc = check_common(q, kv, indices, out, lse, n_tokens, tokens_per_seq, n_heads, topk, d_qk, d_v,
                        page_size, block_table, block_table_stride, kv_seq_stride, kv_rows);
  if (rc != SMLA_OK) return rc;
  if (n_heads > 65535 || n_tokens > 65535) return SMLA_EINVAL_SHAPE;
  if (kv_format != SMLA_KV_BF16 && kv_format != SMLA_KV_FP8_B128 && kv_format != SMLA_KV_F32)
    return SMLA_EINVAL_SHAPE;
  if (!(sm_scale > 0.f) || !(sm_scale < INFINITY)) return SMLA_EINVAL_SCALE;
  Params p;
  fill_params(p, q, kv, indices, block_table, out, lse, n_tokens, tokens_per_seq, n_heads, topk,
              page_size, block_table_stride, kv_seq_stride, kv_rows, sm_scale);
  return launch_fwd_scalar(kv_format, p, static_cast<hipStream_t>(stream));
}

int smla_gather_rows(const void* kv, int32_t row_bytes, const int32_t* indices,
                     const int32_t* block_table, int32_t* phys_out, void* rows_out,
                     int32_t n_tokens, int32_t tokens_per_seq, int32_t topk, int32_t page_size,
                     int32_t block_table_stride, int64_t kv_seq_stride, int64_t kv_rows,
                     void* stream) {
  if (!kv || !indices || !phys_out) return SMLA_EINVAL_NULLPTR;
  if (n_tokens <= 0 || tokens_per_seq <= 0 || topk <= 0 || n_tokens % tokens_per_seq != 0 ||
      n_tokens > 65535)
    return SMLA_EINVAL_SHAPE;
  if (row_bytes <= 0 || row_bytes % 16 != 0) return SMLA_EINVAL_SHAPE;
  if (kv_rows <= 0 || kv_rows > 0x7fffffffLL || kv_seq_stride < 0) return SMLA_EINVAL_SHAPE;
  if (block_table && (page_size <= 0 || block_table_stride <= 0)) return SMLA_EINVAL_SHAPE;
  if (!aligned16(kv) || (rows_out && !aligned16(rows_out))) return SMLA_EINVAL_ALIGN;
  Params p;
  fill_params(p, kv, kv, indices, block_table, rows_out, nullptr, n_tokens, tokens_per_seq, 1, topk,
              page_size, block_table_stride, kv_seq_stride, kv_rows, 1.f);
  return launch_gather(p, row_bytes, phys_out, rows_out, static_cast<hipStream_t>(stream));
}

int smla_merge_splits(const float* part_out, const float* part_lse, void* out, float* lse,
                      int32_t n_tokens, int32_t n_heads, int32_t d_v, int32_t n_splits,
                      void* stream) {
  if (!part_out || !part_lse || !out || !lse) return SMLA_EINVAL_NULLPTR;
  if (n_tokens <= 0 || n_heads <= 0 || d_v != kDv || (long long)n_tokens * n_heads > 0x7fffffffLL) return SMLA_EINVAL_SHAPE;
  if (n_splits < 1 || n_splits > SMLA_MAX_SPLITS) return SMLA_EINVAL_SPLITS;
  if (!aligned16(part_out) || !aligned16(out)) return SMLA_EINVAL_ALIGN;
  return launch_merge(part_out, part_lse, out, lse, n_tokens, n_heads, d_v, n_splits, false,
                      static_cast<hipStream_t>(stream));
}

int smla_kv_quantize_fp8(const void* src, const int64_t* slot, void* records, int64_t n_rows,
                         int64_t record_rows, void* stream) {
  if (!src || !records) return SMLA_EINVAL_NULLPTR;
  if (n_rows < 0 || record_rows <= 0 || n_rows > 0x1ffffffffLL) return SMLA_EINVAL_SHAPE;
  if (!aligned16(src) || !aligned16(records)) return SMLA_EINVAL_ALIGN;
  return launch_quantize(src, slot, records, n_rows, record_rows, static_cast<hipStream_t>(stream));
}

int smla_kv_write(int kv_format, const void* latent, const int64_t* slot_mapping, void* kv_cache,
                  int64_t n_tokens, int64_t cache_rows, void* stream) {
  if (!latent || !kv_cache) return SMLA_EINVAL_NULLPTR;
  if (n_tokens < 0 || cache_rows <= 0 || n_tokens > 0x1ffffffffLL) return SMLA_EINVAL_SHAPE;
  if (!aligned16(latent) || !aligned16(kv_cache)) return SMLA_EINVAL_ALIGN;
  if (kv_format == SMLA_KV_BF16)
    return launch_kv_copy(latent, slot_mapping, kv_cache, n_tokens, cache_rows, static_cast<hipStream_t>(stream));
  if (kv_format == SMLA_KV_FP8_B128)
    return launch_quantize(latent, slot_mapping, kv_cache, n_tokens, cache_rows, static_cast<hipStream_t>(stream));
  return SMLA_EINVAL_SHAPE;
}

size_t smla_topk_workspace_bytes(int32_t n_rows, int32_t n_cols, int32_t k) {
  if (n_rows <= 0 || n_cols <= 0 || k <= 0) return 0;
  return topk_workspace_bytes(n_rows, n_cols, k, device_cus());
}

int smla_topk_indices(const float* scores, const int32_t* context_lens, int32_t* indices_out,
                      int32_t n_rows, int32_t n_cols, int64_t row_stride, int32_t k, void* workspace,
                      size_t workspace_bytes, void* stream) {
  if (!scores || !indices_out) return SMLA_EINVAL_NULLPTR;
  if (n_rows < 0 || n_cols <= 0 || k <= 0 || row_stride < n_cols) return SMLA_EINVAL_SHAPE;
  if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) return SMLA_EINVAL_ALIGN;
  return launch_topk_indices(scores, context_lens, indices_out, n_rows, n_cols, row_stride, k, TopkPaging{nullptr, 0, 1, 1, 0},
                             workspace, workspace_bytes, device_cus(), static_cast<hipStream_t>(stream));
}

int smla_topk_rows(const float* scores, const int32_t* context_lens, const int32_t* block_table, int32_t* rows_out,
                   int32_t n_rows, int32_t n_cols, int64_t row_stride, int32_t k, int32_t rows_per_seq,
                   int32_t page_size, int32_t block_table_stride, int64_t kv_rows, void* workspace,
                   size_t workspace_bytes, void* stream) {
  if (!scores || !rows_out || !block_table) return SMLA_EINVAL_NULLPTR;
  if (n_rows < 0 || n_cols <= 0 || k <= 0 || row_stride < n_cols) return SMLA_EINVAL_SHAPE;
  if (rows_per_seq <= 0 || n_rows % rows_per_seq != 0 || page_size <= 0 || block_table_stride <= 0) return SMLA_EINVAL_SHAPE;
  if (kv_rows <= 0 || kv_rows > 0x7fffffffLL) return SMLA_EINVAL_SHAPE;
  if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) return SMLA_EINVAL_ALIGN;
  return launch_topk_indices(scores, context_lens, rows_out, n_rows, n_cols, row_stride, k,
                             TopkPaging{block_table, block_table_stride, page_size, rows_per_seq, kv_rows}, workspace,
                             workspace_bytes, device_cus(), static_cast<hipStream_t>(stream));
}

int smla_gemm_rs_local(const void* x, const void* w, const float* partial, void* out, int32_t m,
                       int32_t n, int32_t k, int32_t n_chunks, int64_t chunk_stride,
                       void* stream) {
  if (!x || !w || !out) return SMLA_EINVAL_NULLPTR;
  if (m <= 0 || n <= 0 || k <= 0 || n_chunks <= 0) return SMLA_EINVAL_SHAPE;
  if (m % 128 != 0 || m % n_chunks != 0 || n % 256 != 0 || k % 64 != 0) return SMLA_EINVAL_SHAPE;
  if (chunk_stride < (int64_t)(m / n_chunks) * n) return SMLA_EINVAL_SHAPE;
  if (!aligned16(x) || !aligned16(w) || !aligned16(out) || (partial && !aligned16(partial)) ||
      (chunk_stride % 8) != 0)
    return SMLA_EINVAL_ALIGN;
  return launch_gemm_rs(x, w, partial, out, m, n, k, n_chunks, chunk_stride, device_cus(),
                        static_cast<hipStream_t>(stream));
}

}  // extern "C"
