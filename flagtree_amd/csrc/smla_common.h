// Shared declarations for the sparse-MLA HIP kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <smla_hw.h>
#include "../../include/flagtree_smla.h"

namespace smla {

constexpr int kDqk = SMLA_D_QK;     // 576
constexpr int kDv = SMLA_D_V;       // 512
constexpr int kRope = kDqk - kDv;   // 64
constexpr int kRowBytesBf16 = kDqk * 2;              // 1152
constexpr int kRowBytesFp8 = SMLA_FP8_RECORD_BYTES;  // 656
constexpr int kFp8ScaleOff = 512;                    // 4 x f32
constexpr int kFp8RopeOff = 528;                     // 64 x bf16
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct Params {
  const void* q;
  const void* kv;
  const int32_t* indices;       // [T, topk], or null: dense, entry j of every token is position j while j < seq_lens[seq]
  const int32_t* seq_lens;      // [n_seqs] context lengths, used when indices is null
  const int32_t* block_table;
  void* out;
  float* lse;
  float* part_out;   // [T, n_splits, H, d_v] when n_splits > 1
  float* part_lse;   // [T, n_splits, H]
  unsigned long long* counters; // [T, ceil(H/64)] arrival tickets + published bits, zero between calls
  uint32_t* ws_header;          // workspace header {magic, status, spin limit, -}; null (and never read) when n_splits == 1
  int32_t n_tokens, tokens_per_seq, n_heads, topk;
  int32_t page_size, bt_stride, n_splits, split_len;
  int64_t kv_seq_stride, kv_rows;
  float sm_scale;
  float logit_cap;              // > 0: every scaled score s becomes logit_cap * tanh(s / logit_cap) before the softmax
  int32_t token_band;           // 0: tokens dealt to the 8 XCDs in turn; > 0: XCD x takes tokens x*token_band .. (x+1)*token_band - 1
  int32_t persist_workgroups;   // > 0: launches that do not split may run this many persistent workgroups (a multiple of 8) instead of one per item
  int32_t merge_in_launch;      // n_splits > 1 only.  1: the last split of a (token, head block) to arrive folds the others' partials
                                // (needs all workgroups of a token behind one L2); 0: every split publishes, a second launch merges
};

// Which token a workgroup works on.  Block ids are dealt round-robin to the 8 XCDs (`xcd` = id % 8,
// `round` = how many tokens that XCD has been given before).  Dealing tokens in turn keeps the
// XCDs level whatever the lists hold.  Contiguous bands (opt-in) are for causal prefill, where
// token t selects among rows 0 .. t: an XCD then gathers from the rows before its band's end
// instead of from the whole cache, so that the early bands' rows stay in its own L2.
__device__ __forceinline__ int token_of(const Params& p, int xcd, int round) {
  return p.token_band > 0 ? xcd * p.token_band + round : round * 8 + xcd;     // (round < token_band by the grid's size)
}

// The capped score in the base-2 units the softmax works in:
//   log2(e) * cap * tanh(x / cap),  x = raw dot product * sm_scale,
// with tanh(y) = 1 - 2 / (exp(2 y) + 1): one exponential and one reciprocal per score.  Exact at
// both ends (exp2 -> inf gives cap, exp2 -> 0 gives -cap); the cancellation near 0 costs an
// absolute error of a few 1e-7 * cap, far inside the 1e-3 bar on the LSE.
struct LogitCap {
  float a, b;                   // a = 2 log2(e) sm_scale / cap,  b = log2(e) cap
  __device__ __forceinline__ LogitCap(float sm_scale, float cap)
      : a(2.f * 1.4426950408889634f * sm_scale / cap), b(1.4426950408889634f * cap) {}
  // (each instruction takes one of the two constants, so both can stay in scalar registers: a
  // vector instruction reads at most one scalar register)
  __device__ __forceinline__ float operator()(float raw) const {
    const float e = __builtin_amdgcn_exp2f(raw * a);
    return b * __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(e + 1.f), 1.f);
  }
};

// Entry j of token t's list: the index list itself, or (dense attention over the whole context)
// position j while it lies inside the sequence.
__device__ __forceinline__ int32_t list_entry(const Params& p, int t, int seq, int j) {
  if (p.indices != nullptr) return p.indices[(size_t)t * p.topk + j];
  return j < p.seq_lens[seq] ? j : -1;
}

// Logical position -> physical row of a paged cache, -1 when masked (negative, past the table,
// a negative page number, or a row past the pool).  Integer-only.  `bt_row` is the sequence's
// page-table row (any address space the caller has it in).
__device__ __forceinline__ int32_t paged_row(int32_t idx, const int32_t* bt_row, int32_t bt_stride, int32_t page_size, int64_t kv_rows) {
  // (branch-free, the page lookup is unconditional: loads inside branches would be issued one
  // at a time, each waiting for the one before it)
  const int64_t cap = (int64_t)bt_stride * page_size;
  const bool in_table = idx >= 0 && idx < cap;
  const int32_t safe = in_table ? idx : 0;
  const int32_t page = bt_row[safe / page_size];
  const int64_t phys = (int64_t)page * page_size + safe % page_size;
  return in_table && page >= 0 && phys < kv_rows ? (int32_t)phys : -1;
}

// Logical top-k entry -> physical row, -1 when masked; only used when the cache is paged.
__device__ __forceinline__ int32_t translate_index(const Params& p, int32_t idx, const int32_t* bt_row) {
  return paged_row(idx, bt_row, p.bt_stride, p.page_size, p.kv_rows);
}

__device__ __forceinline__ int32_t translate_unpaged(const Params& p, int seq, int32_t idx) {
  const int64_t lim = p.kv_seq_stride ? p.kv_seq_stride : p.kv_rows;
  const int64_t phys = (int64_t)seq * p.kv_seq_stride + idx;
  return idx >= 0 && idx < lim && phys < p.kv_rows ? (int32_t)phys : -1;
}

__device__ __forceinline__ int32_t translate_index(const Params& p, int seq, int32_t idx) {
  if (p.block_table != nullptr) return translate_index(p, idx, p.block_table + (int64_t)seq * p.bt_stride);
  return translate_unpaged(p, seq, idx);
}

// Four entries at once: one (uniform) branch on the cache kind around all of them, so that the
// four page lookups are independent loads in one block and go out together.
__device__ __forceinline__ void translate_entries4(const Params& p, int seq, int32_t (&rr)[4]) {
  if (p.block_table != nullptr) {
    const int32_t* bt_row = p.block_table + (int64_t)seq * p.bt_stride;
    int32_t out[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) out[k] = translate_index(p, rr[k], bt_row);
#pragma unroll
    for (int k = 0; k < 4; ++k) rr[k] = out[k];
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) rr[k] = translate_unpaged(p, seq, rr[k]);
  }
}

// ---- split merge inside a launch: arrival protocol ------------------------------------------
// Every (token, head block) owns one 64-bit word of the workspace: high half = arrival tickets,
// low half = one "partial published" bit per split.  The word is zero between launches.  A word
// that is not (a workspace that never went through smla_workspace_init, two launches sharing a
// workspace at the same time) must neither hang the launch nor pass for a result: the header of
// the workspace carries a magic word, a status word the host can read back, and the number of
// polls the last arrival may spend waiting for the others.
constexpr uint32_t kWsMagic = SMLA_WS_MAGIC;
enum { kRolePublish = 0, kRoleLast = 1, kRoleError = 2 };

__device__ __forceinline__ void ws_flag(const Params& p, uint32_t bits) {
  __hip_atomic_fetch_or(p.ws_header + 1, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The header's magic and status words as they stood when the kernel started (one 8-byte load, long
// before the split merge needs it).  A launch that does not split has no workspace and reads nothing.
struct WsHead { uint32_t magic, status; };
__device__ __forceinline__ WsHead ws_read_head(const Params& p) {
  if (p.n_splits <= 1 || !p.merge_in_launch) return WsHead{0u, 0u};
  const uint2 h = *reinterpret_cast<const uint2*>(p.ws_header);
  return WsHead{h.x, h.y};
}

// One thread of the workgroup: take an arrival ticket and decide the workgroup's role.  `head`
// is the header as read at kernel entry.  A workspace that an earlier launch has flagged stays
// unusable until the host has looked at it (smla_workspace_status re-initialises it): a launch
// that gave up may have left tickets or published bits behind, and a word in such a state can
// look legal to the next launch, which would then fold in a stale partial.  So a non-zero status
// makes every split of every later launch give up at once, without touching the word.
// An inconsistent word (more arrivals than splits, my own bit or a bit past the last split already
// set, more published than arrived) flags the workspace and zeroes the word.
__device__ __forceinline__ int ws_arrive(const Params& p, unsigned long long* word, WsHead head, int ns, int sp) {
  if (!p.merge_in_launch) return kRolePublish;       // a second launch merges: nothing to agree on
  if (head.magic != kWsMagic) {
    ws_flag(p, SMLA_WS_STATUS_UNINITIALISED);
    return kRoleError;
  }
  if (head.status != 0) return kRoleError;
  const unsigned long long old = __hip_atomic_fetch_add(word, 1ull << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint32_t ticket = (uint32_t)(old >> 32), bits = (uint32_t)old;
  const uint32_t legal = ns >= 32 ? 0xffffffffu : (1u << ns) - 1u;
  if (ticket >= (uint32_t)ns || (bits & ~legal) != 0 || (bits & (1u << sp)) != 0 || (uint32_t)__popc(bits) > ticket) {
    ws_flag(p, SMLA_WS_STATUS_STALE);
    __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return kRoleError;
  }
  return ticket == (uint32_t)ns - 1 ? kRoleLast : kRolePublish;
}

// One thread of a publishing workgroup, after its partial's stores have been acknowledged.
__device__ __forceinline__ void ws_publish(const Params& p, unsigned long long* word, int sp) {
  if (p.merge_in_launch) __hip_atomic_fetch_or(word, 1ull << sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One thread of the last workgroup to arrive: poll until every other split has published, at
// most `spin limit` times (the others hold tickets, so they are past their loops and publish
// within microseconds; the limit is what ends the wait when the word was not what it seemed).
// Gives up by flagging the workspace and zeroing the word.
__device__ __forceinline__ bool ws_wait_published(const Params& p, unsigned long long* word, int ns, int sp) {
  const unsigned long long legal = ns >= 32 ? 0xffffffffull : (1ull << ns) - 1ull;
  const unsigned long long others = legal & ~(1ull << sp);
  const uint32_t limit = __hip_atomic_load(p.ws_header + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (uint32_t n = 0; n < limit; ++n) {
    if ((__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & others) == others) return true;
    __builtin_amdgcn_s_sleep(2);
  }
  ws_flag(p, SMLA_WS_STATUS_TIMEOUT);
  __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return false;
}

// Partials cross workgroups without fences: stored and loaded at agent scope (through the L2,
// past the per-CU cache; hw::store_b128_agent / hw::load_b128_agent), a bit is published only
// after the stores have been acknowledged.  The loads are ones the compiler can see: it counts
// them in flight and waits where a landing register is first read, whatever copies or spills
// it puts in between.

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float((uint32_t)b << 16);
}

// fp32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// e4m3fn code -> fp32 by the closed form (sign, 4-bit exponent bias 7, 3-bit mantissa).
__device__ __forceinline__ float e4m3_to_f32(uint32_t c) {
  const uint32_t e = (c >> 3) & 15u, m = c & 7u;
  float v;
  if (e == 0) v = (float)m * 0x1p-9f;
  else if (e == 15u && m == 7u) v = __uint_as_float(0x7fc00000u);
  else v = __uint_as_float(((e + 120u) << 23) | (m << 20));
  return (c & 0x80u) ? -v : v;
}

// fp32 -> e4m3fn code, round to nearest even, saturating at +-448, NaN -> 0x7f.
__device__ __forceinline__ uint32_t f32_to_e4m3(float x) {
  const uint32_t sign = (__float_as_uint(x) >> 24) & 0x80u;
  float a = fabsf(x);
  if (a != a) return 0x7fu;
  a = fminf(a, 448.0f);
  uint32_t code;
  if (a < 0x1p-6f) {
    code = (uint32_t)rintf(a * 512.0f);            // subnormal grid 2^-9; 8 == smallest normal
  } else {
    uint32_t u = __float_as_uint(a);
    u += 0x7ffffu + ((u >> 20) & 1u);
    code = (u >> 20) - (120u << 3);
    if (code > 0x7eu) code = 0x7eu;
  }
  return code | sign;
}

int launch_fwd_scalar(int kv_format, const Params& p, hipStream_t s);
int launch_fwd_tall(int kv_format, const Params& p, hipStream_t s);    // n_heads > 32 (logit cap: a second instantiation)
int launch_fwd_short(int kv_format, const Params& p, hipStream_t s);   // n_heads <= 32
int launch_fwd_group(int kv_format, const Params& p, hipStream_t s);   // n_heads > 32, bf16 rows or fp8 records, 128 heads per workgroup, a wavefront per 32 heads (opt-in)
int launch_fwd_few_fp8(const Params& p, hipStream_t s);                // n_heads <= 32, fp8 records, two workgroups per CU (opt-in)
int launch_fwd_few_f8(const Params& p, hipStream_t s);                 // n_heads <= 32, fp8 records contracted by fp8 MFMAs, two workgroups per CU (opt-in)
int launch_merge(const float* part_out, const float* part_lse, void* out, float* lse,
                 int n_tokens, int n_heads, int d_v, int n_splits, bool partials_bf16, hipStream_t s);
int launch_gather(const Params& p, int row_bytes, int32_t* phys_out, void* rows_out, hipStream_t s);
int launch_quantize(const void* src, const int64_t* slot, void* records, int64_t n_rows,
                    int64_t record_rows, hipStream_t s);
int launch_kv_copy(const void* src, const int64_t* slot, void* pool, int64_t n_rows, int64_t pool_rows, hipStream_t s);
// What the index producer writes for a selected position: the position itself, or (block_table
// given) the physical row of the paged cache it lives in, -1 when masked.
struct TopkPaging {
  const int32_t* block_table;   // [n_rows / rows_per_seq, bt_stride] or null
  int32_t bt_stride, page_size, rows_per_seq;
  int64_t kv_rows;
};
int launch_topk_indices(const float* scores, const int32_t* context_lens, int32_t* out, int n_rows,
                        int n_cols, long long row_stride, int k, const TopkPaging& paging, void* workspace,
                        size_t workspace_bytes, int n_cu, hipStream_t s);
size_t topk_workspace_bytes(int n_rows, int n_cols, int k, int n_cu);
int launch_zero(void* ptr, size_t bytes, hipStream_t s);
int launch_workspace_init(void* workspace, hipStream_t s);
int launch_gemm_rs(const void* x, const void* w, const float* partial, void* out, int m, int n,
                   int k, int n_chunks, int64_t chunk_stride, int n_cu, hipStream_t s);

inline int hip_status(hipError_t e) { return e == hipSuccess ? SMLA_OK : SMLA_EHIP_BASE - (int)e; }

}  // namespace smla
