// Sparse-MLA forward, MFMA kernel for many heads.
//
// One workgroup of 4 wavefronts handles (token, block of 64 heads, split of the top-k list).
// Wavefront w = (hg, dh): head group hg = w/2 (32 heads) and half dh = w%2.  The workgroup gathers
// 32-token tiles of latent rows into a ring of four LDS slots with global -> LDS DMA; the loads of
// a tile are issued three tiles ahead of its use and threaded through the MFMA streams, so the
// memory pipe is fed evenly and a wavefront is never parked on a full queue for long.
// The loop is software pipelined with one barrier per tile; in iteration i each wavefront
//   1. scores tokens 16*dh .. +15 of tile i+1 against its 32 heads
//        S^T[16 tok x 32 heads] = K_rows[16 x 576] . Q^T[576 x 32]     v_mfma_f32_16x16x32_bf16
//        (A = LDS rows, B = Q held in VGPRs for the whole kernel),
//   2. turns them into bf16 probabilities and drops them into the P buffer of tile i+1 in LDS,
//   3. accumulates output columns 256*dh .. +255 over all 32 tokens of tile i
//        O[32 heads x 256] += P[32 heads x 32 tok] . V[32 tok x 256]    v_mfma_f32_32x32x16_bf16
//        (A = P from LDS, B = V through transposing LDS reads of the same tile).
// An fp8 cache takes the same road with one more stage: raw records -> LDS by the same moves,
// LDS -> LDS conversion to bf16 tiles under the P.V MFMAs one tile ahead of the scores (Fp8Pipe).
// The workgroups of one token (head blocks x splits) are given ids 8 apart so they land on the
// same XCD: the head blocks share the L2 for the rows they both gather, and the splits are
// merged by whichever workgroup of a (token, head block) finishes last.
//
// Register layouts (wave64):
//   v_mfma_f32_16x16x32_bf16  A: lane l holds A[m = l%16][k = 8*(l/16) .. +7]   B: B[k = 8*(l/16) .. +7][n = l%16]
//                             D: lane l, reg r holds D[m = 4*(l/16) + r][n = l%16]
//   v_mfma_f32_32x32x16_bf16  A: lane l holds A[m = l%32][k = 8*(l/32) .. +7]   B: B[k = 8*(l/32) .. +7][n = l%32]
//                             D: lane l, reg r holds D[m = 8*(r/4) + 4*(l/32) + r%4][n = l%32]
//   ds_read_b64_tr_b16: inside each group of 16 lanes, lane i receives element (i%4) of the
//   8-byte rows addressed by lanes (i/4), (i/4)+4, (i/4)+8, (i/4)+12.
#include "smla_common.h"
#include "smla_fp8_pipe.h"

namespace smla {

using hw::bf16x8;
using hw::bf16x4;
using hw::short4v;
using hw::f32x4;
using hw::u32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr int kNT = 256;                      // threads per workgroup
constexpr int kTN = 32;                       // tokens per tile
constexpr int kSlots = 4;                     // ring slots
// LDS tile layout.  The 512 NoPE / V columns of row r occupy the 1 KB at r * kMainStride, with
// 16-byte chunk c stored at chunk position c ^ swz(r), swz(r) = ((r & 3) << 2) | ((r >> 2) & 3).
// LDS has 64 banks of 4 bytes; a 16-byte read is served 16 lanes at a time and a transposing 8-byte
// read 32 lanes at a time.  The score MFMAs read one chunk column of 16 consecutive rows (swz is a
// bijection on 16 consecutive rows: 16 distinct bank groups); the P.V MFMAs read 64 contiguous bytes
// of 4 consecutive rows through the transposing read (the four rows differ in bits 2-3 of swz:
// 4 x 64 B cover all banks).  Both patterns are conflict-free; a plain padded stride can only
// satisfy one of them.  The 64 RoPE columns (8 chunks) of rows 2p, 2p+1 share the 256 bytes at
// kRopeBase + p * 256: chunk c of row r sits at slot ((r & 1) << 3) | (c ^ (p & 7)), which spreads
// one chunk column of 16 consecutive rows over all banks as well.
constexpr int kMainStride = 1024;
constexpr int kRopeBase = kTN * kMainStride;          // 32768
constexpr int kTileBytes = kRopeBase + kTN * 128;     // 36864
__host__ __device__ constexpr int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }
constexpr int kPStride = 80;                  // bytes per head row of a P buffer: 32 bf16 + 16 B pad (conflict-free)
constexpr int kPBytes = 32 * kPStride;        // one head group's probabilities for one tile
constexpr int kChunk = 1024;                  // top-k entries compacted into LDS at a time
constexpr int kDvHalf = kDv / 2;              // 256 output columns per wavefront
constexpr int kAccTiles = kDvHalf / 32;       // 8 accumulator tiles of 32 heads x 32 dv
constexpr int kBtLdsMax = 8192;               // page-table entries that fit the staging area (32 KB of a ring slot)
constexpr int kDmaSteps = 9;                  // DMA instructions per wavefront per tile (8 rows + 1 RoPE block)

using hw::lds_read_b128;
__device__ __forceinline__ bf16x4 lds_read_tr(uint32_t a) { return hw::lds_read_tr16_b64(a); }

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

// ---- tile movers ---------------------------------------------------------------------------
// bf16 rows go global -> LDS directly (no staging registers): a wave-wide 16-byte load writes
// the wave's 64 chunks to 1 KB of consecutive LDS starting at M0.  One such load moves the first
// 1 KB of a row (scalar row base + a per-lane chunk offset; lane l fetches chunk l ^ swz(row) so
// the row lands swizzled), and one more moves the remaining 128 bytes of eight rows.  Issued from
// inline asm so the compiler does not order them against LDS reads of other slots; the consumer
// counts them with s_waitcnt vmcnt before the barrier.  Rows past the valid count repeat the last
// valid row (their scores are masked, their probabilities are exactly zero).
struct DmaTile {
  const uint8_t* kv;
  uint32_t tile_lds, voff;
  int32_t rid;
  int wave, lane;
  __device__ __forceinline__ void begin(const uint8_t* kv_, const int32_t* rows, int e0, int n_valid,
                                        uint32_t tile_lds_, int wave_, int lane_) {
    kv = kv_; tile_lds = tile_lds_; wave = wave_; lane = lane_;
    rid = rows[min(e0 + (lane & 31), n_valid - 1)];               // lane l holds the row id of tile row l % 32
    voff = lane * 16;
  }
  // step j = 0..7: first 1 KB of this wave's j-th row (tile row 8 * wave + j); j = 8: RoPE tails of its 8 rows
  __device__ __forceinline__ void step(int j) const {
    if (j < 8) {
      const int r = 8 * wave + j;
      const uint32_t srow = (uint32_t)__builtin_amdgcn_readlane(rid, r);
      const uint64_t sbase = (uint64_t)(uintptr_t)kv + (uint64_t)srow * kRowBytesBf16;
      const uint32_t m0v = tile_lds + r * kMainStride;
      const uint32_t vsw = voff ^ (uint32_t)(swz(r) << 4);
      hw::dma_b128(vsw, sbase, m0v);
    } else {
      // lane l fills slot l of the 1 KB block of pairs 4*wave .. 4*wave+3
      const int pair = 4 * wave + (lane >> 4);
      const int r = 2 * pair + ((lane >> 3) & 1), c = (lane & 7) ^ (pair & 7);
      const int32_t trow = __shfl(rid, r);
      const uint8_t* src = kv + (size_t)trow * kRowBytesBf16 + 1024 + c * 16;
      const uint32_t m0v = tile_lds + kRopeBase + wave * 1024;
      hw::dma_b128(src, m0v);
    }
  }
};

__device__ __forceinline__ uint32_t rope_slot(int r, int c) {     // byte offset of RoPE chunk c of tile row r in a tile's RoPE block
  const int p = r >> 1;
  return p * 256 + ((((r & 1) << 3) | (c ^ (p & 7))) << 4);
}

// fp8 records: raw records -> LDS by moves, LDS -> LDS conversion (smla_fp8_pipe.h).  This kernel's
// row xor: swz(row0 + 2k) = swz(row0) ^ (8 * (k & 1) | (k >> 1)) for row0 = 8 * wave + l/32.
struct TallLayout {
  __device__ static constexpr int swz(int r) { return smla::swz(r); }
  __device__ static constexpr int store_xor(int k) { return (8 * (k & 1)) | (k >> 1); }
};
using Fp8Pipe = fp8pipe::Pipe;
using Fp8Convert = fp8pipe::Convert<TallLayout>;
static_assert(fp8pipe::kTN == kTN && fp8pipe::kMainStride == kMainStride && fp8pipe::kRopeBase == kRopeBase, "tile geometry");
static_assert(fp8pipe::layout_ok<TallLayout>(), "store_xor must describe this kernel's row xor");

// ---- per-tile math -------------------------------------------------------------------------
// Softmax reference handling.  The fast pass takes each head's maximum over the first tile as
// its reference and never moves it, so the accumulators are touched by MFMA only (they stay in
// AGPRs; no VALU rescale in the loop).  Probabilities may then exceed 1, by at most 2^kSlack.
// If some later score exceeds its head's reference by more than kSlack (log2 units) the pass is
// void and the workgroup redoes the split in two passes: exact per-head maximum first, then the
// accumulation against it.  Results do not depend on the reference (fp32 / bf16 keep their
// relative precision under scaling by powers of two).
constexpr float kSlack = 30.f;
enum { kPassFast = 0, kPassMax = 1, kPassFinal = 2 };

// One wavefront per SIMD means nothing hides LDS latency but the instruction stream itself, so
// both MFMA loops keep a few operand fragments in flight and pin the issue order with
// scheduling-group barriers.
constexpr int kPrefetchA = 5;                 // K fragments ahead in the score loop
constexpr int kPrefetchB = 6;                 // V fragments ahead in the P.V loop

// S^T = K_rows . Q^T : tile rows tok0 .. tok0+15 (body at `tile`, RoPE block at `rope`) against this wavefront's 32 heads (two head
// tiles of 16: heads 0..15 and 16..31 of the group).  Four independent accumulation chains
// (head tile x parity of the k-step) keep dependent MFMAs apart; sa[2*ht] + sa[2*ht+1] is the
// score block of head tile ht.  `side(ks)` is called once per k-step: the caller threads DMA
// issue through the MFMA stream.
template <typename Side>
__device__ __forceinline__ void tile_scores(uint32_t tile, uint32_t rope, int tok0, const bf16x8 (&qf)[kDqk / 32][2],
                                            f32x4 (&sa)[4], int lane, Side side) {
  constexpr int kSteps = kDqk / 32, kMainSteps = kDv / 32;     // 18 k-steps of 32, 16 of them in the NoPE part
  const int t = tok0 + (lane & 15), q4 = lane >> 4;
  // chunk 4*ks + q4 of row t sits at ((4*ks + q4) ^ swz(t)) * 16: the low byte of the row address
  // carries (q4 ^ swz(t)) * 16 and each k-step xors in its own (4 * (ks % 4)) * 16
  const uint32_t kmain = tile + t * kMainStride + ((q4 ^ swz(t)) << 4);
  auto frag = [&](int ks) {
    if (ks < kMainSteps) return lds_read_b128((kmain ^ (uint32_t)((ks & 3) << 6)) + (ks >> 2) * 256);
    return lds_read_b128(rope + rope_slot(t, 4 * (ks - kMainSteps) + q4));
  };
#pragma unroll
  for (int i = 0; i < 4; ++i) sa[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  __builtin_amdgcn_sched_barrier(0);
  bf16x8 a[kSteps];
#pragma unroll
  for (int ks = 0; ks < kPrefetchA; ++ks) a[ks] = frag(ks);
#pragma unroll
  for (int ks = 0; ks < kSteps; ++ks) {
    if (ks + kPrefetchA < kSteps) a[ks + kPrefetchA] = frag(ks + kPrefetchA);
    sa[ks & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ks], qf[ks][0], sa[ks & 1], 0, 0, 0);
    sa[2 + (ks & 1)] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ks], qf[ks][1], sa[2 + (ks & 1)], 0, 0, 0);
    side(ks);
  }
#pragma unroll
  for (int ks = 0; ks < kPrefetchA; ++ks) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // DS read
#pragma unroll
  for (int ks = 0; ks < kSteps; ++ks) {
    if (ks + kPrefetchA < kSteps) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);                                         // MFMA
  }
  __builtin_amdgcn_sched_barrier(0);
}

// O[32 heads x 256 dv] += P[32 heads x 32 tok] . V[32 tok x 256 dv] over one tile.  O tiles are
// [32 heads x 32 dv]: lane owns dv column lane%32, register r is head row 8*(r/4) + 4*(lane/32) + r%4.
// P comes from LDS ([head][token] bf16, kPStride bytes per head): lane reads its head's tokens
// 16*s2 + 8*(lane/32) .. +7; the B operand is gathered in the same token order.
// `valu(i)` is independent vector-ALU work of the caller (a slice of the softmax of the next tile).
// With kPinValu it is pinned between MFMA i and MFMA i+1 by scheduling barriers, so it issues
// while the matrix core is busy with MFMA i; the LDS reads then simply stay in source order
// (they are written kAhead steps ahead of their use).
template <bool kPinValu, int kAhead = kPrefetchB, typename Side, typename Valu>
__device__ __forceinline__ void tile_accumulate(uint32_t tile, uint32_t pbuf, int dv0, f32x16 (&acc)[kAccTiles],
                                                int lane, Side side, Valu valu) {
  constexpr int kSteps = 2 * kAccTiles;
  const int g = lane >> 5, l16 = lane & 15, i4 = l16 >> 2;
  // A lane reads 8 bytes of row 16*s2 + 8*g + 4*h + i4 (h = 0 low / 1 high half of its 8 tokens;
  // swz(row) = (i4 << 2) | (2*g + h)) at logical byte column dv0*2 + 64*dt + 32*((lane>>4)&1) + 8*(l16&3),
  // i.e. chunk dv0/8 + 4*dt + c_lane, c_lane = 2*((lane>>4)&1) + ((l16&3)>>1), byte 8*(l16&1) in it.
  // Physical chunk = (dv0/8) + ((4*dt) ^ (i4<<2)) + (c_lane ^ (2*g + h)): per lane one base address,
  // per (dt, h) one xor with the constant 64*dt ^ 16*h (bits 4 and 6..8 only; no carries).
  const int c_lane = 2 * ((lane >> 4) & 1) + ((l16 & 3) >> 1);
  const uint32_t vbase = tile + (8 * g + i4) * kMainStride + dv0 * 2 + (i4 << 6) + ((c_lane ^ (2 * g)) << 4) + 8 * (l16 & 1);
  const uint32_t prow = pbuf + (lane & 31) * kPStride + 16 * g;
  __builtin_amdgcn_sched_barrier(0);
  bf16x8 pa[2];
  pa[0] = lds_read_b128(prow);
  pa[1] = lds_read_b128(prow + 32);
  bf16x4 lo[kSteps], hi[kSteps];
  auto load = [&](int i) {                   // step i = (s2, dt) with dt fastest
    const int s2 = i / kAccTiles, dt = i % kAccTiles;
    lo[i] = lds_read_tr((vbase ^ (uint32_t)(64 * dt)) + 16 * s2 * kMainStride);
    hi[i] = lds_read_tr((vbase ^ (uint32_t)(64 * dt + 16)) + (16 * s2 + 4) * kMainStride);
  };
#pragma unroll
  for (int i = 0; i < kAhead; ++i) load(i);
#pragma unroll
  for (int i = 0; i < kSteps; ++i) {
    if (i + kAhead < kSteps) load(i + kAhead);
    const bf16x8 bv = __builtin_shufflevector(lo[i], hi[i], 0, 1, 2, 3, 4, 5, 6, 7);
    acc[i % kAccTiles] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa[i / kAccTiles], bv, acc[i % kAccTiles], 0, 0, 0);
    side(i);
    if constexpr (kPinValu) {
      __builtin_amdgcn_sched_barrier(0);
      valu(i);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if constexpr (!kPinValu) {
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int i = 0; i < kAhead; ++i) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
      if (i + kAhead < kSteps) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
}

// s_waitcnt vmcnt(n) for a run-time n in {0, kDmaSteps, 2 * kDmaSteps}
__device__ __forceinline__ void wait_dma(int younger_tiles) {
  if (younger_tiles >= 2) hw::wait_vmcnt<2 * kDmaSteps>();
  else if (younger_tiles == 1) hw::wait_vmcnt<kDmaSteps>();
  else hw::wait_vmcnt<0>();
}

// PERSIST (launches that do not split, with several items per compute unit: prefill, dense decode
// over many tokens): one workgroup per compute unit walks the block ids b, b + gridDim.x, ... of
// the one-workgroup-per-item launch (gridDim.x a multiple of 8: all on its own XCD).  The next
// item's index and Q loads go out when the current item's accumulators have been parked for the
// epilogue, which frees the registers they land in, and its page-table look-ups follow the
// epilogue's stores: the three dependent round trips that open an item (indices, page table,
// first rows) shrink to the last one.
template <int FMT, bool CAP, bool PERSIST = false>
__global__ __launch_bounds__(kNT) void fwd_tall_kernel(Params p, int n_hblocks, int n_items) {
  // the ring area: bf16 has four whole tiles (body + RoPE block each); fp8 see Fp8Pipe
  constexpr bool kFp8 = FMT == SMLA_KV_FP8_B128;
  constexpr int kRingBytes = kFp8 ? Fp8Pipe::kRingBytes : kSlots * kTileBytes;
  __shared__ __attribute__((aligned(1024))) uint8_t s_ring[kRingBytes];           // swizzle xors need 1 KB alignment
  __shared__ __attribute__((aligned(16))) uint8_t s_p[2][2][kPBytes];             // [tile parity][head group]
  __shared__ int32_t s_rows[kChunk];
  __shared__ float s_x[4][32];                                    // per-head scalars exchanged inside a pair
  __shared__ float s_m[4][32];
  __shared__ int s_nvalid;
  __shared__ int s_cnt[4];
  __shared__ int s_redo;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c32 = lane & 31, l16 = lane & 15, q4 = lane >> 4;
  const int hg = wave >> 1, dh = wave & 1;

  // block id -> (token, split, head block).  Ids are dealt round-robin to the 8 XCDs, so all
  // workgroups of one token (they gather overlapping rows and later merge) get ids 8 apart.
  auto token_of_id = [&](int id) { return token_of(p, id & 7, (id >> 3) / (n_hblocks * p.n_splits)); };
  auto next_item = [&](int id) {               // the next id of this workgroup that has a token (token counts are rounded up to 8 an XCD round)
    while (id < n_items && token_of_id(id) >= p.n_tokens) id += (int)gridDim.x;
    return id;
  };
  int item = PERSIST ? next_item((int)blockIdx.x) : (int)blockIdx.x;
  if (PERSIST && item >= n_items) return;
  int hb, sp, t, seq, head0, head;
  bool head_ok;
  auto place = [&](int id) {
    const int slot = id >> 3;
    hb = slot % n_hblocks;
    sp = (slot / n_hblocks) % p.n_splits;
    t = token_of_id(id);
    seq = t / p.tokens_per_seq;
    head0 = hb * 64 + hg * 32;
    head = head0 + c32;
    head_ok = head < p.n_heads;
  };
  place(item);
  if (t >= p.n_tokens) return;
  const uint8_t* kv = static_cast<const uint8_t*>(p.kv);
  const int k_begin = sp * p.split_len, k_end = min(k_begin + p.split_len, p.topk);
  const WsHead ws_head = ws_read_head(p);    // read long before the split merge needs it

  // ---- the first chunk's index loads go out before anything else: the row list they lead to
  // (index -> page table -> row fetch) is the longest dependent chain of the kernel
  auto load_indices_of = [&](int tt, int sseq, int c0, int32_t (&rr)[4]) {
    const int c1 = min(c0 + kChunk, k_end);
    // (branch-free: with an index list every lane loads its entry, without one it loads the
    // sequence length instead; a branch per entry or per mode would make the compiler wait for
    // each load where the branches join, ahead of the Q loads that should overlap them)
    const bool listed = p.indices != nullptr;
    const int32_t* base = listed ? p.indices + (size_t)tt * p.topk : p.seq_lens + sseq;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int j = c0 + 256 * wave + 64 * k + lane;
      const int32_t v = base[listed ? min(j, c1 - 1) : 0];
      rr[k] = j < c1 ? (listed ? v : (j < v ? j : -1)) : -1;
    }
  };
  auto load_indices = [&](int c0, int32_t (&rr)[4]) { load_indices_of(t, seq, c0, rr); };
  auto translate_entries = [&](int32_t (&rr)[4]) { translate_entries4(p, seq, rr); };
  // ---- this sequence's page-table row goes global -> LDS (into the last tile body, which stays free
  // until the first chunk's row list exists) while the indices and Q are on their way, so the
  // first chunk's translation reads LDS instead of paying a second dependent trip to memory.
  // It is issued ahead of the index loads: memory operations complete in order, so once a
  // wavefront holds its index values its part of the row has landed too.
  // Needs a 16-byte aligned row of at most kBtLdsMax entries; otherwise the lookups go to memory.
  const int32_t* bt_row = p.block_table ? p.block_table + (size_t)seq * p.bt_stride : nullptr;
  const bool bt_in_lds = bt_row != nullptr && p.bt_stride <= kBtLdsMax && (p.bt_stride & 3) == 0 &&
                         ((uintptr_t)bt_row & 15) == 0;
  uint8_t* const bt_stage = &s_ring[kFp8 ? (Fp8Pipe::kBodies - 1) * kRopeBase : (kSlots - 1) * kTileBytes];
  const uint32_t lds_bt = hw::lds_addr(bt_stage);
  if (bt_in_lds) {
    for (int c = wave; 256 * c < p.bt_stride; c += 4) {            // 1 KB (256 entries) per instruction
      const int e = 256 * c + 4 * lane;
      const uint32_t m0v = lds_bt + 1024 * c;
      if (e < p.bt_stride)
        hw::dma_b128(bt_row + e, m0v);
    }
  }

  int32_t rr_first[4];
  load_indices(k_begin, rr_first);        // the Q loads below are issued while these are in flight

  // ---- Q^T fragments for this wavefront's 32 heads: B operand of S^T; lane holds head 16*ht + lane%16,
  // k = 32*ks + 8*(lane/16) .. +7
  bf16x8 qf[kDqk / 32][2];
  auto load_q = [&](int tt, int hhead0) {
#pragma unroll
    for (int ht = 0; ht < 2; ++ht) {
      const int hq = hhead0 + 16 * ht + l16;
      // Every lane loads; a head past the end reads head 0 again (its results are never stored).
      // Nothing touches the values here: whatever consumed them (a mask, say) would make the
      // compiler wait for Q ahead of the row list, which only needs the index values.
      const uint16_t* qrow = static_cast<const uint16_t*>(p.q) + ((size_t)tt * p.n_heads + (hq < p.n_heads ? hq : 0)) * kDqk + 8 * q4;
#pragma unroll
      for (int ks = 0; ks < kDqk / 32; ++ks) qf[ks][ht] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
    }
  };
  load_q(t, head0);
  if (tid == 0) s_redo = 0;
  if (bt_in_lds) {
    // Touching the index values makes the compiler wait for exactly those loads (the Q loads
    // issued behind them stay in flight); the page-table DMA is older, so it is complete as well.
    hw::wait_for_loads_of(rr_first[0], rr_first[1], rr_first[2], rr_first[3]);
    __syncthreads();
    const int32_t* bt_s = reinterpret_cast<const int32_t*>(bt_stage);
#pragma unroll
    for (int k = 0; k < 4; ++k) rr_first[k] = translate_index(p, rr_first[k], bt_s);
  } else {
    translate_entries(rr_first);          // waits for the indices only; the page-table lookups overlap the Q loads
  }

  // raw dot product -> base-2 exponent: one multiply, or (logit cap) the squashed score, which
  // already is in base-2 units
  const float sc2 = CAP ? 1.f : p.sm_scale * kLog2e;
  [[maybe_unused]] const LogitCap cap(p.sm_scale, CAP ? p.logit_cap : 1.f);
  const uint32_t lds_tile = hw::lds_addr(&s_ring[0]);
  const uint32_t lds_p = hw::lds_addr(&s_p[0][0][0]);
  const int partner = wave ^ 1;

  for (;;) {       // one item a turn (a single turn unless PERSIST)
  f32x16 acc[kAccTiles];
#pragma unroll
  for (int i = 0; i < kAccTiles; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  // softmax state of heads 16*ht + lane%16 (ht = 0, 1): base-2 reference (common to the pair of
  // wavefronts) and this lane's partial sum over its tokens
  float m_ref[2] = {-INFINITY, -INFINITY}, l_part[2] = {0.f, 0.f};

  int pass = kPassFast;
  bool first_chunk = true;
  for (;;) {
    bool failed = false;
    bool have_ref = pass == kPassFinal;
    for (int c0 = k_begin; c0 < k_end; c0 += kChunk) {
      // ---- translate + mask + compact the next chunk of the top-k list (order preserving).
      // All four wavefronts take 256 consecutive entries each; every lane issues its four index
      // loads (and page-table lookups) back to back so the chunk costs two memory latencies.
      __syncthreads();                       // previous chunk's rows and tiles are no longer read
      {
        int32_t rr[4];
        if (first_chunk) {
#pragma unroll
          for (int k = 0; k < 4; ++k) rr[k] = rr_first[k];
        } else {
          load_indices(c0, rr);
          translate_entries(rr);
        }
        first_chunk = false;
        uint64_t mk[4];
        int cnt = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          mk[k] = __ballot(rr[k] >= 0);
          cnt += __popcll(mk[k]);
        }
        if (lane == 0) s_cnt[wave] = cnt;
        __syncthreads();
        int base = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) base += w < wave ? s_cnt[w] : 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (rr[k] >= 0) s_rows[base + __popcll(mk[k] & ((1ull << lane) - 1ull))] = rr[k];
          base += __popcll(mk[k]);
        }
        if (tid == 0) s_nvalid = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
      }
      __syncthreads();
      const int n_valid = s_nvalid;
      const int n_tiles = (n_valid + kTN - 1) / kTN;
      if (n_tiles == 0) continue;

      // ---- tile movers.  bf16: tile `it` lives in ring slot it % kSlots.  fp8: its body in
      // body it % 3, its RoPE block in block it % 3, its raw records in raw block it % 2.
      [[maybe_unused]] Fp8Pipe pipe;
      [[maybe_unused]] Fp8Convert cv;
      DmaTile dma;
      // (fp8: the ring's address is taken afresh for every chunk, so that the per-lane addresses
      // of the first tiles are worked out here rather than once at the top of the kernel and
      // then kept in registers, which that variant does not have to spare)
      uint32_t ring = lds_tile;
      if constexpr (kFp8) hw::pin_uniform(ring);
      auto tile_addr = [&](int it) {
        if constexpr (kFp8) return ring + (uint32_t)(it % Fp8Pipe::kBodies) * kRopeBase;
        else return ring + (it & (kSlots - 1)) * kTileBytes;
      };
      auto rope_addr = [&](int it) {
        if constexpr (kFp8) return ring + Fp8Pipe::kRopeRing + (uint32_t)(it % Fp8Pipe::kRopes) * (kTN * 128);
        else return ring + (it & (kSlots - 1)) * kTileBytes + kRopeBase;
      };
      [[maybe_unused]] auto pipe_begin = [&](int it) {
        pipe.begin(kv, s_rows, it * kTN, n_valid,
                   ring + Fp8Pipe::kRawRing + (it & 1) * Fp8Pipe::kRawSlot + wave * Fp8Pipe::kRawWave, rope_addr(it), wave, lane);
      };
      [[maybe_unused]] auto convert_begin = [&](int it) {
        cv.raw_lds = ring + Fp8Pipe::kRawRing + (it & 1) * Fp8Pipe::kRawSlot + wave * Fp8Pipe::kRawWave;
        cv.body_lds = ring + (uint32_t)(it % Fp8Pipe::kBodies) * kRopeBase;
        cv.wave = wave; cv.lane = lane;
      };
      auto fetch_whole = [&](int it) {       // all moves of a tile at once (prologue)
        if constexpr (!kFp8) {
          dma.begin(kv, s_rows, it * kTN, n_valid, tile_addr(it), wave, lane);
#pragma unroll
          for (int j = 0; j < kDmaSteps; ++j) dma.step(j);
        } else {
          pipe_begin(it);
#pragma unroll
          for (int j = 0; j < Fp8Pipe::kSteps; ++j) pipe.step(j);
        }
      };
      // scores + probabilities of tile `it` into P buffer it & 1; `side` threads DMA issue
      auto score_tile = [&](int it, auto side) {
        const uint32_t tile = tile_addr(it);
        const int my_valid = min(kTN, n_valid - it * kTN) - 16 * dh;   // valid tokens among my 16
        f32x4 sa[4], s[2];
        tile_scores(tile, rope_addr(it), 16 * dh, qf, sa, lane, side);
        s[0] = sa[0] + sa[1];
        s[1] = sa[2] + sa[3];
        if constexpr (CAP) {
#pragma unroll
          for (int r = 0; r < 4; ++r) { s[0][r] = cap(s[0][r]); s[1][r] = cap(s[1][r]); }
        }
        if (my_valid < 16) {                 // ragged tile (uniform): mask the rows past the end
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (4 * q4 + r >= my_valid) { s[0][r] = -INFINITY; s[1][r] = -INFINITY; }
        }
        float mx[2];
#pragma unroll
        for (int ht = 0; ht < 2; ++ht) {
          float v = fmaxf(fmaxf(s[ht][0], s[ht][1]), fmaxf(s[ht][2], s[ht][3]));
          v = fmaxf(v, __shfl_xor(v, 16));
          v = fmaxf(v, __shfl_xor(v, 32));
          mx[ht] = v * sc2;                  // sc2 > 0: scaling commutes with the maximum
        }
        if (!have_ref) {                     // first tile of the pass (uniform): agree on the pair's reference
          if (pass == kPassFast) {
            if (q4 == 0) { s_x[wave][l16] = mx[0]; s_x[wave][16 + l16] = mx[1]; }
            __syncthreads();
            m_ref[0] = fmaxf(mx[0], s_x[partner][l16]);
            m_ref[1] = fmaxf(mx[1], s_x[partner][16 + l16]);
          }
          have_ref = true;
        }
        if (pass == kPassMax) { m_ref[0] = fmaxf(m_ref[0], mx[0]); m_ref[1] = fmaxf(m_ref[1], mx[1]); }
        if (pass == kPassFast) failed |= __any(mx[0] > m_ref[0] + kSlack || mx[1] > m_ref[1] + kSlack);
        // probabilities of my 4 tokens for my 2 heads -> P[head][token] of this tile
        const uint32_t pw = lds_p + ((it & 1) * 2 + hg) * kPBytes + l16 * kPStride + (16 * dh + 4 * q4) * 2;
#pragma unroll
        for (int ht = 0; ht < 2; ++ht) {
          float pr[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) pr[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[ht][r], sc2, -m_ref[ht]));
          l_part[ht] += (pr[0] + pr[1]) + (pr[2] + pr[3]);
          const u32x2 w = {pack_bf16(pr[0], pr[1]), pack_bf16(pr[2], pr[3])};
          hw::lds_write_b64(pw + 16 * ht * kPStride, w);
        }
      };

      // ---- prologue: tiles 0 and 1 go out at once, tile 2 rides on the scores of tile 0
      // The moves go out as soon as the row list exists; Q may still be on its way.  Loads
      // complete in issue order, so waiting for the moves below also waits for everything older.
      for (int it = 0; it < min(n_tiles, 2); ++it) fetch_whole(it);
      if constexpr (!kFp8) {
        wait_dma(n_tiles > 1 ? 1 : 0);
      } else {
        // fp8: convert tile 0, send for tile 2 (its raw block is free again), convert tile 1
        // (a wavefront's lanes read raw chunks that other lanes of it fetched: wave_lds_order)
        if (n_tiles > 1) hw::wait_vmcnt<Fp8Pipe::kSteps>(); else hw::wait_vmcnt<0>();
        hw::wave_lds_order();
        convert_begin(0);
        cv.whole_tile();
        if (n_tiles > 2) fetch_whole(2);
        if (n_tiles > 1) {
          if (n_tiles > 2) hw::wait_vmcnt<Fp8Pipe::kSteps>(); else hw::wait_vmcnt<0>();
          hw::wave_lds_order();
          convert_begin(1);
          cv.whole_tile();
        }
      }
      // Tell the compiler that Q has arrived (it cannot see the waits above): otherwise it would
      // wait for Q inside the first tile's MFMA stream, and with it for the moves issued there.
#pragma unroll
      for (int ks = 0; ks < kDqk / 32; ++ks) hw::wait_for_loads_of(qf[ks][0], qf[ks][1]);
      __syncthreads();                       // tile 0 landed
      if (!kFp8 && n_tiles > 2) {
        dma.begin(kv, s_rows, 2 * kTN, n_valid, tile_addr(2), wave, lane);
        score_tile(0, [&](int ks) { if ((ks & 1) == 0) dma.step(ks >> 1); });
      } else {
        score_tile(0, [](int) {});
      }

      // ---- main loop: iterations that still have a tile to fetch (it + 3 < n_tiles, so tiles it+1
      // and it+2 exist).  The fetch of tile it+3 rides on the score MFMAs of tile it+1, one move
      // instruction every second k-step: early in the iteration (the data has the longest way
      // to go) but spaced out (measured: bursts and later issue are both slower).  Main loop and
      // tail are separate loops, each with one call site per MFMA block, so the accumulators
      // stay in place.
      // fp8: the raw records of tile it+2 (sent for one iteration ago) are converted into the
      // body that tile it-1 has left, in 16 slices under the P.V MFMAs of tile it.
      const int n_main = max(n_tiles - (kSlots - 1), 0);
      int it = 0;
      for (; it < n_main; ++it) {
        // bf16: tile it+1 was issued two iterations ago; only tile it+2 is still outstanding
        if constexpr (!kFp8) wait_dma(1);
        __syncthreads();                     // P of tile `it` is published, tile it+1 landed / converted, tile it-1 is consumed
        if constexpr (!kFp8) {
          dma.begin(kv, s_rows, (it + kSlots - 1) * kTN, n_valid, tile_addr(it + kSlots - 1), wave, lane);
        } else {
          pipe_begin(it + 3);
          convert_begin(it + 2);
        }
        // Tile it+1 is never the last one here, so it is full: no masking, and the reference is
        // fixed, so the softmax is straight-line vector code that is scheduled under the P.V MFMAs.
        f32x4 sa[4];
        tile_scores(tile_addr(it + 1), rope_addr(it + 1), 16 * dh, qf, sa, lane, [&](int ks) {
          if ((ks & 1) == 0) {
            if constexpr (!kFp8) dma.step(ks >> 1);
            else if ((ks >> 1) < Fp8Pipe::kSteps) pipe.step(ks >> 1);
          }
        });
        // softmax of tile it+1 in 16 slices, one after each P.V MFMA of tile it
        f32x4 sv[2];
        float pr[2][4];
        u32x2 pw2[2];
        bool over = false;
        tile_accumulate<true>(tile_addr(it), lds_p + ((it & 1) * 2 + hg) * kPBytes, kDvHalf * dh, acc, lane,
                              [](int) {},
                              [&](int i) {
          if constexpr (kFp8) {
            // chunk k = i / 4 of the conversion: its two halves, its stores, and the next chunk's
            // read three slices ahead of its first use.  The moves of tile it+3, just issued,
            // stay in flight; everything older has landed after the wait.
            if (i == 0) { hw::wait_vmcnt<Fp8Pipe::kSteps>(); hw::wave_lds_order(); cv.load(0); }
            else if ((i & 3) == 1) cv.half(0);
            else if ((i & 3) == 2) cv.half(1);
            else if ((i & 3) == 3) { cv.store(i >> 2); if (i < 15) cv.load((i >> 2) + 1); }
          }
          if (i < 2) {                       // slices 0, 1: score block, per-lane maximum, reference of head tile i
            // (per-lane maximum only: the overflow test does not need the row maximum, and a
            // maximum pass folds the lanes of a head together when it ends)
            sv[i] = sa[2 * i] + sa[2 * i + 1];
            if constexpr (CAP) {
#pragma unroll
              for (int r = 0; r < 4; ++r) sv[i][r] = cap(sv[i][r]);
            }
            const float lm = fmaxf(fmaxf(sv[i][0], sv[i][1]), fmaxf(sv[i][2], sv[i][3])) * sc2;
            m_ref[i] = pass == kPassMax ? fmaxf(m_ref[i], lm) : m_ref[i];
            over |= lm > m_ref[i] + kSlack;
            hw::pin(m_ref[i]);                     // keeps the slice where it is written
          } else if (i < 10) {               // slices 2..9: one probability each
            const int ht = (i - 2) >> 2, r = (i - 2) & 3;
            pr[ht][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[ht][r], sc2, -m_ref[ht]));
            hw::pin(pr[ht][r]);
          } else if (i < 12) {               // slices 10, 11: row sums and bf16 packing
            const int ht = i - 10;
            l_part[ht] += (pr[ht][0] + pr[ht][1]) + (pr[ht][2] + pr[ht][3]);
            pw2[ht] = u32x2{pack_bf16(pr[ht][0], pr[ht][1]), pack_bf16(pr[ht][2], pr[ht][3])};
            hw::pin(l_part[ht], pw2[ht]);
          } else if (i == 12) {
            failed |= pass == kPassFast && __any(over);
          }
        });
        const uint32_t pw = lds_p + (((it + 1) & 1) * 2 + hg) * kPBytes + l16 * kPStride + (16 * dh + 4 * q4) * 2;
        hw::lds_write_b64(pw, pw2[0]);
        hw::lds_write_b64(pw + 16 * kPStride, pw2[1]);
      }
      // ---- tail: the last tiles, nothing left to fetch (fp8: tile it+2 may still await its conversion)
      for (; it < n_tiles; ++it) {
        const bool next = it + 1 < n_tiles;
        if constexpr (!kFp8) { if (next) wait_dma(it + 2 < n_tiles ? 1 : 0); }
        __syncthreads();
        if constexpr (kFp8) {
          if (it + 2 < n_tiles) {
            hw::wait_vmcnt<0>();
            hw::wave_lds_order();
            convert_begin(it + 2);
            cv.whole_tile();
          }
        }
        if (next) score_tile(it + 1, [](int) {});
        tile_accumulate<false>(tile_addr(it), lds_p + ((it & 1) * 2 + hg) * kPBytes, kDvHalf * dh, acc, lane, [](int) {}, [](int) {});
      }
    }
    if (pass == kPassFinal) break;
    if (pass == kPassFast) {
      if (failed && lane == 0) s_redo = 1;
      __syncthreads();
      if (s_redo == 0) break;                // the common case
      m_ref[0] = -INFINITY; m_ref[1] = -INFINITY;
      pass = kPassMax;
    } else {                                 // exact maxima: fold a head's lanes, combine the pair's halves, then accumulate for real
#pragma unroll
      for (int ht = 0; ht < 2; ++ht) {
        m_ref[ht] = fmaxf(m_ref[ht], __shfl_xor(m_ref[ht], 16));
        m_ref[ht] = fmaxf(m_ref[ht], __shfl_xor(m_ref[ht], 32));
      }
      __syncthreads();
      if (q4 == 0) { s_x[wave][l16] = m_ref[0]; s_x[wave][16 + l16] = m_ref[1]; }
      __syncthreads();
      m_ref[0] = fmaxf(m_ref[0], s_x[partner][l16]);
      m_ref[1] = fmaxf(m_ref[1], s_x[partner][16 + l16]);
      pass = kPassFinal;
    }
    l_part[0] = 0.f; l_part[1] = 0.f;        // what the void / max pass accumulated is dropped
#pragma unroll
    for (int i = 0; i < kAccTiles; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  }

  // ---- epilogue.  Bring the per-head scalars from the score layout (lane % 16 = head in tile)
  // to lane = head, then: accumulator registers hold (head row, dv column = lane).  Each
  // wavefront parks its 32 x 256 block in LDS (the ring is free now) and reads it back one head
  // row at a time, 4 consecutive dv columns per lane, so everything below moves 16 bytes per
  // lane in 1 KB runs and per-row scalars are wave-uniform.
  __syncthreads();
  // The lane's coordinates are taken afresh here: derived from the hardware's lane counter, they
  // need not be carried through the main loop in registers (or parked in scratch) for this use.
  const int lane_e = hw::lane_id(), tid_e = 64 * wave + lane_e;
  const int g_e = lane_e >> 5, c32_e = lane_e & 31, l16_e = lane_e & 15, q4_e = lane_e >> 4;
  const int head_e = head0 + c32_e;
  const bool head_ok_e = head_e < p.n_heads;
  // the arrival ticket of the split merge is taken here, so that its round trip to memory
  // overlaps the staging below (the merge itself is described further down)
  if (p.n_splits > 1 && tid_e == 0)
    s_nvalid = ws_arrive(p, p.counters + (size_t)t * n_hblocks + hb, ws_head, p.n_splits, sp);
#pragma unroll
  for (int ht = 0; ht < 2; ++ht) {
    float l = l_part[ht];
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (q4_e == 0) { s_x[wave][16 * ht + l16_e] = l; s_m[wave][16 * ht + l16_e] = m_ref[ht]; }
  }
  __syncthreads();
  const float m_run = s_m[wave][c32_e];
  const float l_tot = s_x[wave][c32_e] + s_x[partner][c32_e];
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  const float lse_nat = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
  constexpr int kStageStride = kDvHalf + 8;                        // floats per staged row (+32 B pad: a store's two half-wavefronts write rows 4 apart, which then land 32 banks apart)
  static_assert(4 * 32 * kStageStride * 4 <= kRingBytes, "the staged blocks must fit the ring area");
  float* stage = reinterpret_cast<float*>(&s_ring[0]) + wave * 32 * kStageStride;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = 8 * (r >> 2) + 4 * g_e + (r & 3);
#pragma unroll
    for (int dt = 0; dt < kAccTiles; ++dt) stage[row * kStageStride + 32 * dt + c32_e] = acc[dt][r];
  }
  __syncthreads();                                                 // staged blocks and scalar exchange are done
  // PERSIST: the accumulators are parked and Q has done its work, so the registers the next
  // item's index values and Q fragments land in are free: send for them now, ahead of this
  // item's stores.  (Nothing reads them before the stores below have been issued.)
  [[maybe_unused]] int item_next = 0;
  if constexpr (PERSIST) {
    item_next = next_item(item + (int)gridDim.x);
    if (item_next < n_items) {
      const int slot_n = item_next >> 3, t_n = token_of_id(item_next);
      load_indices_of(t_n, t_n / p.tokens_per_seq, k_begin, rr_first);
      load_q(t_n, (slot_n % n_hblocks) * 64 + hg * 32);
      if (tid_e == 0) s_redo = 0;
    }
  }
  if (g_e == 0) s_x[wave][c32_e] = inv;                                // per-row normaliser
  hw::wave_lds_order();
  const int n_rows = max(0, min(32, p.n_heads - head0));           // head rows that exist (wave-uniform; 0: the whole head group lies past the last head)
  const int col4 = kDvHalf * dh + 4 * lane_e;                        // this lane's 4 dv columns
  auto staged = [&](int row) { return *reinterpret_cast<const float4*>(stage + row * kStageStride + 4 * lane_e); };
  auto store_bf16x4 = [&](int row, float4 v) {
    uint2 w;
    w.x = pack_bf16(v.x, v.y);
    w.y = pack_bf16(v.z, v.w);
    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + ((size_t)t * p.n_heads + head0 + row) * kDv + col4) = w;
  };
  if (PERSIST || p.n_splits == 1) {
    if (dh == 0 && g_e == 0 && head_ok_e) p.lse[(size_t)t * p.n_heads + head_e] = lse_nat;
    for (int row = 0; row < n_rows; ++row) {
      const float sc = s_x[wave][row];
      float4 v = staged(row);
      v.x *= sc; v.y *= sc; v.z *= sc; v.w *= sc;
      store_bf16x4(row, v);
    }
    if constexpr (PERSIST) {
      if (item_next >= n_items) return;
      item = item_next;
      place(item);                           // from here on t, seq, head0 ... are the next item's
      translate_entries(rr_first);           // waits for its index values only; page-table look-ups straight from memory
      continue;                              // (the barrier that opens its first chunk also ends everyone's reads of the parked blocks)
    } else {
      return;
    }
  }

  // ---- split merge inside the launch.  Every (token, head block) owns one 64-bit word:
  // high half = arrival tickets, low half = one "partial published" bit per split.  All but
  // the last workgroup to arrive publish their normalised partial and leave; the last one
  // waits for the published bits of the others (they hold a ticket, so they are running),
  // folds their partials into its own staged block and writes the final output.
  // Partials move between workgroups without fences: they are stored and loaded with the
  // sc1 (agent scope: write-through / read-through the L2) modifier, and a bit is published
  // only after the stores have been acknowledged.  A release / acquire fence pair would write
  // back and invalidate the whole L2 of the XCD instead.  A word that is not in a legal state,
  // or a wait that outlasts the workspace's poll limit, flags the workspace, marks the rows'
  // LSE with NaN and leaves (see ws_arrive / ws_wait_published).
  const int ns = p.n_splits;
  unsigned long long* word = p.counters + (size_t)t * n_hblocks + hb;
  const int role = s_nvalid;                                       // ticket taken at the top of the epilogue
  auto give_up = [&]() {                                           // the workspace was not what it should be: mark the rows (NaN LSE, zero output)
    if (dh == 0 && g_e == 0 && head_ok_e) p.lse[(size_t)t * p.n_heads + head_e] = __uint_as_float(0x7fc00000u);
    for (int row = 0; row < n_rows; ++row) store_bf16x4(row, make_float4(0.f, 0.f, 0.f, 0.f));
  };
  if (role == kRoleError) { give_up(); return; }
  if (role == kRolePublish) {
    if (dh == 0 && g_e == 0 && head_ok_e)
      __hip_atomic_store(&p.part_lse[((size_t)t * ns + sp) * p.n_heads + head_e], lse_nat, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    float* o = p.part_out + (((size_t)t * ns + sp) * p.n_heads + head0) * kDv + col4;
    for (int row = 0; row < n_rows; ++row) {
      const float sc = s_x[wave][row];
      const float4 v = staged(row);
      const f32x4 vv = {__fmul_rn(v.x, sc), __fmul_rn(v.y, sc), __fmul_rn(v.z, sc), __fmul_rn(v.w, sc)};
      hw::store_b128_agent(o + (size_t)row * kDv, vv);
    }
    hw::wait_vmcnt<0>();
    __syncthreads();
    if (tid_e == 0) ws_publish(p, word, sp);
    return;
  }
  // last arrival: every other split holds a ticket, so it is running and will publish.  Wait for
  // all of them, then fold the normalised partials in split order with every product and sum
  // rounded on its own (no fused multiply-add): the result does not depend on which split
  // happened to arrive last.  Per-head scalars live in lane = head row c32.
  if (tid_e == 0) s_redo = ws_wait_published(p, word, ns, sp) ? 0 : 1;
  __syncthreads();
  if (s_redo != 0) { give_up(); return; }
  auto split_lse = [&](int i) {
    if (i == sp) return lse_nat;
    return head_ok_e ? __hip_atomic_load(&p.part_lse[((size_t)t * ns + i) * p.n_heads + head_e], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT)
                   : -INFINITY;
  };
  float m_all = -INFINITY;
  for (int i = 0; i < ns; ++i) m_all = fmaxf(m_all, split_lse(i));
  const float m_safe = m_all == -INFINITY ? 0.f : m_all;
  float w_sum = 0.f;
  for (int i = 0; i < ns; ++i) w_sum = __fadd_rn(w_sum, __expf(split_lse(i) - m_safe));      // exp(-inf) = 0
  const float rw = w_sum > 0.f ? 1.f / w_sum : 0.f;
  if (dh == 0 && g_e == 0 && head_ok_e)
    p.lse[(size_t)t * p.n_heads + head_e] = w_sum > 0.f ? m_all + __logf(w_sum) : -INFINITY;
  // my own block becomes its normalised partial: the very numbers a publisher would have stored
  for (int row = 0; row < 32; ++row) {
    const float sc = s_x[wave][row];
    float4 v = staged(row);
    v.x = __fmul_rn(v.x, sc); v.y = __fmul_rn(v.y, sc); v.z = __fmul_rn(v.z, sc); v.w = __fmul_rn(v.w, sc);
    *reinterpret_cast<float4*>(stage + row * kStageStride + 4 * lane_e) = v;
  }
  float* s_w = s_m[wave];                                          // per-row weight of the split being folded
                                                                   // (written and read by this wavefront only: its LDS accesses complete in order)
#pragma unroll 1
  for (int r0 = 0; r0 < 32; r0 += 16) {                            // 16 rows per round: 16 loads in flight per lane
    f32x4 sum[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) sum[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
    for (int i = 0; i < ns; ++i) {
      const float wi = __fmul_rn(__expf(split_lse(i) - m_safe), rw);
      hw::wave_lds_order();
      if (g_e == 0) s_w[c32_e] = wi;
      hw::wave_lds_order();
      f32x4 v[16];
      if (i == sp) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const float4 a4 = staged(r0 + j);
          v[j] = f32x4{a4.x, a4.y, a4.z, a4.w};
        }
      } else if (n_rows > 0) {
        const hw::buffer_rsrc src = hw::make_rsrc(p.part_out + (((size_t)t * ns + i) * p.n_heads + head0) * kDv);
#pragma unroll
        for (int j = 0; j < 16; ++j)
          v[j] = hw::load_b128_agent(src, (uint32_t)((min(r0 + j, n_rows - 1) * kDv + col4) * 4));
      } else {                                 // a head group without heads has no partials to read (and stores nothing)
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float rb = s_w[r0 + j];
#pragma unroll
        for (int c = 0; c < 4; ++c) sum[j][c] = __fadd_rn(sum[j][c], __fmul_rn(v[j][c], rb));
      }
    }
#pragma unroll
    for (int j = 0; j < 16; ++j)
      if (r0 + j < n_rows) store_bf16x4(r0 + j, make_float4(sum[j][0], sum[j][1], sum[j][2], sum[j][3]));
  }
  __syncthreads();
  if (tid_e == 0) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
  return;
  }      // (the loop over items)
}

template <int FMT, bool CAP>
static int launch_tall_impl(const Params& p, hipStream_t s) {
  const int n_hblocks = (p.n_heads + 63) / 64;
  const long long blocks = ((long long)p.n_tokens + 7) / 8 * 8 * n_hblocks * p.n_splits;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return SMLA_EINVAL_SHAPE;
  // Persistent workgroups where a compute unit has several items to go through and nothing is
  // split (FLAGTREE_SMLA_PERSIST=1, opt-in until measured): one workgroup per compute unit; the
  // count must be a multiple of 8 for the ids a workgroup walks to stay on its XCD.
  // (built for bf16 rows without a logit cap, the prefill and dense-decode case; the other
  // instantiations have no registers to spare for the loop-carried state)
  if constexpr (FMT == SMLA_KV_BF16 && !CAP) {
    if (p.persist_workgroups > 0 && p.n_splits == 1 && blocks >= 2LL * p.persist_workgroups) {
      hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_tall_kernel<FMT, CAP, true>), dim3((unsigned)p.persist_workgroups), dim3(kNT), 0, s, p, n_hblocks,
                         (int)blocks);
      return hip_status(hipGetLastError());
    }
  }
  hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_tall_kernel<FMT, CAP>), dim3((unsigned)blocks), dim3(kNT), 0, s, p, n_hblocks, (int)blocks);
  return hip_status(hipGetLastError());
}

int launch_fwd_tall(int kv_format, const Params& p, hipStream_t s) {
  const bool cap = p.logit_cap > 0.f;
  if (kv_format == SMLA_KV_BF16) return cap ? launch_tall_impl<SMLA_KV_BF16, true>(p, s) : launch_tall_impl<SMLA_KV_BF16, false>(p, s);
  if (kv_format == SMLA_KV_FP8_B128)
    return cap ? launch_tall_impl<SMLA_KV_FP8_B128, true>(p, s) : launch_tall_impl<SMLA_KV_FP8_B128, false>(p, s);
  return SMLA_EINVAL_SHAPE;
}

}  // namespace smla
