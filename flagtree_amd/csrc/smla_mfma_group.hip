// Sparse-MLA forward, MFMA kernel for many heads, third design: 128 heads of a token in one
// workgroup, every wavefront on its own.
//
// One workgroup of 4 wavefronts, one per SIMD, handles (token, block of 128 heads, split of the
// top-k list); wavefront w owns heads 32w .. 32w+31 from the scores to the output: its 32 x 576 Q
// block (144 registers) and its 32 x 512 fp32 accumulators (256 registers, in AGPRs) stay resident.
// The only thing the wavefronts share is the ring of 32-token tiles that global -> LDS moves fill
// (one barrier per tile); each selected row is fetched into ONE compute unit (the first design,
// smla_mfma_tall.hip, fetches it into two), and nothing else travels through LDS:
//   scores: both 16-token halves of a tile against both 16-head tiles of the group,
//        S^T[16 tok x 16 heads] = K_rows[16 x 576] . Q^T[576 x 16]     4 x 18 v_mfma_f32_16x16x32_bf16
//        lane (q = l/16, n = l%16) then holds head n, tokens 4q .. 4q+3 of either half;
//   probabilities: stay in those registers.  The eight values a lane holds for a head -- tokens
//        4q+j and 16+4q+j, j = 0..3 -- are exactly the A operand of the same MFMA shape with the
//        tile's 32 tokens as its k dimension taken in that order (k-slot 8q+j = token 4q+j, k-slot
//        8q+4+j = token 16+4q+j);
//   output: O[16 heads x 16 dv] += P[16 heads x 32 tok] . V[32 tok x 16 dv]   2 x 32 v_mfma_f32_16x16x32_bf16
//        with B gathered in the same token order by transposing LDS reads of the same tile.
// So there is no P buffer, no exchange between wavefronts for the softmax, and per tile a wavefront
// issues about as many instructions as in the first design for twice the matrix work.
// Per tile, LDS traffic is the four wavefronts' reads of the tile (K once, V once each) plus the
// moves that fill it.
//
// Register layouts (wave64):
//   v_mfma_f32_16x16x32_bf16  A: lane l holds A[m = l%16][k = 8*(l/16) .. +7]   B: B[k = 8*(l/16) .. +7][n = l%16]
//                             D: lane l, reg r holds D[m = 4*(l/16) + r][n = l%16]
//   ds_read_b64_tr_b16: inside each group of 16 lanes, lane i receives element (i%4) of the
//   8-byte rows addressed by lanes (i/4), (i/4)+4, (i/4)+8, (i/4)+12.
#include "smla_common.h"
#include "smla_fp8_pipe.h"

namespace smla {
namespace {

using hw::bf16x8;
using hw::bf16x4;
using hw::f32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

constexpr int kNT = 256;                      // threads per workgroup
constexpr int kTN = 32;                       // tokens per tile
constexpr int kSlots = 4;                     // ring slots
// LDS tile layout.  The 512 NoPE / V columns of tile row r occupy the 1 KB at r * kMainStride,
// 16-byte chunk c stored at chunk position c ^ swz(r), swz(r) = ((r & 7) << 1) | ((r >> 3) & 1)
// (a bijection on any 16 consecutive rows).  LDS has 64 banks of 4 bytes.
//  * The score MFMAs read one chunk column of 16 consecutive rows, 16 lanes at a time: 16 distinct
//    chunk positions inside one 256-byte window, all banks.
//  * The P.V MFMAs read, 32 lanes at a time, 32 contiguous bytes (chunks 2c, 2c+1) of the eight rows
//    4q .. 4q+3, q = 0, 1 (or q = 2, 3) of a 16-row half: the eight rows' swz values differ in bits
//    1-3, so the eight chunk pairs are distinct: all banks again.
// The 64 RoPE columns (8 chunks) of rows 2p, 2p+1 share the 256 bytes at kRopeBase + p * 256: chunk
// c of row r sits at slot ((r & 1) << 3) | (c ^ (p & 7)).
constexpr int kMainStride = 1024;
constexpr int kRopeBase = kTN * kMainStride;          // 32768
constexpr int kTileBytes = kRopeBase + kTN * 128;     // 36864
__host__ __device__ constexpr int swz(int r) { return ((r & 7) << 1) | ((r >> 3) & 1); }
constexpr int kChunk = 1024;                  // top-k entries compacted into LDS at a time
constexpr int kBtLdsMax = 8192;               // page-table entries that fit the staging area (32 KB of a ring slot)
constexpr int kDmaSteps = 9;                  // move instructions per wavefront per tile (8 rows + 1 RoPE block)
constexpr int kColTiles = kDv / 16;           // 32 output column tiles of 16
constexpr float kSlack = 30.f;                // see the softmax reference note in smla_mfma_tall.hip
enum { kPassFast = 0, kPassMax = 1, kPassFinal = 2 };
constexpr int kPrefetchA = 3;                 // k-steps of K fragments ahead in the score loop (2 fragments each)
constexpr int kPrefetchB = 3;                 // column tiles of V fragments ahead in the P.V loop

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ uint32_t rope_slot(int r, int c) {     // byte offset of RoPE chunk c of tile row r in a tile's RoPE block
  const int p = r >> 1;
  return p * 256 + ((((r & 1) << 3) | (c ^ (p & 7))) << 4);
}

// fp8 records: raw records -> LDS by moves, LDS -> LDS conversion (smla_fp8_pipe.h).  This kernel's
// row xor: swz(row0 + 2k) = swz(row0) ^ 4k for row0 = 8 * wave + l/32 (bits 1-3 count the row within its eight).
struct GroupLayout {
  __device__ static constexpr int swz(int r) { return ((r & 7) << 1) | ((r >> 3) & 1); }
  __device__ static constexpr int store_xor(int k) { return 4 * k; }
};
using Fp8Pipe = fp8pipe::Pipe;
using Fp8Convert = fp8pipe::Convert<GroupLayout>;
static_assert(fp8pipe::kTN == kTN && fp8pipe::kMainStride == kMainStride && fp8pipe::kRopeBase == kRopeBase, "tile geometry");
static_assert(fp8pipe::layout_ok<GroupLayout>(), "store_xor must describe this kernel's row xor");

// A tile's rows go global -> LDS directly: one move brings the first 1 KB of a row (scalar row base
// + per-lane chunk offset; lane l fetches chunk l ^ swz(row) so the row lands swizzled), one more
// the remaining 128 bytes of eight rows.  Rows past the valid count repeat the last valid row
// (their scores are masked, their probabilities are exactly zero).
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
      hw::dma_b128(voff ^ (uint32_t)(swz(r) << 4), sbase, tile_lds + r * kMainStride);
    } else {
      const int pair = 4 * wave + (lane >> 4);
      const int r = 2 * pair + ((lane >> 3) & 1), c = (lane & 7) ^ (pair & 7);
      const int32_t trow = __shfl(rid, r);
      hw::dma_b128(kv + (size_t)trow * kRowBytesBf16 + 1024 + c * 16, tile_lds + kRopeBase + wave * 1024);
    }
  }
};

// s_waitcnt vmcnt(n) for a run-time n in {0, kDmaSteps, 2 * kDmaSteps}
__device__ __forceinline__ void wait_dma(int younger_tiles) {
  if (younger_tiles >= 2) hw::wait_vmcnt<2 * kDmaSteps>();
  else if (younger_tiles == 1) hw::wait_vmcnt<kDmaSteps>();
  else hw::wait_vmcnt<0>();
}

// Raw scores of a tile (body at `tile`, RoPE block at `rope`): sa[2 * tt + ht] = S^T of token half tt (tile rows 16 tt .. + 15) against
// head tile ht (heads 16 ht .. + 15 of the group).  Four independent accumulation chains; a K
// fragment feeds two MFMAs.  `side(ks)` is called once per k-step.
template <int kAhead = kPrefetchA, typename Side>
__device__ __forceinline__ void tile_scores(uint32_t tile, uint32_t rope, const bf16x8 (&qf)[kDqk / 32][2], f32x4 (&sa)[4], int lane, Side side) {
  constexpr int kSteps = kDqk / 32, kMainSteps = kDv / 32;
  const int l16 = lane & 15, q4 = lane >> 4;
  // row 16 tt + l16: swz depends on l16 only; chunk 4 ks + q4 sits at ((4 ks + q4) ^ swz) * 16
  const uint32_t kmain = tile + l16 * kMainStride + ((q4 ^ swz(l16)) << 4);
  auto frag = [&](int ks, int tt) {
    if (ks < kMainSteps) return hw::lds_read_b128((kmain ^ (uint32_t)((ks & 3) << 6)) + (ks >> 2) * 256 + tt * 16 * kMainStride);
    return hw::lds_read_b128(rope + rope_slot(16 * tt + l16, 4 * (ks - kMainSteps) + q4));
  };
#pragma unroll
  for (int i = 0; i < 4; ++i) sa[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  __builtin_amdgcn_sched_barrier(0);
  bf16x8 a[kSteps][2];
#pragma unroll
  for (int ks = 0; ks < kAhead; ++ks) { a[ks][0] = frag(ks, 0); a[ks][1] = frag(ks, 1); }
#pragma unroll
  for (int ks = 0; ks < kSteps; ++ks) {
    if (ks + kAhead < kSteps) { a[ks + kAhead][0] = frag(ks + kAhead, 0); a[ks + kAhead][1] = frag(ks + kAhead, 1); }
    sa[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ks][0], qf[ks][0], sa[0], 0, 0, 0);
    sa[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ks][0], qf[ks][1], sa[1], 0, 0, 0);
    sa[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ks][1], qf[ks][0], sa[2], 0, 0, 0);
    sa[3] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ks][1], qf[ks][1], sa[3], 0, 0, 0);
    side(ks);
  }
#pragma unroll
  for (int ks = 0; ks < kAhead; ++ks) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // DS read
#pragma unroll
  for (int ks = 0; ks < kSteps; ++ks) {
    if (ks + kAhead < kSteps) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);                                         // MFMA
  }
  __builtin_amdgcn_sched_barrier(0);
}

// O[32 heads x 512] += P[32 heads x 32 tok] . V[32 tok x 512] over one tile.  acc[ht][ct] is the
// [16 heads x 16 dv] tile of head tile ht and columns 16 ct .. + 15: lane owns column l%16, register
// r is head row 4*(l/16) + r.  pa[ht] is the lane's A operand (its own probabilities, see the top of
// the file).  B for column tile ct: lane p of a 16-lane group q addresses the 8 bytes at columns
// 16 ct + 4 (p%4) .. + 3 of token 4q + p/4 (first read: k-slots 8q .. 8q+3) and of token
// 16 + 4q + p/4 (second read: k-slots 8q+4 .. 8q+7).
// `valu(i)` is independent vector work of the caller, pinned behind MFMA pair i.
// kFreshAddr: the lane's part of the addresses is worked out afresh in every call (the variant short
// of registers cannot afford the eight xor-ed copies the compiler would otherwise keep for the whole kernel).
template <bool kPinValu, bool kFreshAddr, int kAhead = kPrefetchB, typename Valu>
__device__ __forceinline__ void tile_accumulate(uint32_t tile, const bf16x8 (&pa)[2], f32x4 (&acc)[2][kColTiles], int lane, Valu valu) {
  const int q4 = lane >> 4, p16 = lane & 15;
  const int row = 4 * q4 + (p16 >> 2);                           // token of the first read; the second read's is row + 16 (same swz)
  // columns 16 ct + 4 (p%4): chunk 2 ct + (p%4 >> 1), byte 8 (p%4 & 1); the chunk moves to (2 ct) ^ swz(row) ^ (p%4 >> 1)
  uint32_t lane_part = row * kMainStride + ((swz(row) ^ ((p16 & 3) >> 1)) << 4) + 8 * (p16 & 1);
  if constexpr (kFreshAddr) hw::pin(lane_part);
  const uint32_t vbase = tile + lane_part;
  __builtin_amdgcn_sched_barrier(0);
  bf16x4 lo[kColTiles], hi[kColTiles];
  // chunk 2 ct: the xor with swz touches its low four bits only, so column tiles 8 apart share an
  // address up to a constant (bits 8, 9 of vbase are clear): eight xors a tile instead of thirty-two
  auto load = [&](int ct) {
    const uint32_t a = (vbase ^ (uint32_t)(32 * (ct & 7))) + 256 * (ct >> 3);
    lo[ct] = hw::lds_read_tr16_b64(a);
    hi[ct] = hw::lds_read_tr16_b64(a + 16 * kMainStride);
  };
#pragma unroll
  for (int ct = 0; ct < kAhead; ++ct) load(ct);
#pragma unroll
  for (int ct = 0; ct < kColTiles; ++ct) {
    if (ct + kAhead < kColTiles) load(ct + kAhead);
    const bf16x8 bv = __builtin_shufflevector(lo[ct], hi[ct], 0, 1, 2, 3, 4, 5, 6, 7);
    acc[0][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[0], bv, acc[0][ct], 0, 0, 0);
    acc[1][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[1], bv, acc[1][ct], 0, 0, 0);
    if constexpr (kPinValu) {
      __builtin_amdgcn_sched_barrier(0);
      valu(ct);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if constexpr (!kPinValu) {
#pragma unroll
    for (int ct = 0; ct < kAhead; ++ct) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int ct = 0; ct < kColTiles; ++ct) {
      if (ct + kAhead < kColTiles) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
}

// PERSIST: as in fwd_tall_kernel -- for launches that do not split and have several items per
// compute unit, one workgroup per compute unit walks the block ids b, b + gridDim.x, ... of the
// one-workgroup-per-item launch and sends for the next item's indices and Q at the top of the
// current item's epilogue, when Q has done its work and the registers are free.
template <int FMT, bool CAP, bool PERSIST = false>
__global__ __launch_bounds__(kNT) void fwd_group_kernel(Params p, int n_hblocks, int n_items) {
  // the ring area: bf16 has four whole tiles (body + RoPE block each); fp8 see smla_fp8_pipe.h
  constexpr bool kFp8 = FMT == SMLA_KV_FP8_B128;
  static_assert(Fp8Pipe::kRingBytes <= kSlots * kTileBytes, "the fp8 carving fits the same area");
  __shared__ __attribute__((aligned(1024))) uint8_t s_ring[kSlots * kTileBytes];   // swizzle xors need 1 KB alignment
  __shared__ int32_t s_rows[kChunk];
  __shared__ float s_inv[4][32];                                  // per-head normalisers (epilogue)
  __shared__ float s_w[4][4][16];                                 // split merge: [wavefront][split of the batch][row of the head tile] weights
  __shared__ int s_nvalid;
  __shared__ int s_cnt[4];
  __shared__ int s_redo;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, q4 = lane >> 4;

  // block id -> (token, split, head block); all workgroups of a token get ids 8 apart (one XCD)
  auto token_of_id = [&](int id) { return token_of(p, id & 7, (id >> 3) / (n_hblocks * p.n_splits)); };
  auto next_item = [&](int id) {               // the next id of this workgroup that has a token
    while (id < n_items && token_of_id(id) >= p.n_tokens) id += (int)gridDim.x;
    return id;
  };
  int item = PERSIST ? next_item((int)blockIdx.x) : (int)blockIdx.x;
  if (PERSIST && item >= n_items) return;
  int hb, sp, t, seq, head0;                                      // head0: first head of this wavefront
  auto place = [&](int id) {
    const int slot = id >> 3;
    hb = slot % n_hblocks;
    sp = (slot / n_hblocks) % p.n_splits;
    t = token_of_id(id);
    seq = t / p.tokens_per_seq;
    head0 = hb * 128 + wave * 32;
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
  // the sequence's page-table row goes global -> LDS (last tile body, free until the first chunk's
  // row list exists), issued ahead of the index loads so that it has landed once they have
  const int32_t* bt_row = p.block_table ? p.block_table + (size_t)seq * p.bt_stride : nullptr;
  const bool bt_in_lds = bt_row != nullptr && p.bt_stride <= kBtLdsMax && (p.bt_stride & 3) == 0 &&
                         ((uintptr_t)bt_row & 15) == 0;
  const uint32_t lds_tile = hw::lds_addr(&s_ring[0]);
  constexpr int kBtStage = kFp8 ? (Fp8Pipe::kBodies - 1) * kRopeBase : (kSlots - 1) * kTileBytes;
  const uint32_t lds_bt = lds_tile + kBtStage;
  if (bt_in_lds) {
    for (int c = wave; 256 * c < p.bt_stride; c += 4) {            // 1 KB (256 entries) per instruction
      const int e = 256 * c + 4 * lane;
      if (e < p.bt_stride) hw::dma_b128(bt_row + e, lds_bt + 1024 * c);
    }
  }
  int32_t rr_first[4];
  load_indices(k_begin, rr_first);

  // ---- Q^T fragments of the wavefront's 32 heads: B operand of S^T; lane holds head 16 ht + l16,
  // k = 32 ks + 8 q4 .. + 7.  A head past the end reads head 0 again (its results are never
  // stored); nothing touches the values here, so the compiler does not wait for Q ahead of the
  // row list.
  bf16x8 qf[kDqk / 32][2];
  auto load_q = [&](int tt, int hhead0) {
#pragma unroll
    for (int ht = 0; ht < 2; ++ht) {
      const int hq = hhead0 + 16 * ht + l16;
      const uint16_t* qrow = static_cast<const uint16_t*>(p.q) + ((size_t)tt * p.n_heads + (hq < p.n_heads ? hq : 0)) * kDqk + 8 * q4;
#pragma unroll
      for (int ks = 0; ks < kDqk / 32; ++ks) qf[ks][ht] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
    }
  };
  load_q(t, head0);
  if (tid == 0) s_redo = 0;
  if (bt_in_lds) {
    hw::wait_for_loads_of(rr_first[0], rr_first[1], rr_first[2], rr_first[3]);
    __syncthreads();
    const int32_t* bt_s = reinterpret_cast<const int32_t*>(&s_ring[kBtStage]);
#pragma unroll
    for (int k = 0; k < 4; ++k) rr_first[k] = translate_index(p, rr_first[k], bt_s);
  } else {
    translate_entries4(p, seq, rr_first);
  }

  const float sc2 = CAP ? 1.f : p.sm_scale * kLog2e;
  [[maybe_unused]] const LogitCap cap(p.sm_scale, CAP ? p.logit_cap : 1.f);

  for (;;) {       // one item a turn (a single turn unless PERSIST)
  f32x4 acc[2][kColTiles];
#pragma unroll
  for (int ht = 0; ht < 2; ++ht)
#pragma unroll
    for (int ct = 0; ct < kColTiles; ++ct) acc[ht][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  // softmax state of heads 16 ht + l16: base-2 reference and this lane's partial row sum (its 8 tokens of every tile)
  float m_ref[2] = {-INFINITY, -INFINITY}, l_part[2] = {0.f, 0.f};

  int pass = kPassFast;
  bool first_chunk = true;
  for (;;) {
    bool failed = false;
    bool have_ref = pass == kPassFinal;
    for (int c0 = k_begin; c0 < k_end; c0 += kChunk) {
      // ---- translate + mask + compact the next chunk of the top-k list (order preserving)
      __syncthreads();                       // previous chunk's rows and tiles are no longer read
      {
        int32_t rr[4];
        if (first_chunk) {
#pragma unroll
          for (int k = 0; k < 4; ++k) rr[k] = rr_first[k];
        } else {
          load_indices(c0, rr);
          translate_entries4(p, seq, rr);
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

      // bf16: tile `it` lives in ring slot it % kSlots.  fp8: its body in body it % 3, its RoPE block in
      // block it % 3, its raw records in raw block it % 2.
      [[maybe_unused]] Fp8Pipe pipe;
      [[maybe_unused]] Fp8Convert cv;
      DmaTile dma;
      uint32_t ring = lds_tile;
      if constexpr (kFp8) hw::pin_uniform(ring);   // (per-lane addresses of the first tiles are worked out per chunk, not held from the top)
      auto tile_addr = [&](int it) {
        if constexpr (kFp8) return ring + (uint32_t)(it % Fp8Pipe::kBodies) * kRopeBase;
        else return ring + (it & (kSlots - 1)) * kTileBytes;
      };
      auto rope_addr = [&](int it) {
        if constexpr (kFp8) return ring + Fp8Pipe::kRopeRing + (uint32_t)(it % Fp8Pipe::kRopes) * fp8pipe::kRopeBlock;
        else return ring + (it & (kSlots - 1)) * kTileBytes + kRopeBase;
      };
      [[maybe_unused]] auto pipe_begin = [&](int it, int ln) {
        pipe.begin(kv, s_rows, it * kTN, n_valid,
                   ring + Fp8Pipe::kRawRing + (it & 1) * Fp8Pipe::kRawSlot + wave * Fp8Pipe::kRawWave, rope_addr(it), wave, ln);
      };
      [[maybe_unused]] auto convert_begin = [&](int it, int ln) {
        cv.raw_lds = ring + Fp8Pipe::kRawRing + (it & 1) * Fp8Pipe::kRawSlot + wave * Fp8Pipe::kRawWave;
        cv.body_lds = ring + (uint32_t)(it % Fp8Pipe::kBodies) * kRopeBase;
        cv.wave = wave; cv.lane = ln;
      };
      auto fetch_whole = [&](int it) {
        if constexpr (!kFp8) {
          dma.begin(kv, s_rows, it * kTN, n_valid, tile_addr(it), wave, lane);
#pragma unroll
          for (int j = 0; j < kDmaSteps; ++j) dma.step(j);
        } else {
          pipe_begin(it, lane);
#pragma unroll
          for (int j = 0; j < Fp8Pipe::kSteps; ++j) pipe.step(j);
        }
      };
      // scores of tile `it` -> the lane's probabilities as the A operands of the P.V MFMAs (not pipelined:
      // first tile and tail).  s[tt][ht][r]: token 16 tt + 4 q4 + r, head 16 ht + l16.
      auto finish_scores = [&](int it, f32x4 (&sa)[4], bf16x8 (&pa)[2]) {
        const int in_tile = min(kTN, n_valid - it * kTN);             // valid tokens of the tile
        if constexpr (CAP) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) sa[i][r] = cap(sa[i][r]);
        }
        if (in_tile < kTN) {                 // ragged tile (uniform): mask the rows past the end
          int first = lane;                  // this lane's first token of a half, 4 * (lane / 16),
          hw::pin(first);                    // worked out here: the row numbers are not worth registers held through the loops
          first = (first >> 4) << 2;
#pragma unroll
          for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (16 * tt + first + r >= in_tile) { sa[2 * tt][r] = -INFINITY; sa[2 * tt + 1][r] = -INFINITY; }
        }
        float mx[2];
#pragma unroll
        for (int ht = 0; ht < 2; ++ht) {
          float v = fmaxf(fmaxf(fmaxf(sa[ht][0], sa[ht][1]), fmaxf(sa[ht][2], sa[ht][3])),
                          fmaxf(fmaxf(sa[2 + ht][0], sa[2 + ht][1]), fmaxf(sa[2 + ht][2], sa[2 + ht][3])));
          mx[ht] = v * sc2;                  // sc2 > 0: scaling commutes with the maximum
        }
        if (!have_ref) {                     // first tile of the pass (uniform): the head's maximum over the tile is its reference
#pragma unroll
          for (int ht = 0; ht < 2; ++ht) {
            mx[ht] = fmaxf(mx[ht], __shfl_xor(mx[ht], 16));
            mx[ht] = fmaxf(mx[ht], __shfl_xor(mx[ht], 32));
            if (pass == kPassFast) m_ref[ht] = mx[ht];
          }
          have_ref = true;
        }
        if (pass == kPassMax) { m_ref[0] = fmaxf(m_ref[0], mx[0]); m_ref[1] = fmaxf(m_ref[1], mx[1]); }
        if (pass == kPassFast) failed |= __any(mx[0] > m_ref[0] + kSlack || mx[1] > m_ref[1] + kSlack);
#pragma unroll
        for (int ht = 0; ht < 2; ++ht) {
          float pr[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sa[2 * (j >> 2) + ht][j & 3], sc2, -m_ref[ht]));
          l_part[ht] += ((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7]));
          const hw::u32x4 w = {pack_bf16(pr[0], pr[1]), pack_bf16(pr[2], pr[3]), pack_bf16(pr[4], pr[5]), pack_bf16(pr[6], pr[7])};
          pa[ht] = __builtin_bit_cast(bf16x8, w);
        }
      };

      // ---- prologue: tiles 0 and 1 go out at once (Q may still be on its way: loads complete in
      // issue order, so waiting for the moves also waits for everything older), tile 2 rides on
      // the scores of tile 0
      for (int it = 0; it < min(n_tiles, 2); ++it) fetch_whole(it);
      if constexpr (!kFp8) {
        wait_dma(n_tiles > 1 ? 1 : 0);
      } else {
        // fp8: convert tile 0, send for tile 2 (its raw block is free again), convert tile 1
        // (a wavefront's lanes read scale chunks that other lanes of it fetched: wave_lds_order)
        if (n_tiles > 1) hw::wait_vmcnt<Fp8Pipe::kSteps>(); else hw::wait_vmcnt<0>();
        hw::wave_lds_order();
        convert_begin(0, lane);
        cv.whole_tile();
        if (n_tiles > 2) fetch_whole(2);
        if (n_tiles > 1) {
          if (n_tiles > 2) hw::wait_vmcnt<Fp8Pipe::kSteps>(); else hw::wait_vmcnt<0>();
          hw::wave_lds_order();
          convert_begin(1, lane);
          cv.whole_tile();
        }
      }
#pragma unroll
      for (int ks = 0; ks < kDqk / 32; ++ks) hw::wait_for_loads_of(qf[ks][0], qf[ks][1]);   // (tells the compiler that Q is there)
      __syncthreads();                       // tile 0 landed
      bf16x8 pa[2];                          // probabilities of the tile to be accumulated next
      {
        f32x4 sa[4];
        if (!kFp8 && n_tiles > 2) {
          dma.begin(kv, s_rows, 2 * kTN, n_valid, tile_addr(2), wave, lane);
          tile_scores(tile_addr(0), rope_addr(0), qf, sa, lane, [&](int ks) { if ((ks & 1) == 0) dma.step(ks >> 1); });
        } else {
          tile_scores(tile_addr(0), rope_addr(0), qf, sa, lane, [](int) {});
        }
        finish_scores(0, sa, pa);
      }

      // ---- main loop: iterations that still have a tile to fetch (it + 3 < n_tiles, so tiles it+1
      // and it+2 exist and tile it+1 is full).  The fetch of tile it+3 rides on the score MFMAs of
      // tile it+1; the softmax of tile it+1 is cut into slices pinned between the P.V MFMAs of tile it.
      const int n_main = max(n_tiles - (kSlots - 1), 0);
      int it = 0;
      for (; it < n_main; ++it) {
        if constexpr (!kFp8) wait_dma(1);    // tile it+1 was issued two iterations ago; only tile it+2 is still outstanding
        __syncthreads();                     // tile it+1 landed / converted for everyone, tile it-1 is consumed by everyone
        if constexpr (!kFp8) {
          dma.begin(kv, s_rows, (it + kSlots - 1) * kTN, n_valid, tile_addr(it + kSlots - 1), wave, lane);
        }
        // fp8: the lane id is taken afresh in every iteration, so that the dozen per-lane address parts
        // derived from it are worked out here (a few instructions each) rather than held in registers
        // for the whole kernel, which this variant cannot afford
        int ln = lane;
        if constexpr (kFp8) {
          hw::pin(ln);
          pipe_begin(it + 3, ln);            // send for tile it+3; the raw records of tile it+2 are converted under the P.V MFMAs below
          convert_begin(it + 2, ln);
        }
        f32x4 sa[4];
        // (fp8: the conversion shares the loop's registers: one fragment pair and one column tile less ahead)
        tile_scores<kFp8 ? kPrefetchA - 1 : kPrefetchA>(tile_addr(it + 1), rope_addr(it + 1), qf, sa, ln, [&](int ks) {
          if ((ks & 1) == 0) {
            if constexpr (!kFp8) dma.step(ks >> 1);
            else if ((ks >> 1) < Fp8Pipe::kSteps) pipe.step(ks >> 1);
          }
        });
        float pr[8];
        hw::u32x4 pw[2];
        bool over = false;
        tile_accumulate<true, kFp8, kFp8 ? kPrefetchB - 1 : kPrefetchB>(tile_addr(it), pa, acc, ln, [&](int i) {
          if constexpr (kFp8) {
            // slices 23..27 carry the conversion, after the softmax (slices 0..22) has given its
            // registers back: the read of chunk 0, then per chunk its two halves, its stores and the
            // next chunk's read.  The moves of tile it+3, just issued, stay in flight; everything
            // older has landed after the wait.
            if (i == 23) { hw::wait_vmcnt<Fp8Pipe::kSteps>(); hw::wave_lds_order(); cv.load(0); }
            else if (i >= 24 && i < 28) { cv.half(0); cv.half(1); cv.store(i - 24); if (i < 27) cv.load(i - 23); }
          }
          if (i < 4) {                       // slices 0..3: one score block each: cap, per-lane maximum, overflow test
            if constexpr (CAP) {
#pragma unroll
              for (int r = 0; r < 4; ++r) sa[i][r] = cap(sa[i][r]);
            }
            const int ht = i & 1;
            const float lm = fmaxf(fmaxf(sa[i][0], sa[i][1]), fmaxf(sa[i][2], sa[i][3])) * sc2;
            m_ref[ht] = pass == kPassMax ? fmaxf(m_ref[ht], lm) : m_ref[ht];
            over |= lm > m_ref[ht] + kSlack;
            hw::pin(m_ref[ht]);
          } else if (i < 22) {               // slices 4..12 head tile 0, 13..21 head tile 1: eight probabilities, then row sum and bf16 packing
            const int ht = (i - 4) / 9, j = (i - 4) % 9;
            if (j < 8) {
              pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sa[2 * (j >> 2) + ht][j & 3], sc2, -m_ref[ht]));
              hw::pin(pr[j]);
            } else {
              l_part[ht] += ((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7]));
              pw[ht] = hw::u32x4{pack_bf16(pr[0], pr[1]), pack_bf16(pr[2], pr[3]), pack_bf16(pr[4], pr[5]), pack_bf16(pr[6], pr[7])};
              hw::pin(l_part[ht], pw[ht]);
            }
          } else if (i == 22) {
            failed |= pass == kPassFast && __any(over);
          }
        });
        pa[0] = __builtin_bit_cast(bf16x8, pw[0]);
        pa[1] = __builtin_bit_cast(bf16x8, pw[1]);
      }
      // ---- tail: the last tiles, nothing left to fetch
      for (; it < n_tiles; ++it) {
        const bool next = it + 1 < n_tiles;
        if constexpr (!kFp8) { if (next) wait_dma(it + 2 < n_tiles ? 1 : 0); }
        __syncthreads();
        if constexpr (kFp8) {                // tile it+2 may still await its conversion
          if (it + 2 < n_tiles) {
            hw::wait_vmcnt<0>();
            hw::wave_lds_order();
            convert_begin(it + 2, lane);
            cv.whole_tile();
          }
        }
        bf16x8 pn[2] = {pa[0], pa[1]};
        if (next) {
          f32x4 sa[4];
          tile_scores(tile_addr(it + 1), rope_addr(it + 1), qf, sa, lane, [](int) {});
          finish_scores(it + 1, sa, pn);
        }
        tile_accumulate<false, kFp8>(tile_addr(it), pa, acc, lane, [](int) {});
        pa[0] = pn[0]; pa[1] = pn[1];
      }
    }
    if (pass == kPassFinal) break;
    if (pass == kPassFast) {
      if (failed && lane == 0) s_redo = 1;
      __syncthreads();
      if (s_redo == 0) break;                // the common case
      m_ref[0] = -INFINITY; m_ref[1] = -INFINITY;
      pass = kPassMax;
    } else {                                 // exact maxima: fold the four lanes of a head, then accumulate for real
#pragma unroll
      for (int ht = 0; ht < 2; ++ht) {
        m_ref[ht] = fmaxf(m_ref[ht], __shfl_xor(m_ref[ht], 16));
        m_ref[ht] = fmaxf(m_ref[ht], __shfl_xor(m_ref[ht], 32));
      }
      pass = kPassFinal;
    }
    l_part[0] = 0.f; l_part[1] = 0.f;        // what the void / max pass accumulated is dropped
#pragma unroll
    for (int ht = 0; ht < 2; ++ht)
#pragma unroll
      for (int ct = 0; ct < kColTiles; ++ct) acc[ht][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- epilogue.  A wavefront knows all about its own 32 heads; its [32 x 512] block goes through
  // LDS 16 head rows (one head tile) at a time: parked as accumulator tiles (lane = column, register
  // = row), read back one head row at a time, 8 consecutive columns per lane.
  __syncthreads();                           // the ring is free
  // PERSIST: Q has done its work and the first chunk's index values theirs; the registers they
  // live in take the next item's, sent for now, ahead of this item's stores.
  [[maybe_unused]] int item_next = 0;
  if constexpr (PERSIST) {
    item_next = next_item(item + (int)gridDim.x);
    if (item_next < n_items) {
      const int slot_n = item_next >> 3, t_n = token_of_id(item_next);
      load_indices_of(t_n, t_n / p.tokens_per_seq, k_begin, rr_first);
      load_q(t_n, (slot_n % n_hblocks) * 128 + wave * 32);
      if (tid == 0) s_redo = 0;
    }
  }
  if (p.n_splits > 1 && tid == 0)
    s_nvalid = ws_arrive(p, p.counters + (size_t)t * n_hblocks + hb, ws_head, p.n_splits, sp);
  const int lane_e = hw::lane_id();          // (lane coordinates retaken here rather than carried through the loop)
  const int l16_e = lane_e & 15, q4_e = lane_e >> 4;
  float lse_nat[2];                          // of heads 16 ht + l16
#pragma unroll
  for (int ht = 0; ht < 2; ++ht) {
    float l = l_part[ht];
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    lse_nat[ht] = l > 0.f ? (m_ref[ht] + __builtin_amdgcn_logf(l)) * kLn2 : -INFINITY;
    if (q4_e == 0) s_inv[wave][16 * ht + l16_e] = l > 0.f ? 1.f / l : 0.f;
  }
  hw::wave_lds_order();
  const int n_rows = max(0, min(32, p.n_heads - head0));           // head rows that exist (wave-uniform)
  constexpr int kStageStride = kDv + 4;                            // floats per staged row (+16 B pad: the four row groups a store touches start 16 banks apart)
  static_assert(4 * 16 * kStageStride * 4 <= kSlots * kTileBytes, "the staged blocks must fit the ring area");
  float* stage = reinterpret_cast<float*>(&s_ring[0]) + wave * 16 * kStageStride;
  const int col8 = 8 * lane_e;                                     // this lane's 8 output columns when rows are read back
  // head tile ht -> stage, normalised: the very numbers a publisher stores
  // (always inlined: a call would make the accumulators addressable, that is, put them in memory)
  auto stage_rows = [&](const f32x4 (&a)[kColTiles], int ht) __attribute__((always_inline)) {
    hw::wave_lds_order();                                          // the previous tile's rows have been read by every lane
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float sc = s_inv[wave][16 * ht + 4 * q4_e + r];
#pragma unroll
      for (int ct = 0; ct < kColTiles; ++ct)
        stage[(4 * q4_e + r) * kStageStride + 16 * ct + l16_e] = __fmul_rn(a[ct][r], sc);
    }
    hw::wave_lds_order();
  };
  // (the accumulators are registers: which tile is meant must be known at compile time)
  auto stage_tile = [&](int ht) __attribute__((always_inline)) {
    if (ht == 0) stage_rows(acc[0], 0);
    else stage_rows(acc[1], 1);
  };
  auto staged = [&](int row16, int half) { return *reinterpret_cast<const float4*>(stage + row16 * kStageStride + col8 + 4 * half); };
  auto store_bf16x8 = [&](int row, float4 a, float4 b) {
    uint4 w;
    w.x = pack_bf16(a.x, a.y); w.y = pack_bf16(a.z, a.w); w.z = pack_bf16(b.x, b.y); w.w = pack_bf16(b.z, b.w);
    *reinterpret_cast<uint4*>(static_cast<uint16_t*>(p.out) + ((size_t)t * p.n_heads + head0 + row) * kDv + col8) = w;
  };
  auto lse_index = [&](int ht) { return (size_t)t * p.n_heads + head0 + 16 * ht + l16_e; };
  // Partial sums of split i of this item, as bf16: [head][512] from head0 on, in the first half of
  // the area the workspace keeps for fp32 partials.  A normalised partial is an average of cache
  // values, the output is bf16 anyway, and the merge still weighs and adds in fp32.
  auto part16 = [&](int i) {
    return reinterpret_cast<uint16_t*>(p.part_out) + (((size_t)t * p.n_splits + i) * p.n_heads + head0) * kDv;
  };
  auto head_ok = [&](int ht) { return head0 + 16 * ht + l16_e < p.n_heads; };

  const int ns = p.n_splits;
  if (PERSIST || ns == 1) {
#pragma unroll
    for (int ht = 0; ht < 2; ++ht) {
      if (q4_e == 0 && head_ok(ht)) p.lse[lse_index(ht)] = lse_nat[ht];
      stage_tile(ht);
      for (int row = 0; row < 16; ++row)
        if (16 * ht + row < n_rows) store_bf16x8(16 * ht + row, staged(row, 0), staged(row, 1));
    }
    if constexpr (PERSIST) {
      if (item_next >= n_items) return;
      item = item_next;
      place(item);                           // from here on t, seq, head0 are the next item's
      translate_entries4(p, seq, rr_first);  // waits for its index values only; page-table look-ups straight from memory
      continue;                              // (the barrier that opens its first chunk also ends everyone's reads of the staged rows)
    } else {
      return;
    }
  }

  // ---- split merge inside the launch (protocol and failure handling: ws_arrive / ws_wait_published
  // in smla_common.h; described in smla_mfma_tall.hip)
  unsigned long long* word = p.counters + (size_t)t * n_hblocks + hb;
  __syncthreads();                                                 // the ticket lane 0 of wavefront 0 took at the top of the epilogue is in s_nvalid
  const int role = s_nvalid;
  auto give_up = [&]() {                                           // mark the rows: NaN LSE, zero output
#pragma unroll
    for (int ht = 0; ht < 2; ++ht)
      if (q4_e == 0 && head_ok(ht)) p.lse[lse_index(ht)] = __uint_as_float(0x7fc00000u);
    const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int row = 0; row < n_rows; ++row) store_bf16x8(row, z, z);
  };
  if (role == kRoleError) { give_up(); return; }
  if (role == kRolePublish) {
#pragma unroll
    for (int ht = 0; ht < 2; ++ht) {
      if (q4_e == 0 && head_ok(ht))
        __hip_atomic_store(&p.part_lse[((size_t)t * ns + sp) * p.n_heads + head0 + 16 * ht + l16_e], lse_nat[ht], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      stage_tile(ht);
      // (partials of this kernel are bf16: with four splits of 128 heads the fp32 ones were a third
      // of the headline decode's traffic, all of it in the tail; see part16)
      uint16_t* o = part16(sp) + (size_t)(16 * ht) * kDv + col8;
      for (int row = 0; row < 16; ++row) {
        if (16 * ht + row >= n_rows) break;
        const float4 a = staged(row, 0), b = staged(row, 1);
        hw::u32x4 w;
        w[0] = pack_bf16(a.x, a.y); w[1] = pack_bf16(a.z, a.w); w[2] = pack_bf16(b.x, b.y); w[3] = pack_bf16(b.z, b.w);
        hw::store_b128_agent(reinterpret_cast<float*>(o + (size_t)row * kDv), __builtin_bit_cast(f32x4, w));
      }
    }
    hw::wait_vmcnt<0>();
    __syncthreads();
    if (wave == 0 && lane_e == 0) ws_publish(p, word, sp);
    return;
  }
  // last arrival: wait for the others, then fold the normalised partials in split order with every
  // product and sum rounded on its own: the result does not depend on which split arrived last.
  // Per-head scalars live in lanes (q4 = 0..3 redundantly, l16 = head in tile).
  if (wave == 0 && lane_e == 0) s_redo = ws_wait_published(p, word, ns, sp) ? 0 : 1;
  __syncthreads();
  if (s_redo != 0) { give_up(); return; }
  constexpr int kRound = 4, kBatch = 4;
#pragma unroll 1
  for (int ht = 0; ht < 2; ++ht) {
    const float own_lse = ht == 0 ? lse_nat[0] : lse_nat[1];      // (registers: the index must be a constant)
    auto split_lse = [&](int i) {
      if (i == sp) return own_lse;
      return head_ok(ht) ? __hip_atomic_load(&p.part_lse[((size_t)t * ns + i) * p.n_heads + head0 + 16 * ht + l16_e], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT)
                         : -INFINITY;
    };
    float m_all = -INFINITY;
    for (int i = 0; i < ns; ++i) m_all = fmaxf(m_all, split_lse(i));
    const float m_safe = m_all == -INFINITY ? 0.f : m_all;
    float w_sum = 0.f;
    for (int i = 0; i < ns; ++i) w_sum = __fadd_rn(w_sum, __expf(split_lse(i) - m_safe));      // exp(-inf) = 0
    const float rw = w_sum > 0.f ? 1.f / w_sum : 0.f;
    if (q4_e == 0 && head_ok(ht)) p.lse[lse_index(ht)] = w_sum > 0.f ? m_all + __logf(w_sum) : -INFINITY;
    stage_tile(ht);
    const int rows_here = max(0, min(16, n_rows - 16 * ht));
#pragma unroll 1
    for (int r0 = 0; r0 < 16; r0 += kRound) {
      // Rounds of kRound rows; the splits are taken kBatch at a time, all their loads issued before
      // the first is used (2 * kRound * kBatch = 32 sixteen-byte loads in flight per lane, 128 KB per
      // workgroup: what the merge costs is the latency of these loads), then folded in split order.
      f32x4 sum[kRound][2];
#pragma unroll
      for (int j = 0; j < kRound; ++j) { sum[j][0] = f32x4{0.f, 0.f, 0.f, 0.f}; sum[j][1] = f32x4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll 1
      for (int i0 = 0; i0 < ns; i0 += kBatch) {
        hw::wave_lds_order();
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {   // lane (q4, l16): weight of row l16 of the tile for split i0 + b
          const float wi = i0 + b < ns ? __fmul_rn(__expf(split_lse(i0 + b) - m_safe), rw) : 0.f;
          if (q4_e == 0) s_w[wave][b][l16_e] = wi;
        }
        hw::wave_lds_order();
        hw::u32x4 raw[kBatch][kRound];       // eight bf16 values each; this split's own rows rounded like the others'
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          const int i = i0 + b;
          if (i < ns && i != sp && rows_here > r0) {
            const hw::buffer_rsrc src = hw::make_rsrc(part16(i) + (size_t)(16 * ht) * kDv);
#pragma unroll
            for (int j = 0; j < kRound; ++j) {
              const uint32_t off = (uint32_t)((min(r0 + j, rows_here - 1) * kDv + col8) * 2);
              raw[b][j] = __builtin_bit_cast(hw::u32x4, hw::load_b128_agent(src, off));
            }
          } else if (i == sp) {
#pragma unroll
            for (int j = 0; j < kRound; ++j) {
              const float4 a = staged(r0 + j, 0), c = staged(r0 + j, 1);
              raw[b][j] = hw::u32x4{pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(c.x, c.y), pack_bf16(c.z, c.w)};
            }
          } else {                           // no such split, or rows past the last head: nothing to read, nothing stored
#pragma unroll
            for (int j = 0; j < kRound; ++j) raw[b][j] = hw::u32x4{0u, 0u, 0u, 0u};
          }
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          if (i0 + b < ns) {
#pragma unroll
            for (int j = 0; j < kRound; ++j) {
              const float rb = s_w[wave][b][r0 + j];
#pragma unroll
              for (int c = 0; c < 4; ++c) {   // word c of a row = columns 2c (low half) and 2c + 1
                const float even = __uint_as_float(raw[b][j][c] << 16), odd = __uint_as_float(raw[b][j][c] & 0xffff0000u);
                sum[j][c >> 1][2 * (c & 1)] = __fadd_rn(sum[j][c >> 1][2 * (c & 1)], __fmul_rn(even, rb));
                sum[j][c >> 1][2 * (c & 1) + 1] = __fadd_rn(sum[j][c >> 1][2 * (c & 1) + 1], __fmul_rn(odd, rb));
              }
            }
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kRound; ++j)
        if (r0 + j < rows_here)
          store_bf16x8(16 * ht + r0 + j, make_float4(sum[j][0][0], sum[j][0][1], sum[j][0][2], sum[j][0][3]),
                       make_float4(sum[j][1][0], sum[j][1][1], sum[j][1][2], sum[j][1][3]));
    }
  }
  __syncthreads();
  if (wave == 0 && lane_e == 0) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
  return;
  }      // (the loop over items)
}

template <int FMT, bool CAP>
int launch_impl(const Params& p, hipStream_t s) {
  const int n_hblocks = (p.n_heads + 127) / 128;
  const long long blocks = ((long long)p.n_tokens + 7) / 8 * 8 * n_hblocks * p.n_splits;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return SMLA_EINVAL_SHAPE;
  // persistent workgroups (see fwd_tall_kernel's launcher): bf16 rows without a logit cap
  if constexpr (FMT == SMLA_KV_BF16 && !CAP) {
    if (p.persist_workgroups > 0 && p.n_splits == 1 && blocks >= 2LL * p.persist_workgroups) {
      hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_group_kernel<FMT, CAP, true>), dim3((unsigned)p.persist_workgroups), dim3(kNT), 0, s, p,
                         n_hblocks, (int)blocks);
      return hip_status(hipGetLastError());
    }
  }
  hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_group_kernel<FMT, CAP>), dim3((unsigned)blocks), dim3(kNT), 0, s, p, n_hblocks, (int)blocks);
  return hip_status(hipGetLastError());
}

}  // namespace

int launch_fwd_group(int kv_format, const Params& p, hipStream_t s) {
  const bool cap = p.logit_cap > 0.f;
  if (kv_format == SMLA_KV_BF16) return cap ? launch_impl<SMLA_KV_BF16, true>(p, s) : launch_impl<SMLA_KV_BF16, false>(p, s);
  if (kv_format == SMLA_KV_FP8_B128) return cap ? launch_impl<SMLA_KV_FP8_B128, true>(p, s) : launch_impl<SMLA_KV_FP8_B128, false>(p, s);
  return SMLA_EINVAL_SHAPE;
}

}  // namespace smla
