// Sparse-MLA forward, MFMA kernel for many heads, second design: all 128 heads of a token in one
// workgroup (bf16 cache), so every selected row is moved into ONE compute unit's LDS.  (In the
// first design, smla_mfma_tall.hip, a workgroup covers 64 heads and two compute units fetch each
// row; the L2 -> LDS traffic that costs is what bounds its loop.)
//
// One workgroup of 8 wavefronts, two per SIMD, handles (token, block of 128 heads, split of the
// top-k list).  Wavefront w = (hg, x): head group hg = w / 2 (32 heads), x = w % 2.
//   scores: heads 32 hg + 16 x .. + 15 against ALL 16 tokens of a tile over the whole of k,
//        S^T[16 tok x 16 heads] = K_rows[16 x 576] . Q^T[576 x 16]     18 v_mfma_f32_16x16x32_bf16
//        (A = LDS rows, B = Q of 16 heads in 72 registers).  A wavefront owns its heads' softmax
//        outright: reference, row sums and redo decisions need no exchange with other wavefronts.
//   probabilities: bf16, dropped into the P buffer of the tile in LDS ([head][token]).
//   output: heads 32 hg .. + 31, columns 256 x .. + 255 over the tile's 16 tokens,
//        O[32 heads x 256] += P[32 heads x 16 tok] . V[16 tok x 256]    8 v_mfma_f32_32x32x16_bf16
//        (A = P from LDS, B = V through transposing LDS reads of the same tile), 128 accumulator
//        registers.  200 of a wavefront's 256 registers are Q and accumulators.
// Tiles are 16 tokens (18 KB) in a ring of seven slots: one being accumulated, one being scored,
// four on their way, one spare; one barrier per tile.  In iteration i a wavefront scores tile i+1
// and accumulates tile i; the two wavefronts of a SIMD overlap each other's LDS latencies and
// softmax arithmetic.
//
// Register and LDS layouts of the MFMA operands, the row swizzle and the RoPE block are those of
// smla_mfma_tall.hip (a tile here is the first 16 rows of a tile there).
#include "smla_common.h"

namespace smla {
namespace {

using hw::bf16x8;
using hw::bf16x4;
using hw::f32x4;
using hw::u32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kNT = 512;                      // threads per workgroup
constexpr int kTN = 16;                       // tokens per tile
constexpr int kSlots = 7;                     // ring slots
constexpr int kAhead = 5;                     // the tile issued in iteration i is tile i + kAhead
constexpr int kMainStride = 1024;             // bytes of a row's 512 NoPE / V columns in LDS (16-byte chunks swizzled)
constexpr int kRopeBase = kTN * kMainStride;  // 16384
constexpr int kTileBytes = kRopeBase + kTN * 128;   // 18432
__host__ __device__ constexpr int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }
constexpr int kPStride = 48;                  // bytes per head row of a P buffer: 16 bf16 + 16 B pad (conflict-free 16-byte reads)
constexpr int kPBytes = 32 * kPStride;        // one head group's probabilities for one tile
constexpr int kChunk = 1024;                  // top-k entries compacted into LDS at a time
constexpr int kDvHalf = kDv / 2;
constexpr int kAccTiles = kDvHalf / 32;       // 8 accumulator tiles of 32 heads x 32 dv
constexpr int kBtLdsMax = 4096;               // page-table entries staged in LDS (16 KB of the ring's last slot)
constexpr float kSlack = 30.f;
enum { kPassFast = 0, kPassMax = 1, kPassFinal = 2 };
constexpr int kRingBytes = kSlots * kTileBytes;                 // 129 024
constexpr int kPOff = kRingBytes;                               // P buffers [tile parity][head group]
constexpr int kLdsBytes = kPOff + 2 * 4 * kPBytes;              // 141 312
constexpr int kStageStride = kDvHalf + 8;                       // floats per staged output row (+32 B pad: rows 4 apart land 32 banks apart)
static_assert(8 * 16 * kStageStride * 4 <= kLdsBytes, "the epilogue stages 16 rows x 256 columns per wavefront");
static_assert(kBtLdsMax * 4 <= kTileBytes, "the page-table row is staged in one ring slot");

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ uint32_t rope_slot(int r, int c) {     // byte offset of RoPE chunk c of tile row r
  const int p = r >> 1;
  return kRopeBase + p * 256 + ((((r & 1) << 3) | (c ^ (p & 7))) << 4);
}

// s_waitcnt vmcnt(n) for the run-time values a wavefront's move count takes: per tile a wavefront
// issues 2 moves (its two rows), wavefronts 0 and 1 a third (the RoPE tails of 8 rows)
__device__ __forceinline__ void wait_moves(int n) {
  switch (n) {
    case 0: hw::wait_vmcnt<0>(); break;
    case 2: hw::wait_vmcnt<2>(); break;
    case 3: hw::wait_vmcnt<3>(); break;
    case 4: hw::wait_vmcnt<4>(); break;
    case 6: hw::wait_vmcnt<6>(); break;
    case 8: hw::wait_vmcnt<8>(); break;
    case 9: hw::wait_vmcnt<9>(); break;
    default: hw::wait_vmcnt<12>(); break;     // 12: four tiles of three moves
  }
}

template <bool CAP>
__global__ __launch_bounds__(kNT) void fwd_wide_kernel(Params p, int n_hblocks) {
  __shared__ __attribute__((aligned(1024))) uint8_t s_lds[kLdsBytes];   // ring | P buffers; at the end the staged outputs
  __shared__ int32_t s_rows[kChunk];
  __shared__ float s_l[8][16], s_m[8][16];                        // per-head row sums / references of each wavefront's 16 heads
  __shared__ float s_inv[4][32];                                  // per-head normalisers of a head group
  __shared__ float s_w[8][16];                                    // split merge: per-row weights of a wavefront's current round
  __shared__ int s_nvalid;
  __shared__ int s_cnt[8];
  __shared__ int s_redo;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c32 = lane & 31, l16 = lane & 15, q4 = lane >> 4;
  const int hg = wave >> 1, x = wave & 1;

  // block id -> (token, split, head block); all workgroups of a token get ids 8 apart (one XCD)
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int hb = slot % n_hblocks;
  const int sp = (slot / n_hblocks) % p.n_splits;
  const int t = token_of(p, xcd, slot / (n_hblocks * p.n_splits));
  if (t >= p.n_tokens) return;
  const int seq = t / p.tokens_per_seq;
  const int head0 = hb * 128 + hg * 32;                           // first head of this wavefront's output rows
  const int hq = head0 + 16 * x + l16;                            // the head this lane scores
  const uint8_t* kv = static_cast<const uint8_t*>(p.kv);
  const int k_begin = sp * p.split_len, k_end = min(k_begin + p.split_len, p.topk);
  const uint32_t ws_magic = *p.ws_header;
  const int per_tile = wave < 2 ? 3 : 2;                          // moves this wavefront issues per tile

  auto load_indices = [&](int c0, int32_t (&rr)[2]) {
    const int c1 = min(c0 + kChunk, k_end);
    const bool listed = p.indices != nullptr;
    const int32_t* base = listed ? p.indices + (size_t)t * p.topk : p.seq_lens + seq;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int j = c0 + 128 * wave + 64 * k + lane;
      const int32_t v = base[listed ? min(j, c1 - 1) : 0];
      rr[k] = j < c1 ? (listed ? v : (j < v ? j : -1)) : -1;
    }
  };
  auto translate2 = [&](int32_t (&rr)[2], const int32_t* bt_row) {
    if (p.block_table != nullptr) {
      int32_t o0 = translate_index(p, rr[0], bt_row), o1 = translate_index(p, rr[1], bt_row);
      rr[0] = o0; rr[1] = o1;
    } else {
      rr[0] = translate_unpaged(p, seq, rr[0]);
      rr[1] = translate_unpaged(p, seq, rr[1]);
    }
  };

  const uint32_t lds0 = hw::lds_addr(&s_lds[0]);
  // ---- page-table row -> LDS (last ring slot, free until the first chunk's row list exists),
  // issued ahead of the index loads so that it has landed once they have
  const int32_t* bt_row = p.block_table ? p.block_table + (size_t)seq * p.bt_stride : nullptr;
  const bool bt_in_lds = bt_row != nullptr && p.bt_stride <= kBtLdsMax && (p.bt_stride & 3) == 0 &&
                         ((uintptr_t)bt_row & 15) == 0;
  const uint32_t lds_bt = lds0 + (kSlots - 1) * kTileBytes;
  if (bt_in_lds) {
    for (int c = wave; 256 * c < p.bt_stride; c += 8) {
      const int e = 256 * c + 4 * lane;
      if (e < p.bt_stride) hw::dma_b128(bt_row + e, lds_bt + 1024 * c);
    }
  }
  int32_t rr_first[2];
  load_indices(k_begin, rr_first);

  // ---- Q^T fragments of this lane's head: B operand of S^T, k = 32 ks + 8 q4 .. + 7.  A head past
  // the end reads head 0 again (its results are never stored); nothing touches the values here, so
  // the compiler does not wait for Q ahead of the row list.
  bf16x8 qf[kDqk / 32];
  {
    const uint16_t* qrow = static_cast<const uint16_t*>(p.q) + ((size_t)t * p.n_heads + (hq < p.n_heads ? hq : 0)) * kDqk + 8 * q4;
#pragma unroll
    for (int ks = 0; ks < kDqk / 32; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
  }
  if (tid == 0) s_redo = 0;
  if (bt_in_lds) {
    hw::wait_for_loads_of(rr_first[0], rr_first[1]);
    __syncthreads();
    translate2(rr_first, reinterpret_cast<const int32_t*>(&s_lds[(kSlots - 1) * kTileBytes]));
  } else {
    translate2(rr_first, bt_row);
  }

  f32x16 acc[kAccTiles];
#pragma unroll
  for (int i = 0; i < kAccTiles; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float m_ref = -INFINITY, l_part = 0.f;      // this lane's head: base-2 reference, partial row sum over its tokens
  const float sc2 = CAP ? 1.f : p.sm_scale * kLog2e;
  [[maybe_unused]] const LogitCap cap(p.sm_scale, CAP ? p.logit_cap : 1.f);
  const uint32_t lds_p = lds0 + kPOff;

  int pass = kPassFast;
  bool first_chunk = true;
  for (;;) {
    bool failed = false;
    bool have_ref = pass == kPassFinal;
    for (int c0 = k_begin; c0 < k_end; c0 += kChunk) {
      // ---- translate + mask + compact the next chunk of the list (order preserving): 8 wavefronts x 128 entries
      __syncthreads();
      {
        int32_t rr[2];
        if (first_chunk) {
          rr[0] = rr_first[0]; rr[1] = rr_first[1];
        } else {
          load_indices(c0, rr);
          translate2(rr, bt_row);
        }
        first_chunk = false;
        const uint64_t m0 = __ballot(rr[0] >= 0), m1 = __ballot(rr[1] >= 0);
        if (lane == 0) s_cnt[wave] = __popcll(m0) + __popcll(m1);
        __syncthreads();
        int base = 0;
#pragma unroll
        for (int w = 0; w < 8; ++w) base += w < wave ? s_cnt[w] : 0;
        const uint64_t below = (1ull << lane) - 1ull;
        if (rr[0] >= 0) s_rows[base + __popcll(m0 & below)] = rr[0];
        base += __popcll(m0);
        if (rr[1] >= 0) s_rows[base + __popcll(m1 & below)] = rr[1];
        if (tid == 0) {
          int n = 0;
#pragma unroll
          for (int w = 0; w < 8; ++w) n += s_cnt[w];
          s_nvalid = n;
        }
      }
      __syncthreads();
      const int n_valid = s_nvalid;
      const int n_tiles = (n_valid + kTN - 1) / kTN;
      if (n_tiles == 0) continue;

      auto tile_addr = [&](int it) { return lds0 + (uint32_t)(it % kSlots) * kTileBytes; };
      // moves of tile `it`: this wavefront's rows 2 wave, 2 wave + 1 (first 1 KB each: scalar row base +
      // lane offset, the row lands swizzled); wavefronts 0, 1 also the RoPE tails of rows 8 wave .. + 7.
      // Rows past the valid count repeat the last valid row (their scores are masked).
      auto fetch = [&](int it) {
        const uint32_t tile = tile_addr(it);
        const int32_t rid = s_rows[min(it * kTN + (lane & 15), n_valid - 1)];   // lane l holds the row id of tile row l % 16
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int r = 2 * wave + j;
          const uint32_t srow = (uint32_t)__builtin_amdgcn_readlane(rid, r);
          const uint64_t sbase = (uint64_t)(uintptr_t)kv + (uint64_t)srow * kRowBytesBf16;
          hw::dma_b128((uint32_t)(lane * 16) ^ (uint32_t)(swz(r) << 4), sbase, tile + r * kMainStride);
        }
        if (wave < 2) {
          // lane l fills slot l of the 1 KB block of row pairs 4 wave .. 4 wave + 3
          const int pair = 4 * wave + (lane >> 4);
          const int r = 2 * pair + ((lane >> 3) & 1), c = (lane & 7) ^ (pair & 7);
          const int32_t trow = __shfl(rid, r);
          hw::dma_b128(kv + (size_t)trow * kRowBytesBf16 + 1024 + c * 16, tile + kRopeBase + wave * 1024);
        }
      };

      // scores + probabilities of tile `it` -> P buffer it & 1
      auto score_tile = [&](int it) {
        const uint32_t tile = tile_addr(it);
        constexpr int kSteps = kDqk / 32, kMainSteps = kDv / 32, kPf = 4;
        const int tr = l16;                                    // A operand: lane's tile row
        const uint32_t kmain = tile + tr * kMainStride + ((q4 ^ swz(tr)) << 4);
        auto frag = [&](int ks) {
          if (ks < kMainSteps) return hw::lds_read_b128((kmain ^ (uint32_t)((ks & 3) << 6)) + (ks >> 2) * 256);
          return hw::lds_read_b128(tile + rope_slot(tr, 4 * (ks - kMainSteps) + q4));
        };
        f32x4 sa[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
        bf16x8 a[kSteps];
#pragma unroll
        for (int ks = 0; ks < kPf; ++ks) a[ks] = frag(ks);
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
          if (ks + kPf < kSteps) a[ks + kPf] = frag(ks + kPf);
          sa[ks & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ks], qf[ks], sa[ks & 1], 0, 0, 0);
        }
        f32x4 s = sa[0] + sa[1];                               // lane: head l16 of my 16, tokens 4 q4 + r
        if constexpr (CAP) {
#pragma unroll
          for (int r = 0; r < 4; ++r) s[r] = cap(s[r]);
        }
        const int my_valid = n_valid - it * kTN;               // valid tokens of the tile (>= 1)
        if (my_valid < kTN) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (4 * q4 + r >= my_valid) s[r] = -INFINITY;
        }
        float mx = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])) * sc2;   // per-lane maximum: enough for the overflow test
        if (!have_ref) {                                       // first tile of the pass (uniform): the head's maximum over the tile
          mx = fmaxf(mx, __shfl_xor(mx, 16));
          mx = fmaxf(mx, __shfl_xor(mx, 32));
          if (pass == kPassFast) m_ref = mx;
          have_ref = true;
        }
        if (pass == kPassMax) m_ref = fmaxf(m_ref, mx);
        if (pass == kPassFast) failed |= __any(mx > m_ref + kSlack);
        float pr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pr[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], sc2, -m_ref));
        l_part += (pr[0] + pr[1]) + (pr[2] + pr[3]);
        const uint32_t pw = lds_p + ((it & 1) * 4 + hg) * kPBytes + (16 * x + l16) * kPStride + 8 * q4;
        hw::lds_write_b64(pw, u32x2{pack_bf16(pr[0], pr[1]), pack_bf16(pr[2], pr[3])});
      };

      // O[32 heads x 256] += P[32 x 16 tok] . V[16 tok x 256] of tile `it`
      auto accumulate_tile = [&](int it) {
        const uint32_t tile = tile_addr(it);
        const int i4 = l16 >> 2;
        const int c_lane = 2 * ((lane >> 4) & 1) + ((l16 & 3) >> 1);
        const uint32_t vbase = tile + (8 * g + i4) * kMainStride + kDvHalf * x * 2 + (i4 << 6) + ((c_lane ^ (2 * g)) << 4) + 8 * (l16 & 1);
        const bf16x8 pa = hw::lds_read_b128(lds_p + ((it & 1) * 4 + hg) * kPBytes + c32 * kPStride + 16 * g);
        constexpr int kPf = 4;
        bf16x4 lo[kAccTiles], hi[kAccTiles];
#pragma unroll
        for (int dt = 0; dt < kPf; ++dt) {
          lo[dt] = hw::lds_read_tr16_b64(vbase ^ (uint32_t)(64 * dt));
          hi[dt] = hw::lds_read_tr16_b64((vbase ^ (uint32_t)(64 * dt + 16)) + 4 * kMainStride);
        }
#pragma unroll
        for (int dt = 0; dt < kAccTiles; ++dt) {
          if (dt + kPf < kAccTiles) {
            lo[dt + kPf] = hw::lds_read_tr16_b64(vbase ^ (uint32_t)(64 * (dt + kPf)));
            hi[dt + kPf] = hw::lds_read_tr16_b64((vbase ^ (uint32_t)(64 * (dt + kPf) + 16)) + 4 * kMainStride);
          }
          const bf16x8 bv = __builtin_shufflevector(lo[dt], hi[dt], 0, 1, 2, 3, 4, 5, 6, 7);
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa, bv, acc[dt], 0, 0, 0);
        }
      };

      // ---- prologue: the first kAhead tiles go out at once
      const int n_pro = min(n_tiles, kAhead);
      for (int it = 0; it < n_pro; ++it) fetch(it);
      wait_moves((n_pro - 1) * per_tile);      // tile 0 has landed (and, loads completing in order, everything older: Q, indices)
#pragma unroll
      for (int ks = 0; ks < kDqk / 32; ++ks) hw::wait_for_loads_of(qf[ks]);   // (tells the compiler that Q is there)
      __syncthreads();
      score_tile(0);
      // ---- one barrier per tile: tile it + 1 is scored while tile `it` is accumulated
      for (int it = 0; it < n_tiles; ++it) {
        const bool next = it + 1 < n_tiles;
        if (next) wait_moves(min(kAhead - 2, n_tiles - (it + 2)) * per_tile);   // tile it + 1 landed; younger ones may be on their way
        __syncthreads();                       // P of tile `it` is there, tile it + 1 landed for everyone, tile it - 1 is consumed
        if (it + kAhead < n_tiles) fetch(it + kAhead);
        if (next) score_tile(it + 1);
        accumulate_tile(it);
      }
    }
    if (pass == kPassFinal) break;
    if (pass == kPassFast) {
      if (failed && lane == 0) s_redo = 1;
      __syncthreads();
      if (s_redo == 0) break;                // the common case
      m_ref = -INFINITY;
      pass = kPassMax;
    } else {
      m_ref = fmaxf(m_ref, __shfl_xor(m_ref, 16));   // exact maximum: fold the four lanes of a head
      m_ref = fmaxf(m_ref, __shfl_xor(m_ref, 32));
      pass = kPassFinal;
    }
    l_part = 0.f;                            // what the void / max pass accumulated is dropped
#pragma unroll
    for (int i = 0; i < kAccTiles; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  }

  // ---- epilogue.  Per-head scalars: every wavefront knows its own 16 heads; the output rows of a
  // wavefront are the 32 heads of its group, so the pair exchanges through LDS.
  __syncthreads();
  if (p.n_splits > 1 && tid == 0) s_nvalid = ws_arrive(p, p.counters + (size_t)t * n_hblocks + hb, ws_magic, p.n_splits, sp);
  {
    float l = l_part;
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (q4 == 0) { s_l[wave][l16] = l; s_m[wave][l16] = m_ref; }
  }
  __syncthreads();
  // lane c32 = output row (head head0 + c32), scored by wavefront 2 hg + c32 / 16
  const float l_tot = s_l[2 * hg + (c32 >> 4)][c32 & 15];
  const float m_run = s_m[2 * hg + (c32 >> 4)][c32 & 15];
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  const float lse_nat = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
  const int head = head0 + c32;
  const bool head_ok = head < p.n_heads;
  if (x == 0 && g == 0) s_inv[hg][c32] = inv;
  const int n_rows = max(0, min(32, p.n_heads - head0));          // output rows that exist (wave-uniform)
  const int col4 = kDvHalf * x + 4 * lane;                         // this lane's 4 output columns when rows are read back
  float* stage = reinterpret_cast<float*>(&s_lds[0]) + wave * 16 * kStageStride;
  auto staged = [&](int row16) { return *reinterpret_cast<const float4*>(stage + row16 * kStageStride + 4 * lane); };
  auto store_bf16x4 = [&](int row, float4 v) {
    uint2 w;
    w.x = pack_bf16(v.x, v.y);
    w.y = pack_bf16(v.z, v.w);
    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + ((size_t)t * p.n_heads + head0 + row) * kDv + col4) = w;
  };
  // the accumulators go through LDS 16 head rows at a time (registers 8 h .. 8 h + 7 hold rows 16 h .. + 15), normalised
  auto stage_half = [&](int h) {
    __syncthreads();                                               // the area is free (ring / previous half consumed)
#pragma unroll
    for (int r = 8 * h; r < 8 * h + 8; ++r) {
      const int row = 8 * ((r >> 2) & 1) + 4 * g + (r & 3);        // row within the half
#pragma unroll
      for (int dt = 0; dt < kAccTiles; ++dt) stage[row * kStageStride + 32 * dt + c32] = acc[dt][r];
    }
    __syncthreads();
    // normalise in place: the very numbers a publisher stores (every lane its own 4 columns of 16 rows)
    for (int row = 0; row < 16; ++row) {
      const float sc = s_inv[hg][16 * h + row];
      float4 v = staged(row);
      v.x = __fmul_rn(v.x, sc); v.y = __fmul_rn(v.y, sc); v.z = __fmul_rn(v.z, sc); v.w = __fmul_rn(v.w, sc);
      *reinterpret_cast<float4*>(stage + row * kStageStride + 4 * lane) = v;
    }
  };

  const int ns = p.n_splits;
  if (ns == 1) {
    if (x == 0 && g == 0 && head_ok) p.lse[(size_t)t * p.n_heads + head] = lse_nat;
    for (int h = 0; h < 2; ++h) {
      stage_half(h);
      for (int row = 0; row < 16; ++row)
        if (16 * h + row < n_rows) store_bf16x4(16 * h + row, staged(row));
    }
    return;
  }

  // ---- split merge inside the launch (protocol and failure handling: ws_arrive / ws_wait_published)
  unsigned long long* word = p.counters + (size_t)t * n_hblocks + hb;
  const int role = s_nvalid;
  auto give_up = [&]() {
    if (x == 0 && g == 0 && head_ok) p.lse[(size_t)t * p.n_heads + head] = __uint_as_float(0x7fc00000u);
  };
  if (role == kRoleError) { give_up(); return; }
  if (role == kRolePublish) {
    if (x == 0 && g == 0 && head_ok)
      __hip_atomic_store(&p.part_lse[((size_t)t * ns + sp) * p.n_heads + head], lse_nat, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    float* o = p.part_out + (((size_t)t * ns + sp) * p.n_heads + head0) * kDv + col4;
    for (int h = 0; h < 2; ++h) {
      stage_half(h);
      for (int row = 0; row < 16; ++row) {
        if (16 * h + row >= n_rows) break;
        const float4 v = staged(row);
        hw::store_b128_agent(o + (size_t)(16 * h + row) * kDv, f32x4{v.x, v.y, v.z, v.w});
      }
    }
    hw::wait_vmcnt<0>();
    __syncthreads();
    if (tid == 0) __hip_atomic_fetch_or(word, 1ull << sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  // last arrival: wait for the others, then fold the normalised partials in split order with every
  // product and sum rounded on its own: the result does not depend on which split arrived last
  if (tid == 0) s_redo = ws_wait_published(p, word, ns, sp) ? 0 : 1;
  __syncthreads();
  if (s_redo != 0) { give_up(); return; }
  auto split_lse = [&](int i) {
    if (i == sp) return lse_nat;
    return head_ok ? __hip_atomic_load(&p.part_lse[((size_t)t * ns + i) * p.n_heads + head], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT)
                   : -INFINITY;
  };
  float m_all = -INFINITY;
  for (int i = 0; i < ns; ++i) m_all = fmaxf(m_all, split_lse(i));
  const float m_safe = m_all == -INFINITY ? 0.f : m_all;
  float w_sum = 0.f;
  for (int i = 0; i < ns; ++i) w_sum = __fadd_rn(w_sum, __expf(split_lse(i) - m_safe));      // exp(-inf) = 0
  const float rw = w_sum > 0.f ? 1.f / w_sum : 0.f;
  if (x == 0 && g == 0 && head_ok)
    p.lse[(size_t)t * p.n_heads + head] = w_sum > 0.f ? m_all + __logf(w_sum) : -INFINITY;
#pragma unroll 1
  for (int h = 0; h < 2; ++h) {
    stage_half(h);
#pragma unroll 1
    for (int r0 = 0; r0 < 16; r0 += 8) {                           // 8 rows per round: 8 loads in flight per lane, 64 KB per workgroup
      f32x4 sum[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) sum[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
      for (int i = 0; i < ns; ++i) {
        const float wi = __fmul_rn(__expf(split_lse(i) - m_safe), rw);   // lane c32 = row c32 of the group
        hw::wave_lds_order();
        if (g == 0 && (c32 >> 4) == h) s_w[wave][c32 & 15] = wi;
        hw::wave_lds_order();
        f32x4 v[8];
        if (i == sp) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float4 a4 = staged(r0 + j);
            v[j] = f32x4{a4.x, a4.y, a4.z, a4.w};
          }
        } else if (n_rows > 16 * h + r0) {
          const hw::buffer_rsrc src = hw::make_rsrc(p.part_out + (((size_t)t * ns + i) * p.n_heads + head0) * kDv);
#pragma unroll
          for (int j = 0; j < 8; ++j)
            v[j] = hw::load_b128_agent(src, (uint32_t)((min(16 * h + r0 + j, n_rows - 1) * kDv + col4) * 4));
        } else {                               // rows past the last head: nothing to read, nothing stored
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float rb = s_w[wave][r0 + j];
#pragma unroll
          for (int c = 0; c < 4; ++c) sum[j][c] = __fadd_rn(sum[j][c], __fmul_rn(v[j][c], rb));
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (16 * h + r0 + j < n_rows) store_bf16x4(16 * h + r0 + j, make_float4(sum[j][0], sum[j][1], sum[j][2], sum[j][3]));
    }
  }
  __syncthreads();
  if (tid == 0) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
}

template <bool CAP>
int launch_impl(const Params& p, hipStream_t s) {
  const int n_hblocks = (p.n_heads + 127) / 128;
  const long long blocks = ((long long)p.n_tokens + 7) / 8 * 8 * n_hblocks * p.n_splits;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return SMLA_EINVAL_SHAPE;
  hipLaunchKernelGGL(fwd_wide_kernel<CAP>, dim3((unsigned)blocks), dim3(kNT), 0, s, p, n_hblocks);
  return hip_status(hipGetLastError());
}

}  // namespace

int launch_fwd_wide(const Params& p, hipStream_t s) {
  return p.logit_cap > 0.f ? launch_impl<true>(p, s) : launch_impl<false>(p, s);
}

}  // namespace smla
