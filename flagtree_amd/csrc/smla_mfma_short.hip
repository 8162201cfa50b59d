// Sparse-MLA forward, MFMA kernel for few heads (<= 16 per workgroup): the memory-bound shape,
// e.g. one GPU's 16-head slice of a 128-head model over an fp8 KV cache.
//
// One workgroup of 4 wavefronts handles (token, block of 16 heads, split of the top-k list).
// Wavefront w owns tokens 16w .. 16w+15 of every 64-token tile and is otherwise independent of its
// siblings: it has its own softmax reference, row sums and [16 heads x 512] accumulator, which
// are merged once at the end.
//   * bf16 rows stream global -> LDS through direct-to-LDS loads into a two-deep ring shared by
//     the workgroup (one barrier per tile).
//   * fp8 records stream through registers, every wavefront its own 16 records of a tile, two
//     tiles in flight; a landed tile is dequantised into the wavefront's private bf16 staging
//     area in LDS: the e4m3 values are converted exactly, the per-128-block fp32 scales multiply
//     the per-block partial scores and the probabilities (all in fp32).  No barrier in the loop.
// Per tile a wavefront computes
//   * S^T[16 tok x 16 heads] = K[16 x 576] . Q^T[576 x 16]   v_mfma_f32_16x16x32_bf16, Q in VGPRs
//   * probabilities per head (lane = head), kept as the A operand of the next product
//   * O[16 heads x 512] += P[16 x 16 tok] . V[16 tok x 512]    v_mfma_f32_16x16x16_bf16, B through
//     transposing LDS reads.
// Register layouts (wave64), q = lane / 16:
//   16x16x32: A lane holds A[m = lane%16][k = 8q .. 8q+7], B lane holds B[k = 8q .. 8q+7][n = lane%16]
//   16x16x16: A lane holds A[m = lane%16][k = 4q .. 4q+3], B lane holds B[k = 4q .. 4q+3][n = lane%16]
//   D (both): lane, reg r holds D[m = 4q + r][n = lane%16]
#include "smla_common.h"

namespace smla {
namespace {

using hw::bf16x8;
using hw::bf16x4;
using hw::short4v;
using hw::f32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr int kNT = 256;
constexpr int kTN = 64;                       // tokens per tile, 16 per wavefront
constexpr int kRowLds = 1168;                 // bf16 row in LDS: 1152 + 16 B pad
constexpr int kChunk = 1024;                  // top-k entries compacted into LDS at a time
constexpr int kDvTiles = kDv / 16;            // 32 accumulator tiles of 16 heads x 16 dv
constexpr float kSlack = 30.f;                // see the softmax reference note below
enum { kPassFast = 0, kPassMax = 1, kPassFinal = 2 };

template <int FMT> struct Geometry;
template <> struct Geometry<SMLA_KV_BF16> {
  static constexpr int kRawRow = kRowLds;                         // ring rows are already bf16 (padded)
  static constexpr int kRingBytes = 2 * kTN * kRowLds;            // 149504
  static constexpr int kStageBytes = 0;
};
template <> struct Geometry<SMLA_KV_FP8_B128> {
  static constexpr int kRawRow = kRowBytesFp8;                    // 656
  static constexpr int kRingBytes = 0;                            // records are streamed through registers, not LDS
  static constexpr int kStageBytes = 2 * 4 * 16 * kRowLds;        // 149504: a 16-row bf16 area per wavefront (the end-of-kernel parking needs 132 KB anyway)
};

__device__ __forceinline__ bf16x4 lds_read_tr(const uint8_t* p) { return hw::lds_read_tr16_b64(p); }
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

// bf16: direct-to-LDS gather of one tile: wave-wide 16-byte loads, the wave's 64 chunks land in 1 KB
// of consecutive LDS at M0; tile = 64 rows x 73 slots (72 data + 1 pad) = 73 wave loads over a
// linear slot space; a lane on a pad slot re-reads the row's last chunk.  Rows past the valid count
// repeat the last valid row (masked later).
__device__ __forceinline__ void dma_tile_bf16(const uint8_t* kv, const int32_t* rows, int e0, int n_valid,
                                              uint32_t tile_lds, int wave, int lane) {
  constexpr int kSlots = kRowLds / 16, kData = kRowBytesBf16 / 16;
  constexpr int kLoads = kTN * kSlots / 64;                       // 73 wave loads per tile
  constexpr int kIters = (kLoads + 3) / 4;
  int32_t r[kIters];
#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    const int s = (4 * i + wave) * 64 + lane;
    r[i] = rows[min(e0 + min(s / kSlots, kTN - 1), n_valid - 1)];
  }
#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    const int s = (4 * i + wave) * 64 + lane;
    const int col = min(s % kSlots, kData - 1);
    const uint8_t* src = kv + (size_t)r[i] * kRowBytesBf16 + col * 16;
    const uint32_t m0v = __builtin_amdgcn_readfirstlane(tile_lds + (4 * i + wave) * 1024);
    if (4 * i + 3 < kLoads || 4 * i + wave < kLoads) {           // wave-uniform
      hw::dma_b128(src, m0v);
    }
  }
}

// fp8: every wavefront streams its own 16 records of a tile through registers.  Direct-to-LDS
// loads accept only a dozen instructions per CU before the issuing wavefront is parked, which with
// one wavefront per SIMD stops its matrix work too; plain loads queue up to 64 deep per wavefront,
// so two tiles (2 x 10.5 KB per wavefront) stay in flight while a third is consumed, and nothing
// needs a workgroup barrier: records, staging area, softmax state and accumulators are private to
// the wavefront.  Eleven 16-byte loads per lane and tile, each uniform in what it fetches:
//   i = 0..7   NoPE codes: lane owns chunk column lane%32 of rows lane/32 + 2i
//   i = 8, 9   RoPE:       lane owns chunk lane%8 of rows lane/8 + 8(i-8)
//   i = 10     the 4 block scales of row lane%16
// They are ordinary loads: the compiler counts them and waits (s_waitcnt vmcnt) exactly where a
// landing register is first read, which also covers any register copies it decides to make.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
constexpr int kFp8Loads = 11;

__device__ __forceinline__ void fp8_issue(const uint8_t* kv, const int32_t* rows, int e0, int n_valid, int lane,
                                          u32x4 (&L)[kFp8Loads]) {
  const int last = n_valid - 1;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint8_t* src = kv + (size_t)rows[min(e0 + (lane >> 5) + 2 * i, last)] * kRowBytesFp8 + (lane & 31) * 16;
    L[i] = *reinterpret_cast<const u32x4*>(src);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint8_t* src = kv + (size_t)rows[min(e0 + (lane >> 3) + 8 * i, last)] * kRowBytesFp8 + kFp8RopeOff + (lane & 7) * 16;
    L[8 + i] = *reinterpret_cast<const u32x4*>(src);
  }
  const uint8_t* src = kv + (size_t)rows[min(e0 + (lane & 15), last)] * kRowBytesFp8 + kFp8ScaleOff;
  L[10] = *reinterpret_cast<const u32x4*>(src);
}

// landed records -> bf16 rows in the wavefront's staging area + its 16 x 4 block scales.
// The e4m3 values are converted exactly (every e4m3 value is a bf16 value; one convert per pair
// with a unit scale); the per-128-block fp32 scales are applied in fp32 where they are cheap:
// to the per-block partial scores and to the probabilities that multiply the block's columns.
__device__ __forceinline__ void fp8_stage(const u32x4 (&L)[kFp8Loads], uint8_t* stage, float4* scales, int lane) {
  const int col = lane & 31, row0 = lane >> 5;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    uint32_t o[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      o[2 * k] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(L[i][k], 1.0f, false));
      o[2 * k + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(L[i][k], 1.0f, true));
    }
    uint4* d4 = reinterpret_cast<uint4*>(stage + (row0 + 2 * i) * kRowLds + col * 32);
    d4[0] = make_uint4(o[0], o[1], o[2], o[3]);
    d4[1] = make_uint4(o[4], o[5], o[6], o[7]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
    *reinterpret_cast<uint4*>(stage + ((lane >> 3) + 8 * i) * kRowLds + kDv * 2 + (lane & 7) * 16) =
        make_uint4(L[8 + i][0], L[8 + i][1], L[8 + i][2], L[8 + i][3]);
  if (lane < 16)
    scales[lane] = make_float4(__uint_as_float(L[10][0]), __uint_as_float(L[10][1]), __uint_as_float(L[10][2]),
                               __uint_as_float(L[10][3]));
}

// Softmax reference: each wavefront takes its heads' maxima over its first 16 tokens as the
// reference and never moves it, so the accumulators are only ever touched by MFMA.
// Probabilities may exceed 1, by at most 2^kSlack; if a later score exceeds the reference by more
// the workgroup redoes its split in two passes (exact maxima, then the accumulation).
template <int FMT, bool CAP>
__global__ __launch_bounds__(kNT) void fwd_short_kernel(Params p, int n_hblocks) {
  using G = Geometry<FMT>;
  __shared__ __attribute__((aligned(16))) uint8_t s_ring[G::kRingBytes + G::kStageBytes];   // ring, then staging
  uint8_t* const s_stage = s_ring + G::kRingBytes;
  __shared__ int32_t s_rows[kChunk];
  __shared__ float4 s_scale[4][16];         // fp8: block scales of each wavefront's 16 rows
  __shared__ float s_m[4][16], s_l[4][16], s_f[4][16];
  __shared__ int s_cnt[4];
  __shared__ int s_nvalid;
  __shared__ int s_flag;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q4 = lane >> 4, l16 = lane & 15;

  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int hb = slot % n_hblocks;
  const int sp = (slot / n_hblocks) % p.n_splits;
  const int t = token_of(p, xcd, slot / (n_hblocks * p.n_splits));
  if (t >= p.n_tokens) return;
  const int seq = t / p.tokens_per_seq;
  const int head0 = hb * 16;
  const int head = head0 + l16;
  const bool head_ok = head < p.n_heads;
  const uint8_t* kv = static_cast<const uint8_t*>(p.kv);
  const WsHead ws_head = ws_read_head(p);    // read long before the split merge needs it

  // ---- the first chunk's index loads go out before anything else: the row list they lead to
  // (index -> page table -> row fetch) is the longest dependent chain of the kernel
  const int k_begin = sp * p.split_len, k_end = min(k_begin + p.split_len, p.topk);
  auto load_indices = [&](int c0, int32_t (&rr)[4]) {
    const int c1 = min(c0 + kChunk, k_end);
    // (branch-free: with an index list every lane loads its entry, without one it loads the
    // sequence length instead; a branch per entry or per mode would make the compiler wait for
    // each load where the branches join, ahead of the Q loads that should overlap them)
    const bool listed = p.indices != nullptr;
    const int32_t* base = listed ? p.indices + (size_t)t * p.topk : p.seq_lens + seq;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int j = c0 + 256 * wave + 64 * k + lane;
      const int32_t v = base[listed ? min(j, c1 - 1) : 0];
      rr[k] = j < c1 ? (listed ? v : (j < v ? j : -1)) : -1;
    }
  };
  auto translate_entries = [&](int32_t (&rr)[4]) { translate_entries4(p, seq, rr); };
  int32_t rr_first[4];
  load_indices(k_begin, rr_first);          // the Q loads below go out while these are in flight
  bool first_chunk = true;

  // ---- Q^T fragments: B operand of S^T, lane = head, k = 32*ks + 8*q4 + j
  bf16x8 qf[kDqk / 32];
  {
    // (every lane loads; a head past the end reads head 0 again and its results are never stored.
    // Nothing touches the values here: a mask would make the compiler wait for Q ahead of the
    // row list, which only needs the index values)
    const uint16_t* qrow = static_cast<const uint16_t*>(p.q) + ((size_t)t * p.n_heads + (head_ok ? head : 0)) * kDqk + 8 * q4;
#pragma unroll
    for (int ks = 0; ks < kDqk / 32; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
  }
  if (tid == 0) s_flag = 0;
  translate_entries(rr_first);               // waits for the index values only; the page lookups overlap the Q loads

  f32x4 acc[kDvTiles];
#pragma unroll
  for (int i = 0; i < kDvTiles; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;     // this wavefront's base-2 reference / partial row sum (lane = head)
  // raw dot product -> base-2 exponent: one multiply, or (logit cap) the squashed score, which
  // already is in base-2 units
  const float sc2 = CAP ? 1.f : p.sm_scale * kLog2e;
  [[maybe_unused]] const LogitCap cap(p.sm_scale, CAP ? p.logit_cap : 1.f);
  const uint32_t lds_ring = hw::lds_addr(&s_ring[0]);
  constexpr int kTileRaw = kTN * G::kRawRow;

  int pass = kPassFast;
  for (;;) {
    bool failed = false;
    bool have_ref = pass == kPassFinal;        // this wavefront has seen a tile in this pass (or needs no reference)
    for (int c0 = k_begin; c0 < k_end; c0 += kChunk) {
      // ---- translate + mask + compact the next chunk of the top-k list (order preserving)
      __syncthreads();
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

      // ---- per-tile math of one wavefront: rows16 = its 16 bf16 rows in LDS (kRowLds apart),
      // scales = their fp8 block scales (fp8 only), my_valid = how many of the 16 exist
      auto tile_math = [&](const uint8_t* rows16, [[maybe_unused]] const float4* scales, int my_valid) {
        // ---- S^T[16 tok x 16 heads]; lane = head l16, its 4 scores are tokens 4*q4 + r.
        // fp8: one accumulator per 128-column block (4 k-steps each) plus one for the RoPE part,
        // combined with the tokens' block scales.
        constexpr int kSteps = kDqk / 32;                            // 18
        constexpr int kPfA = 6;
        [[maybe_unused]] float4 scl[4];                              // fp8: block scales of my 4 tokens, read ahead of the MFMAs
        if constexpr (FMT == SMLA_KV_FP8_B128) {
#pragma unroll
          for (int r = 0; r < 4; ++r) scl[r] = scales[4 * q4 + r];
        }
        const uint8_t* krow = rows16 + l16 * kRowLds + q4 * 16;
        bf16x8 af[kSteps];
#pragma unroll
        for (int ks = 0; ks < kPfA; ++ks) af[ks] = *reinterpret_cast<const bf16x8*>(krow + ks * 64);
        f32x4 sacc[5];
#pragma unroll
        for (int i = 0; i < 5; ++i) sacc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
          if (ks + kPfA < kSteps) af[ks + kPfA] = *reinterpret_cast<const bf16x8*>(krow + (ks + kPfA) * 64);
          const int a = FMT == SMLA_KV_FP8_B128 ? min(ks >> 2, 4) : (ks & 1);     // bf16: two chains
          sacc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[ks], qf[ks], sacc[a], 0, 0, 0);
        }
        f32x4 s;
        if constexpr (FMT == SMLA_KV_FP8_B128) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            s[r] = sacc[4][r] + sacc[0][r] * scl[r].x + sacc[1][r] * scl[r].y + sacc[2][r] * scl[r].z + sacc[3][r] * scl[r].w;
        } else {
          s = sacc[0] + sacc[1];
        }
        if constexpr (CAP) {
#pragma unroll
          for (int r = 0; r < 4; ++r) s[r] = cap(s[r]);
        }
        if (my_valid < 16) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (4 * q4 + r >= my_valid) s[r] = -INFINITY;
        }
        // per-lane maximum: enough for the overflow test; only the first tile (which fixes the
        // reference, common to the four lanes of a head) pays for the cross-lane exchange, and a
        // maximum pass folds a head's lanes when it ends
        float mx = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])) * sc2;
        if (!have_ref) {                                             // wave-uniform
          mx = fmaxf(mx, __shfl_xor(mx, 16));
          mx = fmaxf(mx, __shfl_xor(mx, 32));
          if (pass != kPassMax) m_run = mx;
          have_ref = true;
        }
        if (pass == kPassMax) m_run = fmaxf(m_run, mx);
        if (pass == kPassFast) failed |= __any(mx > m_run + kSlack);
        float pr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          pr[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], sc2, -m_run));
          l_run += pr[r];
        }
        // A operand(s) of P.V: plain probabilities, or per block scale-weighted ones for fp8
        bf16x4 pa[4];
        if constexpr (FMT == SMLA_KV_FP8_B128) {
          pa[0] = __builtin_bit_cast(bf16x4, make_uint2(pack_bf16(pr[0] * scl[0].x, pr[1] * scl[1].x), pack_bf16(pr[2] * scl[2].x, pr[3] * scl[3].x)));
          pa[1] = __builtin_bit_cast(bf16x4, make_uint2(pack_bf16(pr[0] * scl[0].y, pr[1] * scl[1].y), pack_bf16(pr[2] * scl[2].y, pr[3] * scl[3].y)));
          pa[2] = __builtin_bit_cast(bf16x4, make_uint2(pack_bf16(pr[0] * scl[0].z, pr[1] * scl[1].z), pack_bf16(pr[2] * scl[2].z, pr[3] * scl[3].z)));
          pa[3] = __builtin_bit_cast(bf16x4, make_uint2(pack_bf16(pr[0] * scl[0].w, pr[1] * scl[1].w), pack_bf16(pr[2] * scl[2].w, pr[3] * scl[3].w)));
        } else {
          pa[0] = pa[1] = pa[2] = pa[3] = __builtin_bit_cast(bf16x4, make_uint2(pack_bf16(pr[0], pr[1]), pack_bf16(pr[2], pr[3])));
        }

        // ---- O[16 heads x 512] += P . V : B[k = token 4*q4 + j][n = dv] through transposing reads
        const uint8_t* vbase = rows16 + (4 * q4 + (l16 >> 2)) * kRowLds + (4 * (l16 & 3)) * 2;
        constexpr int kPf = 8;               // B fragments in flight
        bf16x4 bv[kDvTiles];
#pragma unroll
        for (int dt = 0; dt < kPf; ++dt) bv[dt] = lds_read_tr(vbase + dt * 32);
#pragma unroll
        for (int dt = 0; dt < kDvTiles; ++dt) {
          if (dt + kPf < kDvTiles) bv[dt + kPf] = lds_read_tr(vbase + (dt + kPf) * 32);
          acc[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4v, pa[dt / 8]),
                                                              __builtin_bit_cast(short4v, bv[dt]), acc[dt], 0, 0, 0);
        }
#pragma unroll
        for (int dt = 0; dt < kPf; ++dt) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#pragma unroll
        for (int dt = 0; dt < kDvTiles; ++dt) {
          if (dt + kPf < kDvTiles) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
      };

      if constexpr (FMT == SMLA_KV_BF16) {
        // bf16: the workgroup gathers 64-row tiles straight into a double-buffered LDS ring
        dma_tile_bf16(kv, s_rows, 0, n_valid, lds_ring, wave, lane);
        for (int it = 0; it < n_tiles; ++it) {
          hw::wait_vmcnt<0>();
          __syncthreads();                   // tile `it` landed; the other ring slot is no longer read
          if (it + 1 < n_tiles)
            dma_tile_bf16(kv, s_rows, (it + 1) * kTN, n_valid, lds_ring + ((it + 1) & 1) * kTileRaw, wave, lane);
          const int my_valid = min(kTN, n_valid - it * kTN) - 16 * wave;    // valid tokens among my 16
          if (my_valid <= 0) continue;       // wave-uniform: nothing of mine in this (last) tile
          tile_math(s_ring + (it & 1) * kTileRaw + 16 * wave * G::kRawRow, nullptr, my_valid);
        }
      } else {
        // fp8: this wavefront's share of the chunk is rows 64*it + 16*wave .. +15, it < n_my; two
        // landing sets alternate, so the loop is unrolled by two and a set is refilled with tile
        // it+2 as soon as tile `it` has been converted out of it
        const int n_my = (n_valid - 16 * wave + kTN - 1) / kTN;             // <= 0: nothing for this wavefront
        uint8_t* stage = s_stage + wave * 16 * kRowLds;
        float4* scales = s_scale[wave];
        u32x4 la[kFp8Loads], lb[kFp8Loads];
        // (every issue is unconditional so that the compiler can count the loads in flight: a
        // tile past the end re-reads the last valid row, which costs a cache hit)
        fp8_issue(kv, s_rows, 16 * wave, n_valid, lane, la);
        fp8_issue(kv, s_rows, kTN + 16 * wave, n_valid, lane, lb);
        for (int it = 0; it < n_my; it += 2) {
          fp8_stage(la, stage, scales, lane);
          hw::wave_lds_order();              // the staged rows are read by other lanes of this wavefront
          fp8_issue(kv, s_rows, (it + 2) * kTN + 16 * wave, n_valid, lane, la);
          tile_math(stage, scales, min(16, n_valid - it * kTN - 16 * wave));
          if (it + 1 >= n_my) break;
          hw::wave_lds_order();              // ... and are overwritten only after all of them have read
          fp8_stage(lb, stage, scales, lane);
          hw::wave_lds_order();
          fp8_issue(kv, s_rows, (it + 3) * kTN + 16 * wave, n_valid, lane, lb);
          tile_math(stage, scales, min(16, n_valid - (it + 1) * kTN - 16 * wave));
          hw::wave_lds_order();
        }
      }
    }
    if (pass == kPassFinal) break;
    if (pass == kPassFast) {
      if (failed && lane == 0) s_flag = 1;
      __syncthreads();
      if (s_flag == 0) break;                // the common case
      m_run = -INFINITY;
      pass = kPassMax;
    } else {
      m_run = fmaxf(m_run, __shfl_xor(m_run, 16));   // fold the four lanes of a head
      m_run = fmaxf(m_run, __shfl_xor(m_run, 32));
      pass = kPassFinal;
    }
    l_run = 0.f;                             // what the void / max pass accumulated is dropped
#pragma unroll
    for (int i = 0; i < kDvTiles; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- merge the four wavefronts: (m, l) per head through LDS, then the weighted accumulators
  __syncthreads();
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  if (q4 == 0) { s_m[wave][l16] = m_run; s_l[wave][l16] = l_run; }
  __syncthreads();
  float m_all = fmaxf(fmaxf(s_m[0][l16], s_m[1][l16]), fmaxf(s_m[2][l16], s_m[3][l16]));
  const float m_safe = m_all == -INFINITY ? 0.f : m_all;
  float l_all = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) l_all += s_l[w][l16] * __builtin_amdgcn_exp2f(s_m[w][l16] - m_safe);   // exp2(-inf) = 0
  const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
  const float lse_nat = l_all > 0.f ? (m_safe + __builtin_amdgcn_logf(l_all)) * kLn2 : -INFINITY;
  if (q4 == 0) s_f[wave][l16] = __builtin_amdgcn_exp2f(m_run - m_safe) * inv;     // my row factors
  __syncthreads();
  // each wavefront parks its scaled [16 x 512] block in the (now free) ring; rows are heads 4*q4 + r
  constexpr int kOStride = kDv + 4;                                    // floats per parked row
  float* park = reinterpret_cast<float*>(s_ring) + wave * 16 * kOStride;
  static_assert(4 * 16 * kOStride * 4 <= G::kRingBytes + G::kStageBytes, "parking area must fit the tile buffers");
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float f = s_f[wave][4 * q4 + r];
#pragma unroll
    for (int dt = 0; dt < kDvTiles; ++dt) park[(4 * q4 + r) * kOStride + 16 * dt + l16] = acc[dt][r] * f;
  }
  __syncthreads();
  // thread -> (head row = tid / 16, 8 float4 columns): sum of the four parked blocks = normalised output
  const int orow = tid >> 4, ocol = (tid & 15) * 4;                    // + 64 * j
  const bool row_ok = head0 + orow < p.n_heads;
  auto summed = [&](int j) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<float*>(s_ring) + (w * 16 + orow) * kOStride + ocol + 64 * j);
      v.x += x.x; v.y += x.y; v.z += x.z; v.w += x.w;
    }
    return v;
  };
  auto store_final = [&](int j, float4 v) {
    uint2 w2;
    w2.x = pack_bf16(v.x, v.y);
    w2.y = pack_bf16(v.z, v.w);
    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + ((size_t)t * p.n_heads + head0 + orow) * kDv + ocol + 64 * j) = w2;
  };
  if (p.n_splits == 1) {
    if (wave == 0 && q4 == 0 && head_ok) p.lse[(size_t)t * p.n_heads + head] = lse_nat;
    if (row_ok) {
#pragma unroll
      for (int j = 0; j < 8; ++j) store_final(j, summed(j));
    }
    return;
  }

  // ---- split merge inside the launch (ticket word per (token, head block): high half arrival
  // count, low half one "published" bit per split; partials move with agent-scope accesses; an
  // illegal word or a wait past the workspace's poll limit flags the workspace and marks the
  // rows' LSE with NaN, see ws_arrive / ws_wait_published).
  const int ns = p.n_splits;
  unsigned long long* word = p.counters + (size_t)t * n_hblocks + hb;
  if (tid == 0) s_nvalid = ws_arrive(p, word, ws_head, ns, sp);
  __syncthreads();
  const int role = s_nvalid;
  auto give_up = [&]() {                     // the workspace was not what it should be: mark the rows (NaN LSE, zero output)
    if (wave == 0 && q4 == 0 && head_ok) p.lse[(size_t)t * p.n_heads + head] = __uint_as_float(0x7fc00000u);
    if (row_ok) {
#pragma unroll
      for (int j = 0; j < 8; ++j) store_final(j, make_float4(0.f, 0.f, 0.f, 0.f));
    }
  };
  if (role == kRoleError) { give_up(); return; }
  if (role == kRolePublish) {
    if (wave == 0 && q4 == 0 && head_ok)
      __hip_atomic_store(&p.part_lse[((size_t)t * ns + sp) * p.n_heads + head], lse_nat, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    if (row_ok) {
      float* o = p.part_out + (((size_t)t * ns + sp) * p.n_heads + head0 + orow) * kDv + ocol;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float4 v = summed(j);
        const f32x4 vv = {v.x, v.y, v.z, v.w};
        hw::store_b128_agent(o + 64 * j, vv);
      }
    }
    hw::wait_vmcnt<0>();
    __syncthreads();
    if (tid == 0) ws_publish(p, word, sp);
    return;
  }
  // last arrival: every other split holds a ticket, so it is running and will publish.  Wait for
  // all of them, then fold the normalised partials in split order with every product and sum
  // rounded on its own (no fused multiply-add): the result does not depend on which split
  // happened to arrive last.  Per-head scalars live in lane = head l16 of every wavefront.
  if (tid == 0) s_flag = ws_wait_published(p, word, ns, sp) ? 0 : 1;
  __syncthreads();
  if (s_flag != 0) { give_up(); return; }
  auto split_lse = [&](int i) {
    if (i == sp) return lse_nat;
    return head_ok ? __hip_atomic_load(&p.part_lse[((size_t)t * ns + i) * p.n_heads + head], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT)
                   : -INFINITY;
  };
  float m_glob = -INFINITY;
  for (int i = 0; i < ns; ++i) m_glob = fmaxf(m_glob, split_lse(i));
  const float m_ref = m_glob == -INFINITY ? 0.f : m_glob;
  float w_sum = 0.f;
  for (int i = 0; i < ns; ++i) w_sum = __fadd_rn(w_sum, __expf(split_lse(i) - m_ref));      // exp(-inf) = 0
  const float rw = w_sum > 0.f ? 1.f / w_sum : 0.f;
  if (wave == 0 && q4 == 0 && head_ok)
    p.lse[(size_t)t * p.n_heads + head] = w_sum > 0.f ? m_glob + __logf(w_sum) : -INFINITY;
  f32x4 sum[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) sum[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int i = 0; i < ns; ++i) {
    const float wi = __fmul_rn(__expf(split_lse(i) - m_ref), rw);
    hw::wave_lds_order();
    if (q4 == 0) s_f[wave][l16] = wi;        // read back by this wavefront only (its LDS accesses complete in order)
    hw::wave_lds_order();
    f32x4 v[8];
    if (i == sp) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float4 a4 = summed(j);
        v[j] = f32x4{a4.x, a4.y, a4.z, a4.w};
      }
    } else {
      const hw::buffer_rsrc src = hw::make_rsrc(p.part_out + (((size_t)t * ns + i) * p.n_heads + head0) * kDv);
      const uint32_t off = (uint32_t)((min(orow, p.n_heads - 1 - head0) * kDv + ocol) * 4);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = hw::load_b128_agent(src, off + 256 * j);
    }
    const float rb = s_f[wave][orow];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int c = 0; c < 4; ++c) sum[j][c] = __fadd_rn(sum[j][c], __fmul_rn(v[j][c], rb));
  }
  if (row_ok) {
#pragma unroll
    for (int j = 0; j < 8; ++j) store_final(j, make_float4(sum[j][0], sum[j][1], sum[j][2], sum[j][3]));
  }
  __syncthreads();
  if (tid == 0) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
}

template <int FMT, bool CAP>
int launch_short_impl(const Params& p, hipStream_t s) {
  const int n_hblocks = (p.n_heads + 15) / 16;
  const long long blocks = ((long long)p.n_tokens + 7) / 8 * 8 * n_hblocks * p.n_splits;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return SMLA_EINVAL_SHAPE;
  hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_short_kernel<FMT, CAP>), dim3((unsigned)blocks), dim3(kNT), 0, s, p, n_hblocks);
  return hip_status(hipGetLastError());
}

}  // namespace

int launch_fwd_short(int kv_format, const Params& p, hipStream_t s) {
  const bool cap = p.logit_cap > 0.f;
  if (kv_format == SMLA_KV_BF16) return cap ? launch_short_impl<SMLA_KV_BF16, true>(p, s) : launch_short_impl<SMLA_KV_BF16, false>(p, s);
  if (kv_format == SMLA_KV_FP8_B128)
    return cap ? launch_short_impl<SMLA_KV_FP8_B128, true>(p, s) : launch_short_impl<SMLA_KV_FP8_B128, false>(p, s);
  return SMLA_EINVAL_SHAPE;
}

}  // namespace smla
