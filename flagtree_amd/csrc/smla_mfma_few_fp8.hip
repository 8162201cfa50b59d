// Sparse-MLA forward over an fp8 KV cache for few heads (<= 16 per workgroup), second design:
// small enough that two workgroups share a compute unit.
//
// The first design (smla_mfma_short.hip) gives every wavefront its own tokens and a whole
// [16 heads x 512] accumulator; merging the four at the end needs 132 KB of LDS and the
// accumulators 128 registers, so one workgroup fills a compute unit and all of them run their
// set-up, their streaming loop and their tail at the same time, the memory idle in two of the three.
// Here the output columns are split instead: wavefront w owns columns 128 w .. 128 w + 127 (one
// scale block of the records) for all tokens, 32 accumulator registers.  Per 32-record tile
//   1. every wavefront converts the 8 records it streamed through registers (two tiles in flight)
//      into one bf16 tile in LDS that the workgroup shares (barrier),
//   2. wavefronts 0 and 1 score 16 tokens each against the 16 heads (v_mfma_f32_16x16x32_bf16, Q in
//      registers, one accumulator per 128-column block so the fp32 block scales apply to partial
//      sums), turn the scores into probabilities and leave them in LDS once per scale block,
//      already multiplied by the token's scale for that block (barrier),
//   3. every wavefront accumulates its column block over the 32 tokens (8 v_mfma_f32_16x16x32_bf16,
//      P from LDS, V through transposing reads of the shared tile) (barrier).
// 48 KB of LDS and at most 256 registers: two workgroups per compute unit, one's barriers, set-up
// and tail filled by the other's work.  Softmax reference, redo passes, split merge: as in the
// other forward kernels.
//
// Register layouts (wave64), q = lane / 16:
//   16x16x32: A lane holds A[m = lane%16][k = 8q .. 8q+7], B lane holds B[k = 8q .. 8q+7][n = lane%16]
//   D: lane, reg r holds D[m = 4q + r][n = lane%16]
#include "smla_common.h"

namespace smla {
namespace {

using hw::bf16x8;
using hw::bf16x4;
using hw::f32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int kNT = 256;
constexpr int kTN = 32;                       // records per tile, 8 streamed by each wavefront
constexpr int kRowLds = 1168;                 // bf16 row in LDS: 1152 + 16 B pad
constexpr int kChunk = 1024;                  // top-k entries compacted into LDS at a time
constexpr int kPRow = 80;                     // bytes per head row of a probability block: 32 bf16 + 16 B pad
constexpr int kPBlock = 16 * kPRow;           // one scale block's probabilities [16 heads][32 tokens]
constexpr int kRecChunks = kRowBytesFp8 / 16; // 41 sixteen-byte pieces per record
constexpr int kLoads = (8 * kRecChunks + 63) / 64;   // 6 loads per lane move a wavefront's 8 records
constexpr float kSlack = 30.f;
enum { kPassFast = 0, kPassMax = 1, kPassFinal = 2 };

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

// Which piece of which of its wavefront's 8 records a lane's i-th load fetches: piece 64 i + lane of
// 8 x 41; the last load's lanes past the end repeat their first piece (every load is unconditional,
// so the compiler can count what is in flight).  Recomputed where it is needed (a multiply and a
// shift: c / 41 = c * 1599 >> 16 for c < 328) rather than held in 18 registers.
struct LoadPlan {
  int lane;
  __device__ __forceinline__ explicit LoadPlan(int lane_) : lane(lane_) {}
  __device__ __forceinline__ bool live(int i) const { return 64 * i + lane < 8 * kRecChunks; }
  __device__ __forceinline__ int piece(int i) const { return live(i) ? 64 * i + lane : lane; }
  __device__ __forceinline__ int rec(int i) const { return (piece(i) * 1599) >> 16; }
  __device__ __forceinline__ int col(int i) const { return piece(i) - kRecChunks * rec(i); }
};
static_assert((327 * 1599) >> 16 == 327 / 41 && (286 * 1599) >> 16 == 6 && (287 * 1599) >> 16 == 7, "c / 41 by multiply and shift");

__device__ __forceinline__ void fp8_issue(const uint8_t* kv, const int32_t* rows, int e0, int n_valid, const LoadPlan& lp,
                                          u32x4 (&L)[kLoads]) {
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const uint8_t* src = kv + (size_t)rows[min(e0 + lp.rec(i), n_valid - 1)] * kRowBytesFp8 + lp.col(i) * 16;
    L[i] = *reinterpret_cast<const u32x4*>(src);
  }
}

// landed pieces -> the shared bf16 tile (rows row0 .. row0 + 7) and the rows' block scales.  e4m3
// values are converted exactly (every e4m3 value is a bf16 value); the scales are applied later, in fp32.
__device__ __forceinline__ void fp8_stage(const u32x4 (&L)[kLoads], const LoadPlan& lp, uint8_t* tile, float4* scales, int row0) {
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    if (!lp.live(i)) continue;
    const int row = row0 + lp.rec(i), col = lp.col(i);
    uint8_t* dst = tile + row * kRowLds;
    if (col < 32) {
      uint32_t o[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        o[2 * k] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(L[i][k], 1.0f, false));
        o[2 * k + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(L[i][k], 1.0f, true));
      }
      uint4* d4 = reinterpret_cast<uint4*>(dst + col * 32);
      d4[0] = make_uint4(o[0], o[1], o[2], o[3]);
      d4[1] = make_uint4(o[4], o[5], o[6], o[7]);
    } else if (col == 32) {
      scales[row] = make_float4(__uint_as_float(L[i][0]), __uint_as_float(L[i][1]), __uint_as_float(L[i][2]),
                                __uint_as_float(L[i][3]));
    } else {
      *reinterpret_cast<uint4*>(dst + kDv * 2 + (col - 33) * 16) = make_uint4(L[i][0], L[i][1], L[i][2], L[i][3]);
    }
  }
}

template <bool CAP>
__global__ __launch_bounds__(kNT, 2) void fwd_few_fp8_kernel(Params p, int n_hblocks) {
  __shared__ __attribute__((aligned(16))) uint8_t s_tile[kTN * kRowLds];      // 37 376 B: the tile; at the end, the parked outputs
  __shared__ __attribute__((aligned(16))) uint8_t s_p[4 * kPBlock];            // probabilities, one block per scale block
  __shared__ float4 s_scale[kTN];
  __shared__ int32_t s_rows[kChunk];
  __shared__ float s_m[2][16], s_l[2][16], s_f[16];
  __shared__ int s_cnt[4];
  __shared__ int s_nvalid;
  __shared__ int s_flag;
  static_assert(4 * 16 * (128 + 4) * 4 <= kTN * kRowLds, "the parked outputs must fit the tile buffer");

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
  const bool scorer = wave < 2;              // wavefronts 0, 1: tokens 16 wave .. + 15 of every tile

  // ---- the first chunk's index loads go out before anything else
  const int k_begin = sp * p.split_len, k_end = min(k_begin + p.split_len, p.topk);
  auto load_indices = [&](int c0, int32_t (&rr)[4]) {
    const int c1 = min(c0 + kChunk, k_end);
    const bool listed = p.indices != nullptr;
    const int32_t* base = listed ? p.indices + (size_t)t * p.topk : p.seq_lens + seq;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int j = c0 + 256 * wave + 64 * k + lane;
      const int32_t v = base[listed ? min(j, c1 - 1) : 0];
      rr[k] = j < c1 ? (listed ? v : (j < v ? j : -1)) : -1;
    }
  };
  int32_t rr_first[4];
  load_indices(k_begin, rr_first);
  bool first_chunk = true;

  // ---- Q^T fragments (every wavefront loads them: register use is per kernel, and it keeps the
  // code free of divergent loads): B operand of S^T, lane = head, k = 32 ks + 8 q4 + j
  bf16x8 qf[kDqk / 32];
  {
    // (a head past the end reads head 0 again and its results are never stored; nothing touches the
    // values here, so the compiler waits for Q where the first MFMA uses it, not ahead of the row list)
    const uint16_t* qrow = static_cast<const uint16_t*>(p.q) + ((size_t)t * p.n_heads + (head_ok ? head : 0)) * kDqk + 8 * q4;
#pragma unroll
    for (int ks = 0; ks < kDqk / 32; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
  }
  if (tid == 0) s_flag = 0;
  translate_entries4(p, seq, rr_first);

  const LoadPlan lp(lane);
  f32x4 acc[8];                               // [16 heads x 128 columns of block `wave`]: reg r = head 4 q4 + r, column 16 nt + l16
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_ref = -INFINITY, l_run = 0.f;       // base-2 reference (all wavefronts), this scorer's partial row sum (lane = head)
  const float sc2 = CAP ? 1.f : p.sm_scale * kLog2e;
  [[maybe_unused]] const LogitCap cap(p.sm_scale, CAP ? p.logit_cap : 1.f);

  int pass = kPassFast;
  for (;;) {
    bool failed = false;
    bool have_ref = pass == kPassFinal;
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

      // ---- one tile: convert (all) | barrier | score (wavefronts 0, 1) | barrier | accumulate (all) | barrier
      auto do_tile = [&](const u32x4 (&L)[kLoads], int it) {
        fp8_stage(L, lp, s_tile, s_scale, 8 * wave);
        __syncthreads();                       // the tile is complete
        float mx_first = -INFINITY;
        f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
        float4 scl[4];
        if (scorer) {
          // S^T[16 tok x 16 heads]; lane = head l16, its 4 scores are tokens 16 wave + 4 q4 + r
          constexpr int kSteps = kDqk / 32, kPfA = 4;
#pragma unroll
          for (int r = 0; r < 4; ++r) scl[r] = s_scale[16 * wave + 4 * q4 + r];
          const uint8_t* krow = s_tile + (16 * wave + l16) * kRowLds + q4 * 16;
          bf16x8 af[kSteps];
#pragma unroll
          for (int ks = 0; ks < kPfA; ++ks) af[ks] = *reinterpret_cast<const bf16x8*>(krow + ks * 64);
          f32x4 sacc[5];
#pragma unroll
          for (int i = 0; i < 5; ++i) sacc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < kSteps; ++ks) {
            if (ks + kPfA < kSteps) af[ks + kPfA] = *reinterpret_cast<const bf16x8*>(krow + (ks + kPfA) * 64);
            const int a = min(ks >> 2, 4);     // one accumulator per 128-column block, one for the RoPE part
            sacc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[ks], qf[ks], sacc[a], 0, 0, 0);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r)
            s[r] = sacc[4][r] + sacc[0][r] * scl[r].x + sacc[1][r] * scl[r].y + sacc[2][r] * scl[r].z + sacc[3][r] * scl[r].w;
          if constexpr (CAP) {
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] = cap(s[r]);
          }
          const int my_valid = n_valid - it * kTN - 16 * wave;      // valid tokens among my 16 (may be <= 0)
          if (my_valid < 16) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (4 * q4 + r >= my_valid) s[r] = -INFINITY;
          }
          mx_first = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])) * sc2;
        }
        if (!have_ref) {                       // first tile of a pass (uniform over the workgroup): agree on the reference
          if (scorer) {
            float mx = mx_first;
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            if (q4 == 0) s_m[wave][l16] = mx;
          }
          __syncthreads();
          if (pass != kPassMax) m_ref = fmaxf(s_m[0][l16], s_m[1][l16]);
          have_ref = true;
        }
        if (scorer) {
          if (pass == kPassMax) m_ref = fmaxf(m_ref, mx_first);
          if (pass == kPassFast) failed |= __any(mx_first > m_ref + kSlack);
          float pr[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            pr[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], sc2, -m_ref));
            l_run += pr[r];
          }
          // P[head l16][tokens 16 wave + 4 q4 .. + 3], once per scale block with the tokens' scales folded in
          uint8_t* pw = s_p + l16 * kPRow + (16 * wave + 4 * q4) * 2;
          *reinterpret_cast<uint2*>(pw + 0 * kPBlock) = make_uint2(pack_bf16(pr[0] * scl[0].x, pr[1] * scl[1].x), pack_bf16(pr[2] * scl[2].x, pr[3] * scl[3].x));
          *reinterpret_cast<uint2*>(pw + 1 * kPBlock) = make_uint2(pack_bf16(pr[0] * scl[0].y, pr[1] * scl[1].y), pack_bf16(pr[2] * scl[2].y, pr[3] * scl[3].y));
          *reinterpret_cast<uint2*>(pw + 2 * kPBlock) = make_uint2(pack_bf16(pr[0] * scl[0].z, pr[1] * scl[1].z), pack_bf16(pr[2] * scl[2].z, pr[3] * scl[3].z));
          *reinterpret_cast<uint2*>(pw + 3 * kPBlock) = make_uint2(pack_bf16(pr[0] * scl[0].w, pr[1] * scl[1].w), pack_bf16(pr[2] * scl[2].w, pr[3] * scl[3].w));
        }
        __syncthreads();                       // the probabilities are there
        // ---- O[16 heads x 128] += P_w[16 x 32 tok] . V[32 tok x 128]: A = P (lane: head l16, tokens 8 q4 .. + 7),
        // B[k = token 8 q4 + j][n = column] through two transposing reads of four tokens each
        {
          const bf16x8 pa = *reinterpret_cast<const bf16x8*>(s_p + wave * kPBlock + l16 * kPRow + 16 * q4);
          const uint8_t* vbase = s_tile + (8 * q4 + (l16 >> 2)) * kRowLds + wave * 256 + (4 * (l16 & 3)) * 2;
#pragma unroll
          for (int h = 0; h < 2; ++h) {        // four column tiles at a time: eight operand registers in flight
            bf16x4 lo[4], hi[4];
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
              lo[nt] = hw::lds_read_tr16_b64(vbase + (4 * h + nt) * 32);
              hi[nt] = hw::lds_read_tr16_b64(vbase + 4 * kRowLds + (4 * h + nt) * 32);
            }
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
              const bf16x8 bv = __builtin_shufflevector(lo[nt], hi[nt], 0, 1, 2, 3, 4, 5, 6, 7);
              acc[4 * h + nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, bv, acc[4 * h + nt], 0, 0, 0);
            }
          }
        }
        __syncthreads();                       // everyone is done reading the tile and the probabilities
      };

      // two landing sets alternate: a set is refilled with tile it + 2 as soon as tile `it` has been converted out of it
      u32x4 la[kLoads], lb[kLoads];
      fp8_issue(kv, s_rows, 8 * wave, n_valid, lp, la);
      fp8_issue(kv, s_rows, kTN + 8 * wave, n_valid, lp, lb);
      for (int it = 0; it < n_tiles; it += 2) {
        do_tile(la, it);
        fp8_issue(kv, s_rows, (it + 2) * kTN + 8 * wave, n_valid, lp, la);
        if (it + 1 >= n_tiles) break;
        do_tile(lb, it + 1);
        fp8_issue(kv, s_rows, (it + 3) * kTN + 8 * wave, n_valid, lp, lb);
      }
    }
    if (pass == kPassFinal) break;
    if (pass == kPassFast) {
      if (failed && lane == 0) s_flag = 1;
      __syncthreads();
      if (s_flag == 0) break;                // the common case
      m_ref = -INFINITY;
      pass = kPassMax;
    } else {
      // exact maxima: fold a head's lanes, combine the two scorers, hand the result to everyone
      m_ref = fmaxf(m_ref, __shfl_xor(m_ref, 16));
      m_ref = fmaxf(m_ref, __shfl_xor(m_ref, 32));
      __syncthreads();
      if (scorer && q4 == 0) s_m[wave][l16] = m_ref;
      __syncthreads();
      m_ref = fmaxf(s_m[0][l16], s_m[1][l16]);
      pass = kPassFinal;
    }
    l_run = 0.f;                             // what the void / max pass accumulated is dropped
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- row sums of the two scorers -> per-head normaliser and LSE (lane = head l16 in every wavefront)
  __syncthreads();
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  if (scorer && q4 == 0) s_l[wave][l16] = l_run;
  __syncthreads();
  const float l_all = s_l[0][l16] + s_l[1][l16];
  const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
  const float m_safe = m_ref == -INFINITY ? 0.f : m_ref;
  const float lse_nat = l_all > 0.f ? (m_safe + __builtin_amdgcn_logf(l_all)) * kLn2 : -INFINITY;
  if (wave == 0 && q4 == 0) s_f[l16] = inv;
  __syncthreads();
  // each wavefront parks its normalised [16 heads x 128 columns] block in the (now free) tile buffer
  constexpr int kOStride = 128 + 4;                                    // floats per parked row
  float* park = reinterpret_cast<float*>(s_tile) + wave * 16 * kOStride;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float f = s_f[4 * q4 + r];
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) park[(4 * q4 + r) * kOStride + 16 * nt + l16] = acc[nt][r] * f;
  }
  __syncthreads();
  // thread -> (head row = tid / 16, 8 float4 pieces): piece j = columns 64 j + 4 (tid % 16) .. + 3, parked by wavefront j / 2
  const int orow = tid >> 4, ocol = (tid & 15) * 4;
  const bool row_ok = head0 + orow < p.n_heads;
  auto parked = [&](int j) {
    return *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(s_tile) + ((j >> 1) * 16 + orow) * kOStride +
                                            64 * (j & 1) + ocol);
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
      for (int j = 0; j < 8; ++j) store_final(j, parked(j));
    }
    return;
  }

  // ---- split merge inside the launch (protocol and failure handling: ws_arrive / ws_wait_published)
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
        const float4 v = parked(j);
        hw::store_b128_agent(o + 64 * j, f32x4{v.x, v.y, v.z, v.w});
      }
    }
    hw::wait_vmcnt<0>();
    __syncthreads();
    if (tid == 0) ws_publish(p, word, sp);
    return;
  }
  if (tid == 0) s_flag = ws_wait_published(p, word, ns, sp) ? 0 : 1;
  __syncthreads();
  if (s_flag != 0) { give_up(); return; }
  // last arrival: fold the normalised partials in split order, every product and sum rounded on its
  // own, so the result does not depend on which split happened to arrive last
  auto split_lse = [&](int i) {
    if (i == sp) return lse_nat;
    return head_ok ? __hip_atomic_load(&p.part_lse[((size_t)t * ns + i) * p.n_heads + head], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT)
                   : -INFINITY;
  };
  float m_glob = -INFINITY;
  for (int i = 0; i < ns; ++i) m_glob = fmaxf(m_glob, split_lse(i));
  const float m_fold = m_glob == -INFINITY ? 0.f : m_glob;
  float w_sum = 0.f;
  for (int i = 0; i < ns; ++i) w_sum = __fadd_rn(w_sum, __expf(split_lse(i) - m_fold));      // exp(-inf) = 0
  const float rw = w_sum > 0.f ? 1.f / w_sum : 0.f;
  if (wave == 0 && q4 == 0 && head_ok)
    p.lse[(size_t)t * p.n_heads + head] = w_sum > 0.f ? m_glob + __logf(w_sum) : -INFINITY;
  f32x4 sum[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) sum[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int i = 0; i < ns; ++i) {
    const float wi = __fmul_rn(__expf(split_lse(i) - m_fold), rw);
    __syncthreads();                          // (s_f: written by wavefront 0, read by all)
    if (wave == 0 && q4 == 0) s_f[l16] = wi;
    __syncthreads();
    f32x4 v[8];
    if (i == sp) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float4 a4 = parked(j);
        v[j] = f32x4{a4.x, a4.y, a4.z, a4.w};
      }
    } else {
      const hw::buffer_rsrc src = hw::make_rsrc(p.part_out + (((size_t)t * ns + i) * p.n_heads + head0) * kDv);
      const uint32_t off = (uint32_t)((min(orow, p.n_heads - 1 - head0) * kDv + ocol) * 4);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = hw::load_b128_agent(src, off + 256 * j);
    }
    const float rb = s_f[orow];
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

template <bool CAP>
int launch_impl(const Params& p, hipStream_t s) {
  const int n_hblocks = (p.n_heads + 15) / 16;
  const long long blocks = ((long long)p.n_tokens + 7) / 8 * 8 * n_hblocks * p.n_splits;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return SMLA_EINVAL_SHAPE;
  hipLaunchKernelGGL(fwd_few_fp8_kernel<CAP>, dim3((unsigned)blocks), dim3(kNT), 0, s, p, n_hblocks);
  return hip_status(hipGetLastError());
}

}  // namespace

int launch_fwd_few_fp8(const Params& p, hipStream_t s) {
  return p.logit_cap > 0.f ? launch_impl<true>(p, s) : launch_impl<false>(p, s);
}

}  // namespace smla
