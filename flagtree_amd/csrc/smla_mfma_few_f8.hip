// Sparse-MLA forward over an fp8 KV cache for few heads (<= 16 per workgroup), contracted in fp8 on
// the matrix cores: the records' e4m3 codes are the MFMA operands as they come from the cache.
//
// The other two few-heads kernels turn every record into bf16 (conversion instructions, twice the
// LDS bytes) before any matrix instruction sees it.  Here
//   * raw 656-byte records go global -> LDS by direct moves (no staging registers) into a ring of
//     three 32-record tiles, two tiles ahead of their use;
//   * Q K^T, NoPE part: v_mfma_scale_f32_16x16x128_f8f6f4 with both scales 2^0.  One instruction
//     contracts one 128-column scale block of 16 tokens with 16 heads, so the records' fp32 block
//     scales multiply the instructions' results.  Q is split once per kernel into TWO e4m3 terms per
//     (head, block) with a power-of-two scale: q = s_q (hi + lo).  One term is inside the accuracy
//     bars on inputs of unit scale but not on large or peaked scores; two terms hold the 8
//     significant bits of a bf16 value exactly, so the scores are those of the records' exact
//     values (the other kernels round code * scale to bf16 first).
//     RoPE part: bf16 in the record, bf16 MFMA.
//   * P V: v_mfma_f32_16x16x32_fp8_fp8.  The probabilities times the tokens' block scales are
//     quantised to two e4m3 terms against a per-wavefront power-of-two ceiling R of the scales seen
//     so far (x = 28 p scale / R <= 448; the accumulators hold sums in units of R / 28 and are
//     rescaled when a tile raises R, which scales of one order of magnitude do once).  The V
//     operand needs 8 tokens of one column in a lane while the records hold columns side by side:
//     two transposing 16-bit LDS reads fetch 4 tokens x 2 neighbouring columns each and two byte
//     permutes split them into the operands of the even and the odd column.
// Matrix-core k indices: an MFMA multiplies byte j of lane 16 g + m of A with byte j of lane
// 16 g + n of B, whatever k that pair is called.  Both operands are loaded by the same rule here
// (K and Q: bytes 32 g .. 32 g + 31 of a block; P and V: the tokens 8 g + {0, 2, 4, 6, 1, 3, 5, 7}),
// so the kernel does not depend on the instructions' k numbering, only on the 16 x 16 result layout
// they share with the bf16 instructions: lane l, register r holds D[m = 4 (l / 16) + r][n = l % 16].
//
// Work split as in the column-split kernel (smla_mfma_few_fp8.hip): wavefront w owns output columns
// 128 w .. 128 w + 127 (scale block w) for all tokens; wavefronts 0 and 1 score 16 tokens each.
// 69 KB of LDS and at most 256 registers: two workgroups per compute unit.
#include "smla_common.h"

namespace smla {
namespace {

using hw::bf16x8;
using hw::bf16x4;
using hw::f32x4;
using hw::u32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(8))) int i32x8;

constexpr int kNT = 256;
constexpr int kTN = 32;                       // records per tile, 8 moved by each wavefront
constexpr int kSlots = 3;                     // ring slots
constexpr int kRec = kRowBytesFp8;            // 656: records lie in LDS as in the cache, back to back
constexpr int kTileBytes = kTN * kRec;        // 20 992
constexpr int kWaveBytes = 8 * kRec;          // 5248 = 5 moves of 1 KB + one of 128 bytes
constexpr int kMoves = 6;                     // move instructions per wavefront per tile
constexpr int kChunk = 1024;                  // top-k entries compacted into LDS at a time
constexpr int kPRow = 80;                     // bytes per head row of the probabilities: 32 bf16 + 16 B pad
constexpr float kSlack = 4.f;                 // a probability may exceed 1 by 2^4 before the pass is redone
constexpr float kPTop = 28.f;                 // 28 * 2^4 = 448, the largest e4m3 value
enum { kPassFast = 0, kPassMax = 1, kPassFinal = 2 };
// LDS banks (64 of 4 bytes): a record starts 164 words after the one before, 36 modulo 64.  The
// 16-byte score reads of 16 consecutive records start at 16 different multiples of 4 words: no
// conflict.  The 8-byte transposing reads are served 32 lanes at a time, 32 bytes of each of 8
// records: records two apart start 8 words apart modulo 64, so the reads take the even records
// of 16 and then the odd ones (which is why a lane's 8 tokens come in the order 0 2 4 6 1 3 5 7).

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

// x0 .. x3 -> four e4m3 codes (round to nearest even), x0 in the low byte
__device__ __forceinline__ uint32_t to_e4m3x4(float x0, float x1, float x2, float x3) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(x0, x1, 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(x2, x3, w, true);
  return (uint32_t)w;
}
// the second term of the two-term form: codes of x - value(hi)
__device__ __forceinline__ uint32_t residual_e4m3x4(float x0, float x1, float x2, float x3, uint32_t hi) {
  const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false), b = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
  return to_e4m3x4(x0 - a[0], x1 - a[1], x2 - b[0], x3 - b[1]);
}

// Moves of one wavefront for one tile: its records 8 w .. 8 w + 7, 328 sixteen-byte pieces, piece
// c = 64 i + lane of move i from record c / 41 (a multiply and a shift for c < 328), landing back
// to back.  The sixth move is 8 lanes wide.
struct Mover {
  const uint8_t* kv;
  int32_t rid;
  int wave, lane;
  __device__ __forceinline__ void begin(const uint8_t* kv_, const int32_t* rows, int e0, int n_valid, int wave_, int lane_) {
    kv = kv_; wave = wave_; lane = lane_;
    rid = rows[min(e0 + (lane & 31), n_valid - 1)];       // lane l holds the row id of tile row l % 32 (rows past the end repeat the last one)
  }
  __device__ __forceinline__ void step(int i, uint32_t tile_lds) const {
    const int c = min(64 * i + lane, 8 * 41 - 1);
    const int rec = (c * 1599) >> 16, col = c - 41 * rec;
    const int32_t trow = __shfl(rid, 8 * wave + rec);
    const uint8_t* src = kv + (size_t)trow * kRec + col * 16;
    const uint32_t dst = tile_lds + wave * kWaveBytes + 1024 * i;
    if (i < kMoves - 1) hw::dma_b128(src, dst);
    else hw::dma_b128_first_lanes<8>(src, dst);
  }
};
static_assert((327 * 1599) >> 16 == 7 && (286 * 1599) >> 16 == 6 && (287 * 1599) >> 16 == 7 && (40 * 1599) >> 16 == 0 && (41 * 1599) >> 16 == 1,
              "c / 41 by multiply and shift");

template <bool CAP>
__global__ __launch_bounds__(kNT, 2) void fwd_few_f8_kernel(Params p, int n_hblocks) {
  __shared__ __attribute__((aligned(16))) uint8_t s_ring[kSlots * kTileBytes];   // raw tiles; at the end, the parked outputs
  __shared__ __attribute__((aligned(16))) uint8_t s_p[16 * kPRow];               // probabilities [16 heads][32 tokens] bf16
  __shared__ int32_t s_rows[kChunk];
  __shared__ float s_m[2][16], s_l[2][16], s_f[16];
  __shared__ int s_cnt[4];
  __shared__ int s_nvalid;
  __shared__ int s_flag;
  static_assert(4 * 16 * (128 + 4) * 4 <= kSlots * kTileBytes, "the parked outputs must fit the ring");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q4 = lane >> 4, l16 = lane & 15;

  const int xcd = blockIdx.x & 7, slot_id = blockIdx.x >> 3;
  const int hb = slot_id % n_hblocks;
  const int sp = (slot_id / n_hblocks) % p.n_splits;
  const int t = token_of(p, xcd, slot_id / (n_hblocks * p.n_splits));
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

  // ---- Q of head l16 (a head past the end reads head 0 again; its results are never stored).
  // NoPE part: the 32 values 128 b + 32 q4 .. + 31 of every block b, bf16, to be quantised below;
  // RoPE part: B operand of the bf16 MFMA, k = 512 + 32 ks + 8 q4 + j.
  const uint16_t* qrow = static_cast<const uint16_t*>(p.q) + ((size_t)t * p.n_heads + (head_ok ? head : 0)) * kDqk;
  bf16x8 qraw[4][4];
#pragma unroll
  for (int b = 0; b < 4; ++b)
#pragma unroll
    for (int c = 0; c < 4; ++c) qraw[b][c] = *reinterpret_cast<const bf16x8*>(qrow + 128 * b + 32 * q4 + 8 * c);
  bf16x8 qrope[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) qrope[ks] = *reinterpret_cast<const bf16x8*>(qrow + kDv + 32 * ks + 8 * q4);
  if (tid == 0) s_flag = 0;
  translate_entries4(p, seq, rr_first);

  // Q in two e4m3 terms per (head, block): q = s_q (hi + lo) with s_q the power of two that puts the
  // block's largest magnitude (over its 128 values; four lanes hold 32 each) into [128, 256),
  // hi = e4m3(q / s_q), lo = e4m3(q / s_q - hi).  q is bf16, 8 significant bits, and dividing by a
  // power of two keeps them: hi takes the top 4 and the remainder has at most 4, so the two terms
  // are q EXACTLY for every value within 2^-9 of the block's largest (below that the e4m3
  // subnormal grid cuts bits worth 2^-17 of the largest).  A block whose largest magnitude is
  // below 2^-119 counts as zero.  (Q was sent for right behind the indices and has arrived with them.)
  i32x8 qhi[4], qlo[4];
  float qs[4];
  {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      float v[32];
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) v[8 * c + j] = (float)qraw[b][c][j];
      float am = 0.f;
#pragma unroll
      for (int j = 0; j < 32; ++j) am = fmaxf(am, fabsf(v[j]));
      am = fmaxf(am, __shfl_xor(am, 16));
      am = fmaxf(am, __shfl_xor(am, 32));
      const uint32_t e = (__float_as_uint(am) >> 23) & 0xffu;        // am = 1.m * 2^(e - 127)
      const float inv = e >= 8u ? __uint_as_float((261u - e) << 23) : 0.f;   // 2^(134 - e): am * inv in [128, 256)
      qs[b] = e >= 8u ? __uint_as_float((e - 7u) << 23) : 0.f;      // s_q = 2^(e - 134)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x0 = v[4 * j] * inv, x1 = v[4 * j + 1] * inv, x2 = v[4 * j + 2] * inv, x3 = v[4 * j + 3] * inv;
        const uint32_t hi = to_e4m3x4(x0, x1, x2, x3);
        qhi[b][j] = (int)hi;
        qlo[b][j] = (int)residual_e4m3x4(x0, x1, x2, x3, hi);
      }
    }
  }

  f32x4 acc[8];       // [16 heads x 128 columns of block `wave`], in units of R / 28: reg r = head 4 q4 + r,
                      // acc[nt] = column 32 (nt / 2) + 2 l16 + nt % 2 of the block
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float big_r = 0.f;                          // power of two above every block scale this wavefront has met (wave-uniform)
  float m_ref = -INFINITY, l_run = 0.f;       // base-2 reference (all wavefronts), this scorer's partial row sum (lane = head)
  const float sc2 = CAP ? 1.f : p.sm_scale * kLog2e;
  [[maybe_unused]] const LogitCap cap(p.sm_scale, CAP ? p.logit_cap : 1.f);
  const uint32_t lds_ring = hw::lds_addr(&s_ring[0]);
  const uint32_t lds_p = hw::lds_addr(&s_p[0]);

  int pass = kPassFast;
  for (;;) {
    bool failed = false;
    bool have_ref = pass == kPassFinal;
    for (int c0 = k_begin; c0 < k_end; c0 += kChunk) {
      // ---- translate + mask + compact the next chunk of the top-k list (order preserving)
      __syncthreads();                       // the previous chunk's tiles and row list are no longer read
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

      Mover mv;
      auto issue = [&](int it) {               // all moves of this wavefront for tile `it`, into ring slot it % 3
        mv.begin(kv, s_rows, it * kTN, n_valid, wave, lane);
        const uint32_t dst = lds_ring + (uint32_t)(it % kSlots) * kTileBytes;
#pragma unroll
        for (int i = 0; i < kMoves; ++i) mv.step(i, dst);
      };
      for (int it = 0; it < min(n_tiles, 2); ++it) issue(it);

      for (int it = 0; it < n_tiles; ++it) {
        if (it + 1 < n_tiles) hw::wait_vmcnt<kMoves>(); else hw::wait_vmcnt<0>();     // my part of tile `it` has landed
        __syncthreads();                       // ... and everyone's; everyone is done with tile it - 1 and its probabilities
        if (it + 2 < n_tiles) issue(it + 2);   // into the slot tile it - 1 has left
        const uint32_t tile = lds_ring + (uint32_t)(it % kSlots) * kTileBytes;

        // ---- scores of my 16 tokens (wavefronts 0, 1): S^T[16 tok x 16 heads], lane = head l16, reg r = token 16 wave + 4 q4 + r
        float mx_first = -INFINITY;
        f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
        if (scorer) {
          const uint32_t krow = tile + (uint32_t)(16 * wave + l16) * kRec;
          const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
          f32x4 sacc[5];
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const u32x4 lo = hw::lds_read_u128(krow + 128 * b + 32 * q4), hi = hw::lds_read_u128(krow + 128 * b + 32 * q4 + 16);
            const i32x8 a = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
            sacc[b] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, qhi[b], zero4, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
            sacc[b] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, qlo[b], sacc[b], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
          }
          sacc[4] = zero4;
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
            sacc[4] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hw::lds_read_b128(krow + kFp8RopeOff + 64 * ks + 16 * q4), qrope[ks], sacc[4], 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const u32x4 sw = hw::lds_read_u128(tile + (uint32_t)(16 * wave + 4 * q4 + r) * kRec + kFp8ScaleOff);
            s[r] = sacc[4][r] + sacc[0][r] * (__uint_as_float(sw[0]) * qs[0]) + sacc[1][r] * (__uint_as_float(sw[1]) * qs[1]) +
                   sacc[2][r] * (__uint_as_float(sw[2]) * qs[2]) + sacc[3][r] * (__uint_as_float(sw[3]) * qs[3]);
          }
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
          // P[head l16][tokens 16 wave + 4 q4 .. + 3]
          hw::lds_write_b64(lds_p + l16 * kPRow + (16 * wave + 4 * q4) * 2, hw::u32x2{pack_bf16(pr[0], pr[1]), pack_bf16(pr[2], pr[3])});
        }
        __syncthreads();                       // the probabilities are there

        // ---- O[16 heads x 128] += P[16 x 32 tok] . (scale V)[32 tok x 128], my block's scales folded into P
        {
          const bf16x8 pa = hw::lds_read_b128(lds_p + l16 * kPRow + 16 * q4);          // tokens 8 q4 .. + 7 of head l16
          float sc8[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) sc8[j] = hw::lds_read_f32(tile + (uint32_t)(8 * q4 + j) * kRec + kFp8ScaleOff + 4 * wave);
          float smax = fmaxf(fmaxf(fmaxf(sc8[0], sc8[1]), fmaxf(sc8[2], sc8[3])), fmaxf(fmaxf(sc8[4], sc8[5]), fmaxf(sc8[6], sc8[7])));
          smax = fmaxf(smax, __shfl_xor(smax, 16));
          smax = fmaxf(smax, __shfl_xor(smax, 32));                // the tile's largest scale of my block: the same in every lane
          const float tile_max = __uint_as_float((uint32_t)__builtin_amdgcn_readfirstlane((int)__float_as_uint(smax)));
          if (tile_max > big_r) {                                  // (wave-uniform, rare) raise the ceiling: 2^(exponent + 2) > 2 tile_max
            const float new_r = __uint_as_float((__float_as_uint(tile_max) & 0x7f800000u) + (2u << 23));
            const float down = big_r / new_r;                      // 0 the first time, when the accumulators are 0
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
              for (int r = 0; r < 4; ++r) acc[i][r] *= down;
            big_r = new_r;
          }
          const float c = kPTop / big_r;
          float x[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) x[j] = (float)pa[j] * (sc8[j] * c);
          // operand bytes 0 .. 7 = tokens 8 q4 + {0, 2, 4, 6, 1, 3, 5, 7}: the order the V reads below deliver
          const uint32_t h0 = to_e4m3x4(x[0], x[2], x[4], x[6]), h1 = to_e4m3x4(x[1], x[3], x[5], x[7]);
          const uint32_t l0 = residual_e4m3x4(x[0], x[2], x[4], x[6], h0), l1 = residual_e4m3x4(x[1], x[3], x[5], x[7], h1);
          const long p_hi = (long)(((uint64_t)h1 << 32) | h0), p_lo = (long)(((uint64_t)l1 << 32) | l0);
          // V: inside a group of 16 lanes, lane i supplies the 8 bytes = columns 8 (i % 4) .. + 7 of the group of 32, of
          // token 8 q4 + 2 (i / 4) (+ 1 for the second read), and receives 16-bit element i % 4 of the rows of lanes
          // i / 4 + 4 j: columns 2 i, 2 i + 1 of the four tokens j = 0 .. 3 -- four tokens, two neighbouring columns.
          const uint32_t vbase = tile + (uint32_t)(8 * q4 + 2 * (l16 >> 2)) * kRec + 128 * wave + 8 * (l16 & 3);
#pragma unroll
          for (int cg = 0; cg < 4; ++cg) {
            const bf16x4 ev = hw::lds_read_tr16_b64(vbase + 32 * cg), od = hw::lds_read_tr16_b64(vbase + 32 * cg + kRec);
            const hw::u32x2 e2 = __builtin_bit_cast(hw::u32x2, ev), o2 = __builtin_bit_cast(hw::u32x2, od);
            // bytes (t0 c0, t0 c1, t2 c0, t2 c1), (t4 c0, t4 c1, t6 c0, t6 c1) -> column c0 of tokens 0 2 4 6, column c1 of the same
            const uint32_t e_c0 = __builtin_amdgcn_perm(e2[1], e2[0], 0x06040200u), e_c1 = __builtin_amdgcn_perm(e2[1], e2[0], 0x07050301u);
            const uint32_t o_c0 = __builtin_amdgcn_perm(o2[1], o2[0], 0x06040200u), o_c1 = __builtin_amdgcn_perm(o2[1], o2[0], 0x07050301u);
            const long v_c0 = (long)(((uint64_t)o_c0 << 32) | e_c0), v_c1 = (long)(((uint64_t)o_c1 << 32) | e_c1);
            acc[2 * cg] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(p_hi, v_c0, acc[2 * cg], 0, 0, 0);
            acc[2 * cg + 1] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(p_hi, v_c1, acc[2 * cg + 1], 0, 0, 0);
            acc[2 * cg] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(p_lo, v_c0, acc[2 * cg], 0, 0, 0);
            acc[2 * cg + 1] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(p_lo, v_c1, acc[2 * cg + 1], 0, 0, 0);
          }
        }
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
  // each wavefront parks its normalised [16 heads x 128 columns] block in the (now free) ring, columns in their own order
  constexpr int kOStride = 128 + 4;                                    // floats per parked row
  float* park = reinterpret_cast<float*>(s_ring) + wave * 16 * kOStride;
  const float unit = big_r * (1.f / kPTop);                            // what one unit of the accumulators is worth
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float f = s_f[4 * q4 + r] * unit;
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) park[(4 * q4 + r) * kOStride + 32 * (nt >> 1) + 2 * l16 + (nt & 1)] = acc[nt][r] * f;
  }
  __syncthreads();
  // thread -> (head row = tid / 16, 8 float4 pieces): piece j = columns 64 j + 4 (tid % 16) .. + 3, parked by wavefront j / 2
  const int orow = tid >> 4, ocol = (tid & 15) * 4;
  const bool row_ok = head0 + orow < p.n_heads;
  auto parked = [&](int j) {
    return *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(s_ring) + ((j >> 1) * 16 + orow) * kOStride +
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
  hipLaunchKernelGGL(fwd_few_f8_kernel<CAP>, dim3((unsigned)blocks), dim3(kNT), 0, s, p, n_hblocks);
  return hip_status(hipGetLastError());
}

}  // namespace

int launch_fwd_few_f8(const Params& p, hipStream_t s) {
  return p.logit_cap > 0.f ? launch_impl<true>(p, s) : launch_impl<false>(p, s);
}

}  // namespace smla
