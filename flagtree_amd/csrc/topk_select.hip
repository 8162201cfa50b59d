// Top-k index producer: for every row of a score matrix, the indices of its k largest entries.
//
// This is the step that feeds the sparse-MLA forward its index lists.  One workgroup per row;
// wavefront w owns the contiguous segment w of the row, so "index order" is wavefront order and
// nothing but the histogram merge needs a workgroup barrier:
//   1. radix select on an order-preserving 32-bit key (four passes of 8 bits): a 256-bin histogram
//      in LDS with several copies of every bin (score exponents are heavily skewed: plain bins
//      would serialise whole wavefronts on a few LDS words), the copies are summed, and wavefront
//      0 walks the bins from the top for the digit that holds the k-th largest entry;
//   2. every entry above the selected key is taken, plus the first `need` entries equal to it
//      (ties go to the lower index); the list is written in ascending index order and padded with -1.
// Rows of up to 65 536 entries are read once and their keys kept in registers (16 or 64 per lane)
// through all passes (topk_resident_kernel); longer rows are walked from memory in every pass
// and stay in L2 between them (topk_stream_kernel).
// Entries at or past the row's context length do not take part; NaN ranks with -inf.
//
// Few long rows (fewer rows than half the compute units, given a workspace): a row is cut into
// parts of equal length, one workgroup each, and every part selects ITS k largest entries by the
// same rule (topk_part_kernel).  An entry of the row's answer is in its part's answer: if it were
// not, k entries of the part would rank ahead of it, and so would they in the row.  The parts'
// answers (key and index of every entry, in index order, parts in index order) are one candidate
// list per row in the workspace, still in ascending index order, and a second launch selects the
// row's k largest from it, again by the same rule, reading the indices through the list
// (topk_merge_kernel).  Ties at the k-th value go to the candidate that comes first, which is the
// one of lower index: the answer is the same list, entry for entry, as one workgroup gives.
#include "smla_common.h"

namespace smla {
namespace {

// larger float <-> larger key.  x + 0 turns -0 into +0 (they compare equal) and max(., -inf)
// turns NaN into -inf (v_max_f32 returns the operand that is a number), so NaN ranks with -inf.
__device__ __forceinline__ uint32_t score_key(float x) {
  const uint32_t u = __float_as_uint(__builtin_fmaxf(x + 0.0f, -INFINITY));
  return u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
}

// Walks a wavefront's segment in index order, 256 entries per step (lane l holds entries
// 4l .. 4l+3 of the step), with kBatch (8 for long rows, 4 for short ones) 16-byte loads in flight per lane: a load-use-load-use loop
// would pay a full memory latency per step, and with one workgroup per row the bytes in flight per
// CU are what bounds a pass.  f(i0, keys, n_live) is called once per step with the index of the
// lane's first entry, its four keys and how many of them exist (0..4); steps are wave-uniform, so f
// may use cross-lane operations.  `vec` = the row may be read 16 bytes at a time.
struct Keys4 { uint32_t k[4]; };
template <int kBatch, typename F>
__device__ __forceinline__ void walk_segment(const float* __restrict__ x, int seg0, int seg1, int lane, bool vec, F f) {
  for (int base = seg0; base < seg1; base += 256 * kBatch) {
    float4 v[kBatch];
    if (vec && base + 256 * kBatch <= seg1) {   // wave-uniform: a whole batch of straight-line 16-byte loads
#pragma unroll
      for (int j = 0; j < kBatch; ++j) v[j] = *reinterpret_cast<const float4*>(x + base + 256 * j + 4 * lane);
    } else {
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int i = base + 256 * j + 4 * lane;
        v[j].x = i < seg1 ? x[i] : 0.f;
        v[j].y = i + 1 < seg1 ? x[i + 1] : 0.f;
        v[j].z = i + 2 < seg1 ? x[i + 2] : 0.f;
        v[j].w = i + 3 < seg1 ? x[i + 3] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = base + 256 * j + 4 * lane;
      if (base + 256 * j < seg1) {              // wave-uniform
        Keys4 q;
        q.k[0] = score_key(v[j].x); q.k[1] = score_key(v[j].y); q.k[2] = score_key(v[j].z); q.k[3] = score_key(v[j].w);
        f(i, q, max(0, min(4, seg1 - i)));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Rows of up to 65 536 entries: read once, keys held in registers for every pass.
//
// What bounds this kernel is the instruction count per entry and per pass (a wavefront's vector
// instruction takes four cycles; with many short rows a CU's issue slots are the limit, with few
// long rows the LDS atomics of the first pass are), so:
//  * A wavefront owns a contiguous segment of the row and handles it in rounds of 1024 entries.
//    The entries are loaded 16 bytes a lane (whole lines) and turned through LDS so that lane l
//    holds the 16 consecutive entries 16 l .. 16 l + 15 of the round.  Index order is then
//    (wavefront, round, lane, entry): which entries are selected is one 16-bit mask per lane and
//    round, output positions are a prefix sum over the masks' population counts, and every lane
//    writes out its own set bits; no per-entry cross-lane work anywhere.
//  * An entry past the segment's end gets key 0, which no real entry has (the smallest real key,
//    that of -inf, is 0x007fffff), so no pass needs a liveness test: key 0 falls into the lowest
//    bin of every pass and is never above or equal to the selected key, and the count of real
//    entries in the bins looked at is never below what is still to be found.
//  * After two passes (16 key bits fixed) few entries usually still match: they are collected in
//    LDS (four entries tested at a time, the group skipped when no lane has a match) and either
//    ranked directly (up to 64) or histogrammed from the list (up to 1024); only heavily tied
//    rows run passes 2 and 3 over every entry.
//  * The output list is put together in LDS and copied out in whole lines when it fits.

// Inclusive prefix sum over the 64 lanes in data-parallel-primitive moves (a shuffle through the
// LDS crossbar costs several instructions and its latency per step): shifts by 1, 2, 4, 8 inside
// each row of 16 lanes, then row 0's and 2's last lane added to the row above, then lane 31 to
// the upper half.  Lanes without a source add 0.
__device__ __forceinline__ uint32_t wave_prefix_sum(uint32_t v) {
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);   // row_shr:1
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);   // row_shr:2
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);   // row_shr:4
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);   // row_shr:8
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
  return v;
}

constexpr int kRound = 1024;                    // entries of a wavefront's round
constexpr int kFewCandidates = 64;              // up to this many entries in the selected 16-bit bin: ranked directly
constexpr int kListCandidates = 1024;           // up to this many: passes 2 and 3 run over a list of them, not over every entry
constexpr int kRoundWords = kRound + kRound / 4;              // LDS words to turn one round: 16 bytes of padding every 64

// Loads one round of a wavefront's segment, 16 bytes a lane: q[s] = entries base + 256 s + 4 lane ..
// + 3.  The addresses are clamped into the row (no load sits behind a branch); what a slot past
// the row's end holds is not used.
__device__ __forceinline__ void load_round(const float* __restrict__ x, int n, int base, int lane, bool vec, float4 (&q)[4]) {
  if (vec && n >= 4) {
    const int last4 = (n - 4) & ~3;             // the last whole 16-byte group of the row
#pragma unroll
    for (int s = 0; s < 4; ++s) q[s] = *reinterpret_cast<const float4*>(x + min(base + 256 * s + 4 * lane, last4));
    if (n & 3) {                                // the row's last, partial group: re-read by the lane that holds it
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int i = base + 256 * s + 4 * lane;
        if (i > last4 && i < n) { q[s].x = x[i]; q[s].y = x[min(i + 1, n - 1)]; q[s].z = x[min(i + 2, n - 1)]; }
      }
    }
  } else {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int i = base + 256 * s + 4 * lane;
      q[s].x = x[min(i, n - 1)]; q[s].y = x[min(i + 1, n - 1)]; q[s].z = x[min(i + 2, n - 1)]; q[s].w = x[min(i + 3, n - 1)];
    }
  }
}

// Turns a loaded round through the wavefront's own LDS area (kRoundWords words): on return v[j] =
// entry base + 16 lane + j.  Entry p of the round lives at word p + 4 (p / 16): lane l's 64-byte
// run starts 80 bytes after lane l - 1's, which spreads the 16-byte reads of 16 lanes over all banks.
__device__ __forceinline__ void turn_round(const float4 (&q)[4], int lane, float* turn, float (&v)[16]) {
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int p = 256 * s + 4 * lane;
    *reinterpret_cast<float4*>(turn + p + 4 * (p >> 4)) = q[s];
  }
  __builtin_amdgcn_wave_barrier();              // (a wavefront's LDS operations complete in order)
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float4 t = *reinterpret_cast<const float4*>(turn + 20 * lane + 4 * j);
    v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w;
  }
  __builtin_amdgcn_wave_barrier();
}

// What a selection reads and writes:
//   kWhole  scores of a whole row -> the row's answer (indices)
//   kPart   scores of one part of a row -> the part's answer as candidates (key and index of each)
//   kMerge  a row's candidate keys (entry j of `x` is a key's bit pattern, never 0) -> the row's
//           answer, entry j standing for index cand_idx[j]
enum { kWhole = 0, kPart = 1, kMerge = 2 };
template <int MODE>
__device__ __forceinline__ uint32_t key_of(float x) {
  if constexpr (MODE == kMerge) return __float_as_uint(x);
  else return score_key(x);
}

// R = rounds a wavefront can hold (16 R keys a lane); `n` entries at x (up to 1024 R WAVES), the
// `want` largest wanted.  Entry i stands for index index0 + i (kWhole, kPart) or cand_idx[i]
// (kMerge).  The answer goes to o[0 .. want) (kWhole, kMerge) or, key and index, to cand_key_out /
// cand_idx_out[0 .. want) (kPart).
// `bt_row` (kWhole, kMerge): null, or the page-table row of the row's sequence; the answer is then
// written as physical rows of the paged cache (-1 where the table masks a position).
template <int WAVES, int R, int MODE>
__device__ __forceinline__ void resident_select(const float* __restrict__ x, int n, int want, int index0,
                                                const int32_t* __restrict__ cand_idx, int32_t* __restrict__ o,
                                                uint32_t* __restrict__ cand_key_out, int32_t* __restrict__ cand_idx_out,
                                                const int32_t* __restrict__ bt_row, const TopkPaging& pg) {
  constexpr int kThreads = 64 * WAVES;
  // copies of every histogram bin, picked by lane % kCopies: score exponents are heavily skewed,
  // and lanes adding to one LDS word serialise.  A workgroup of 16 wavefronts has the LDS for one
  // copy per lane (its rounds' turning areas are larger than that), which makes the adds of a
  // wavefront free of conflicts altogether.
  constexpr int kCopies = WAVES >= 16 ? 64 : 16;
  constexpr int kHistWords = 256 * kCopies;
  constexpr int kRawWords = WAVES * kRoundWords > kHistWords ? WAVES * kRoundWords : kHistWords;
  // s_raw is, in turn: the wavefronts' areas for turning the loaded rounds; the histogram; the output list
  __shared__ __align__(16) uint32_t s_raw[kRawWords];
  __shared__ uint32_t s_sum[256];
  __shared__ uint32_t s_prefix, s_need;         // key bits fixed so far, entries still to find at / below them
  __shared__ uint32_t s_tot[2 * WAVES];         // entries above / equal to the selected key per wavefront
  __shared__ uint32_t s_bin, s_ncand;           // entries in the bin the last merge chose; candidates collected so far
  __shared__ uint32_t s_ckey[kListCandidates];
  uint32_t (*s_hist)[kCopies] = reinterpret_cast<uint32_t (*)[kCopies]>(s_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (want == 0) return;
  const bool vec = ((uintptr_t)x & 15) == 0;

  // this wavefront's segment [seg0, seg1): whole 256-entry steps, at most R rounds
  const int seg_len = ((n + WAVES - 1) / WAVES + 255) & ~255;
  const int seg0 = min(wave * seg_len, n), seg1 = min(seg0 + seg_len, n);
  const int n_rounds = __builtin_amdgcn_readfirstlane((seg1 - seg0 + kRound - 1) / kRound);

  uint32_t key[R][16];
  float4 loaded[R][4];                          // every round's loads are in flight before the first is turned
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (r < n_rounds) load_round(x, n, seg0 + kRound * r, lane, vec, loaded[r]);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r < n_rounds) {
      float v[16];
      turn_round(loaded[r], lane, reinterpret_cast<float*>(s_raw) + wave * kRoundWords, v);
      const int i0 = seg0 + kRound * r + 16 * lane;
      if (seg0 + kRound * (r + 1) <= seg1) {    // wave-uniform: a full round needs no liveness test
#pragma unroll
        for (int j = 0; j < 16; ++j) key[r][j] = key_of<MODE>(v[j]);
      } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) key[r][j] = i0 + j < seg1 ? key_of<MODE>(v[j]) : 0u;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 16; ++j) key[r][j] = 0u;
    }
  }

  // ---- 1. the key of the want-th largest entry
  if (tid == 0) { s_prefix = 0u; s_need = (uint32_t)want; }
  const uint32_t copy = lane & (kCopies - 1);
  // sums the bins' copies and fixes the next 8 bits of the selected key (wavefront 0)
  auto merge_and_find = [&](int shift, uint32_t prefix) {
    __syncthreads();
    constexpr int kParts = kCopies / 16;        // threads that share a bin, 16 copies each
    for (int i = tid; i < 256 * kParts; i += kThreads) {
      // 16 bytes at a time, starting at a quarter that differs between the lanes that share banks
      const int b = i / kParts, part = i % kParts;
      const int turn = kParts == 1 ? b >> 2 : b;
      uint32_t t = 0;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint4 h = *reinterpret_cast<const uint4*>(&s_hist[b][16 * part + 4 * ((q + turn) & 3)]);
        t += h.x + h.y + h.z + h.w;
      }
      if constexpr (kParts == 4) {              // the four lanes of a bin: quad_perm [1,0,3,2], then [2,3,0,1]
        t += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0xb1, 0xf, 0xf, false);
        t += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x4e, 0xf, 0xf, false);
      }
      if (part == 0) s_sum[b] = t;
    }
    __syncthreads();
    if (wave == 0) {
      // digit d (from the top) where the count of entries with a larger digit is < need <= that + hist[d];
      // lane l looks after digits 255 - 4l .. 252 - 4l
      const uint32_t need = s_need;
      uint32_t h[4], sum = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) { h[j] = s_sum[255 - 4 * lane - j]; sum += h[j]; }
      const uint32_t incl = wave_prefix_sum(sum);
      uint32_t above = incl - sum;              // entries with a digit above this lane's four
      if (above < need && need <= incl) {       // exactly one lane
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (above < need && need <= above + h[j]) {
            s_prefix = prefix | ((uint32_t)(255 - 4 * lane - j) << shift);
            s_need = need - above;
            s_bin = h[j];
            above = 0xffffffffu;                // done
          } else if (above != 0xffffffffu) {
            above += h[j];
          }
        }
      }
    }
  };
  auto clear_histogram = [&]() {
    for (int j = 4 * tid; j < kHistWords; j += 4 * kThreads) *reinterpret_cast<uint4*>(&s_raw[j]) = make_uint4(0u, 0u, 0u, 0u);
    __syncthreads();                            // (also publishes s_prefix / s_need of the previous pass)
  };

  // pass 0: every entry counts (outside the loop over the later passes: inside it, the bin
  // addresses would be hoisted out of the loop as invariants, and 64 keys leave no registers for them)
  __syncthreads();                              // every wavefront is done turning its rounds
  clear_histogram();
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (r < n_rounds) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        atomicAdd(&s_hist[key[r][j] >> 24][copy], 1u);
        if ((j & 3) == 3) __builtin_amdgcn_sched_barrier(0);  // (nor may the scheduler compute every address up front)
      }
    }
  merge_and_find(24, 0u);

  // pass 1: entries whose top 8 bits match
  {
    if (tid == 0) s_ncand = 0u;
    clear_histogram();
    const uint32_t prefix = s_prefix;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (r < n_rounds) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const uint32_t d = key[r][j] ^ prefix;
          if (d < (1u << 24)) atomicAdd(&s_hist[d >> 16][copy], 1u);
          if ((j & 3) == 3) __builtin_amdgcn_sched_barrier(0);
        }
      }
    merge_and_find(16, prefix);
  }
  __syncthreads();
  const uint32_t n_bin = s_bin;
  if (n_bin <= (uint32_t)kListCandidates) {
    // Few entries share the 16 bits fixed so far (the usual case for scores that are not heavily
    // quantised): instead of two more histogram passes over every entry, the candidates' keys are
    // collected (their order does not matter).  Up to 64 of them: wavefront 0 finds the s_need-th
    // largest by counting, for every candidate, the candidates above it.  More: passes 2 and 3
    // run over the list.
    const uint32_t prefix = s_prefix;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (r < n_rounds) {
#pragma unroll
        for (int j4 = 0; j4 < 16; j4 += 4) {
          uint32_t d[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) d[c] = key[r][j4 + c] ^ prefix;
          if (__ballot(min(min(d[0], d[1]), min(d[2], d[3])) < (1u << 16)) != 0ull) {   // wave-uniform
#pragma unroll
            for (int c = 0; c < 4; ++c)
              if (d[c] < (1u << 16)) s_ckey[atomicAdd(&s_ncand, 1u)] = key[r][j4 + c];
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    __syncthreads();
    if (n_bin > (uint32_t)kFewCandidates) {
      for (int pass = 2; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        clear_histogram();
        const uint32_t fixed = s_prefix;
        const uint32_t lim = 1u << (shift + 8);
        for (uint32_t c = tid; c < n_bin; c += kThreads) {
          const uint32_t d = s_ckey[c] ^ fixed;
          if (d < lim) atomicAdd(&s_hist[d >> shift][copy], 1u);
        }
        merge_and_find(shift, fixed);
      }
    } else if (wave == 0) {
      const int n_cand = (int)s_ncand;          // == n_bin
      const int need = (int)s_need;
      const uint32_t mine = lane < n_cand ? s_ckey[lane] : 0u;
      int n_above = 0;
      for (int m = 0; m < n_cand; ++m) n_above += s_ckey[m] > mine ? 1 : 0;
      // the need-th largest is the smallest candidate with fewer than `need` candidates above it
      uint32_t v = (lane < n_cand && n_above < need) ? mine : 0xffffffffu;
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) v = min(v, (uint32_t)__shfl_xor((int)v, d));
      const unsigned long long holders = __ballot(lane < n_cand && mine == v);
      const int first = __builtin_ctzll(holders);
      const int above_v = __shfl(n_above, first);
      if (lane == 0) { s_prefix = v; s_need = (uint32_t)(need - above_v); }
    }
  } else {
    for (int pass = 2; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      clear_histogram();
      const uint32_t prefix = s_prefix;
      const uint32_t lim = 1u << (shift + 8);   // key ^ prefix < lim <=> the bits fixed so far match
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (r < n_rounds) {
#pragma unroll
          for (int j4 = 0; j4 < 16; j4 += 4) {
            uint32_t d[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) d[c] = key[r][j4 + c] ^ prefix;
            if (__ballot(min(min(d[0], d[1]), min(d[2], d[3])) < lim) != 0ull) {    // wave-uniform
#pragma unroll
              for (int c = 0; c < 4; ++c)
                if (d[c] < lim) atomicAdd(&s_hist[d[c] >> shift][copy], 1u);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      merge_and_find(shift, prefix);
    }
  }
  __syncthreads();
  const uint32_t thr = s_prefix;
  const int need_eq = (int)s_need;              // entries equal to thr that are taken (the lowest indices)

  // ---- 2. per lane and round: which entries are above / equal to the selected key, how many
  uint32_t above[R], equal[R];                  // 16-bit masks, bit j = entry j of the lane's run
  int n_above = 0, n_equal = 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    uint32_t a = 0, e = 0;
    if (r < n_rounds) {
#pragma unroll
      for (int j = 15; j >= 0; --j) {
        // mask = 2 mask + (compare): a compare into vcc and an add with carry-in, two vector
        // instructions a bit (the compiler's own lowering takes three and a half); the wait state
        // between a vcc write and its use as carry-in is spelled out
        hw::shift_in_gt_u32(a, key[r][j], thr);
        hw::shift_in_eq_u32(e, key[r][j], thr);
      }
    }
    above[r] = a; equal[r] = e;
    n_above += __popc(a); n_equal += __popc(e);
  }
  // entries above / equal before this wavefront's: totals of the wavefronts below
  {
    const uint32_t ta = wave_prefix_sum((uint32_t)n_above), te = wave_prefix_sum((uint32_t)n_equal);
    if (lane == 63) { s_tot[2 * wave] = ta; s_tot[2 * wave + 1] = te; }
  }
  __syncthreads();
  int above_before = 0, equal_before = 0;
  for (int w = 0; w < wave; ++w) { above_before += (int)s_tot[2 * w]; equal_before += (int)s_tot[2 * w + 1]; }

  // ---- 3. write the selected entries out in ascending order: (round, lane, entry) within the
  // wavefront.  Neighbouring lanes' outputs lie a few entries apart, so when the list fits the LDS
  // it is put together there (as positions in x) and copied out in whole lines.  What a position
  // stands for is looked up on the way out: the index itself, the candidate's index, or (a part's
  // answer) index and key, the key recomputed from the score, which is in L2.
  int32_t* s_list = reinterpret_cast<int32_t*>(s_raw);
  const bool staged = want <= kRawWords;
  auto emit = [&](int at, int pos) {
    if constexpr (MODE == kPart) {
      cand_idx_out[at] = index0 + pos;
      cand_key_out[at] = score_key(x[pos]);
    } else {
      const int32_t idx = MODE == kWhole ? index0 + pos : cand_idx[pos];
      o[at] = bt_row == nullptr ? idx : paged_row(idx, bt_row, pg.bt_stride, pg.page_size, pg.kv_rows);
    }
  };
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r < n_rounds) {
      // inclusive prefix over the lanes of this round's counts, both packed in one word (a
      // wavefront's round holds at most 1024 of either)
      const uint32_t mine = (uint32_t)__popc(above[r]) | ((uint32_t)__popc(equal[r]) << 16);
      const uint32_t incl = wave_prefix_sum(mine);
      const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
      const int a_before = above_before + (int)((incl - mine) & 0xffffu);
      const int e_before = equal_before + (int)((incl - mine) >> 16);
      // ties: the first need_eq in index order are taken (signed arithmetic on purpose: with
      // unsigned operands the compiler marks need_eq - e_before as never wrapping and then treats
      // min(e_before, need_eq) as e_before)
      const int take = max(0, min(need_eq - e_before, __popc(equal[r])));
      uint32_t eq = equal[r];
      while (__popc(eq) > take) eq &= ~(0x80000000u >> __builtin_clz(eq));          // drop the highest
      uint32_t sel = above[r] | eq;
      int at = a_before + min(e_before, need_eq);
      const int i0 = seg0 + kRound * r + 16 * lane;
      while (sel != 0u) {
        const int j = __builtin_ctz(sel);
        if (staged) s_list[at] = i0 + j;
        else emit(at, i0 + j);
        ++at;
        sel &= sel - 1u;
      }
      above_before += (int)(total & 0xffffu);
      equal_before += (int)(total >> 16);
    }
  }
  if (staged) {
    __syncthreads();
    for (int j = tid; j < want; j += kThreads) emit(j, s_list[j]);
  }
}

template <int WAVES, int R>
__global__ __launch_bounds__(64 * WAVES) void topk_resident_kernel(const float* __restrict__ scores,
                                                                  const int32_t* __restrict__ context_lens,
                                                                  int32_t* __restrict__ out, int n_cols,
                                                                  long long row_stride, int k, TopkPaging pg) {
  const int row = blockIdx.x;
  const int n = context_lens ? max(0, min(context_lens[row], n_cols)) : n_cols;
  const int want = min(k, n);                   // entries to select
  int32_t* o = out + (size_t)row * k;
  for (int j = want + (int)threadIdx.x; j < k; j += 64 * WAVES) o[j] = -1;
  const int32_t* bt_row = pg.block_table ? pg.block_table + (size_t)(row / pg.rows_per_seq) * pg.bt_stride : nullptr;
  resident_select<WAVES, R, kWhole>(scores + (size_t)row * row_stride, n, want, 0, nullptr, o, nullptr, nullptr, bt_row, pg);
}

// ---- a row cut into parts ----------------------------------------------------------------------
// Part p of a row holds entries [p part_len, (p + 1) part_len) below the row's context length and
// answers with min(k, its length) candidates; the row's candidates lie back to back from
// (row * n_parts) * k on, part after part, so that entry j of the list is a position in index order.
__device__ __forceinline__ int part_answers(int n, int part_len, int k, int p) {
  return min(k, max(0, min(n - p * part_len, part_len)));
}

template <int WAVES, int R>
__global__ __launch_bounds__(64 * WAVES) void topk_part_kernel(const float* __restrict__ scores,
                                                              const int32_t* __restrict__ context_lens,
                                                              uint32_t* __restrict__ cand_key, int32_t* __restrict__ cand_idx,
                                                              int n_cols, long long row_stride, int k, int n_parts, int part_len) {
  const int row = blockIdx.x / n_parts, part = blockIdx.x % n_parts;
  const int n = context_lens ? max(0, min(context_lens[row], n_cols)) : n_cols;
  int before = 0;
  for (int p = 0; p < part; ++p) before += part_answers(n, part_len, k, p);
  const int want = part_answers(n, part_len, k, part);
  const size_t base = (size_t)row * n_parts * k + before;
  const int first = part * part_len;
  resident_select<WAVES, R, kPart>(scores + (size_t)row * row_stride + first, max(0, min(n - first, part_len)), want, first, nullptr,
                                   nullptr, cand_key + base, cand_idx + base, nullptr, TopkPaging{});
}

template <int WAVES, int R>
__global__ __launch_bounds__(64 * WAVES) void topk_merge_kernel(const uint32_t* __restrict__ cand_key,
                                                               const int32_t* __restrict__ cand_idx,
                                                               const int32_t* __restrict__ context_lens,
                                                               int32_t* __restrict__ out, int n_cols, int k, int n_parts, int part_len,
                                                               TopkPaging pg) {
  const int row = blockIdx.x;
  const int n = context_lens ? max(0, min(context_lens[row], n_cols)) : n_cols;
  int n_cand = 0;
  for (int p = 0; p < n_parts; ++p) n_cand += part_answers(n, part_len, k, p);
  const int want = min(k, n);                   // (== min(k, n_cand): every part answers with all it has, up to k)
  int32_t* o = out + (size_t)row * k;
  for (int j = want + (int)threadIdx.x; j < k; j += 64 * WAVES) o[j] = -1;
  const size_t base = (size_t)row * n_parts * k;
  const int32_t* bt_row = pg.block_table ? pg.block_table + (size_t)(row / pg.rows_per_seq) * pg.bt_stride : nullptr;
  resident_select<WAVES, R, kMerge>(reinterpret_cast<const float*>(cand_key + base), n_cand, want, 0, cand_idx + base, o, nullptr, nullptr,
                                    bt_row, pg);
}

// Rows of any length: every pass walks the row in memory.
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void topk_stream_kernel(const float* __restrict__ scores,
                                                                 const int32_t* __restrict__ context_lens,
                                                                 int32_t* __restrict__ out, int n_cols,
                                                                 long long row_stride, int k, TopkPaging pg) {
  constexpr int kThreads = 64 * WAVES;
  constexpr int kBatch = WAVES >= 16 ? 8 : 4;
  // 16 copies of every bin, picked by lane % 16: score exponents are heavily skewed, and 64 lanes
  // adding to one LDS word serialise; spread over 16 words (16 banks) they take 4 turns
  __shared__ uint32_t s_hist[256][16];
  __shared__ uint32_t s_sum[256];
  __shared__ uint32_t s_prefix, s_need;         // key bits fixed so far, entries still to find at / below them
  __shared__ int s_wave_gt[WAVES], s_wave_eq[WAVES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int row = blockIdx.x;
  const float* x = scores + (size_t)row * row_stride;
  int32_t* o = out + (size_t)row * k;
  const int n = context_lens ? max(0, min(context_lens[row], n_cols)) : n_cols;
  const int want = min(k, n);                   // entries to select
  for (int j = want + tid; j < k; j += kThreads) o[j] = -1;
  if (want == 0) return;
  const bool vec = ((uintptr_t)x & 15) == 0;
  const int32_t* bt_row = pg.block_table ? pg.block_table + (size_t)(row / pg.rows_per_seq) * pg.bt_stride : nullptr;

  // this wavefront's segment [seg0, seg1): whole 256-entry steps
  const int seg_len = ((n + WAVES - 1) / WAVES + 255) & ~255;
  const int seg0 = min(wave * seg_len, n), seg1 = min(seg0 + seg_len, n);

  auto walk = [&](auto f) { walk_segment<kBatch>(x, seg0, seg1, lane, vec, f); };

  // ---- 1. the key of the want-th largest entry
  static_assert(kThreads >= 256, "the histogram merge uses one thread per bin");
  if (tid == 0) { s_prefix = 0u; s_need = (uint32_t)want; }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int j = tid; j < 256 * 16; j += kThreads) (&s_hist[0][0])[j] = 0u;
    __syncthreads();                            // (also publishes s_prefix / s_need of the previous pass)
    const uint32_t prefix = s_prefix;
    const uint32_t mask = pass == 0 ? 0u : 0xffffffffu << (shift + 8);
    walk([&](int, const Keys4& q, int n_live) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (e < n_live && (q.k[e] & mask) == prefix) atomicAdd(&s_hist[(q.k[e] >> shift) & 255u][lane & 15], 1u);
    });
    __syncthreads();
    if (tid < 256) {
      uint32_t t = 0;
#pragma unroll
      for (int c = 0; c < 16; ++c) t += s_hist[tid][(c + tid) & 15];     // (rotated: fewer bank conflicts)
      s_sum[tid] = t;
    }
    __syncthreads();
    if (wave == 0) {
      // digit d (from the top) where the count of entries with a larger digit is < need <= that + hist[d];
      // lane l looks after digits 255 - 4l .. 252 - 4l
      const uint32_t need = s_need;
      uint32_t h[4], sum = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) { h[j] = s_sum[255 - 4 * lane - j]; sum += h[j]; }
      uint32_t incl = sum;                      // inclusive prefix over lanes
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t u = __shfl_up(incl, d);
        if (lane >= d) incl += u;
      }
      uint32_t above = incl - sum;              // entries with a digit above this lane's four
      if (above < need && need <= incl) {       // exactly one lane
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (above < need && need <= above + h[j]) {
            s_prefix = prefix | ((uint32_t)(255 - 4 * lane - j) << shift);
            s_need = need - above;
            above = 0xffffffffu;                // done
          } else if (above != 0xffffffffu) {
            above += h[j];
          }
        }
      }
    }
  }
  __syncthreads();
  const uint32_t thr = s_prefix;
  const int need_eq = (int)s_need;              // entries equal to thr that are taken (the lowest indices)

  // ---- 2. entries above / equal to the key per segment
  {
    int n_gt = 0, n_eq = 0;
    walk([&](int, const Keys4& q, int n_live) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        n_gt += __popcll(__ballot(e < n_live && q.k[e] > thr));
        n_eq += __popcll(__ballot(e < n_live && q.k[e] == thr));
      }
    });
    if (lane == 0) { s_wave_gt[wave] = n_gt; s_wave_eq[wave] = n_eq; }
  }
  __syncthreads();
  int eq_rank = 0, pos = 0;                     // equal entries / selected entries before my segment
  for (int w = 0; w < wave; ++w) {
    const int e = s_wave_eq[w];
    pos += s_wave_gt[w] + max(0, min(e, need_eq - eq_rank));
    eq_rank += e;
  }

  // ---- 3. emit in index order: entry (lane, e) of a step comes after every entry of the lanes
  // below and after entries 0 .. e-1 of its own lane
  const unsigned long long below = (1ull << lane) - 1ull;
  walk([&](int i0, const Keys4& q, int n_live) {
    bool gt[4], eq[4];
    int gt_lanes_below = 0, eq_lanes_below = 0, gt_step = 0, eq_step = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      gt[e] = e < n_live && q.k[e] > thr;
      eq[e] = e < n_live && q.k[e] == thr;
      const unsigned long long mg = __ballot(gt[e]), me = __ballot(eq[e]);
      gt_lanes_below += __popcll(mg & below); eq_lanes_below += __popcll(me & below);
      gt_step += __popcll(mg); eq_step += __popcll(me);
    }
    int gt_before = gt_lanes_below, my_rank = eq_rank + eq_lanes_below;     // before my entry 0
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int eq_taken_before = min(my_rank, need_eq) - min(eq_rank, need_eq);
      if (gt[e] || (eq[e] && my_rank < need_eq))
        o[pos + gt_before + eq_taken_before] = bt_row == nullptr ? i0 + e : paged_row(i0 + e, bt_row, pg.bt_stride, pg.page_size, pg.kv_rows);
      gt_before += gt[e] ? 1 : 0;
      my_rank += eq[e] ? 1 : 0;
    }
    pos += gt_step + (min(eq_rank + eq_step, need_eq) - min(eq_rank, need_eq));
    eq_rank += eq_step;
  });
}

}  // namespace

// How many parts a row is cut into (1: not at all).  Cutting pays when the rows alone leave most
// compute units idle and a part is still long enough to be worth a workgroup; a part must fit the
// register-resident selection (65 536 entries) and so must the candidates of a row (n_parts * k).
int topk_parts(int n_rows, int n_cols, int k, int n_cu, int* part_len_out) {
  int parts = 1;
  if (n_rows > 0 && 2 * n_rows <= n_cu && n_cols >= 8192) {
    parts = n_cu / n_rows;
    if (parts > 8) parts = 8;
    while (parts > 1 && (n_cols + parts - 1) / parts < 4096) --parts;
    while (parts > 1 && (long long)parts * k > 65536) --parts;
  }
  int part_len = ((n_cols + parts - 1) / parts + 1023) & ~1023;
  if (parts > 1 && part_len > 65536) { parts = 1; part_len = n_cols; }
  if (parts > 1) parts = (n_cols + part_len - 1) / part_len;      // (rounding the length up may leave the last part empty)
  if (part_len_out) *part_len_out = part_len;
  return parts;
}

size_t topk_workspace_bytes(int n_rows, int n_cols, int k, int n_cu) {
  const int parts = topk_parts(n_rows, n_cols, k, n_cu, nullptr);
  return parts > 1 ? (size_t)n_rows * parts * k * 8 : 0;
}

int launch_topk_indices(const float* scores, const int32_t* context_lens, int32_t* out, int n_rows,
                        int n_cols, long long row_stride, int k, const TopkPaging& pg, void* workspace, size_t workspace_bytes,
                        int n_cu, hipStream_t s) {
  if (n_rows == 0) return SMLA_OK;
  int part_len = n_cols;
  const int parts = topk_parts(n_rows, n_cols, k, n_cu, &part_len);
  if (parts > 1 && workspace != nullptr && workspace_bytes >= (size_t)n_rows * parts * k * 8) {
    uint32_t* cand_key = static_cast<uint32_t*>(workspace);
    int32_t* cand_idx = reinterpret_cast<int32_t*>(cand_key + (size_t)n_rows * parts * k);
    const dim3 grid1((unsigned)(n_rows * parts));
    if (part_len <= 4096)
      hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_part_kernel<4, 1>), grid1, dim3(256), 0, s, scores, context_lens, cand_key, cand_idx, n_cols, row_stride, k, parts, part_len);
    else if (part_len <= 16384)
      hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_part_kernel<16, 1>), grid1, dim3(1024), 0, s, scores, context_lens, cand_key, cand_idx, n_cols, row_stride, k, parts, part_len);
    else
      hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_part_kernel<16, 4>), grid1, dim3(1024), 0, s, scores, context_lens, cand_key, cand_idx, n_cols, row_stride, k, parts, part_len);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_status(e);
    const dim3 grid2((unsigned)n_rows);
    const long long n_cand = (long long)parts * k;
    if (n_cand <= 4096)
      hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_merge_kernel<4, 1>), grid2, dim3(256), 0, s, cand_key, cand_idx, context_lens, out, n_cols, k, parts, part_len, pg);
    else if (n_cand <= 16384)
      hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_merge_kernel<16, 1>), grid2, dim3(1024), 0, s, cand_key, cand_idx, context_lens, out, n_cols, k, parts, part_len, pg);
    else
      hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_merge_kernel<16, 4>), grid2, dim3(1024), 0, s, cand_key, cand_idx, context_lens, out, n_cols, k, parts, part_len, pg);
    return hip_status(hipGetLastError());
  }
  const dim3 grid((unsigned)n_rows);
  // Rows of up to 65 536 entries are held in registers, 16 or 64 entries a lane.  With many rows a
  // CU works on several at once and what counts is instructions per row: few wavefronts (the
  // per-pass histogram clearing, merging and barriers are per workgroup).  With few rows a row's
  // latency counts: 16 wavefronts.
  const bool many = n_rows >= 1024;
  if (n_cols <= 4096)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_resident_kernel<4, 1>), grid, dim3(256), 0, s, scores, context_lens, out, n_cols, row_stride, k, pg);
  else if (n_cols <= 16384 && many)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_resident_kernel<4, 4>), grid, dim3(256), 0, s, scores, context_lens, out, n_cols, row_stride, k, pg);
  else if (n_cols <= 16384)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_resident_kernel<16, 1>), grid, dim3(1024), 0, s, scores, context_lens, out, n_cols, row_stride, k, pg);
  else if (n_cols <= 65536)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_resident_kernel<16, 4>), grid, dim3(1024), 0, s, scores, context_lens, out, n_cols, row_stride, k, pg);
  else
    hipLaunchKernelGGL(HIP_KERNEL_NAME(topk_stream_kernel<16>), grid, dim3(1024), 0, s, scores, context_lens, out, n_cols, row_stride, k, pg);
  return hip_status(hipGetLastError());
}

}  // namespace smla
