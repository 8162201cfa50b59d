// Local GEMM of GEMM + reduce-scatter: out = bf16(X . W + partial), written as n_chunks row chunks.
// Two kernels: gemm_rs_big_kernel (further down) when M is a multiple of 256, else gemm_rs_kernel:
//
// 128 x 256 output tile per workgroup of 4 wavefronts (2 x 2, each 64 x 128 = 2 x 4 MFMA tiles of
// 32 x 32, fp32 accumulators), K advanced 64 at a time through one LDS buffer (the next K-step
// waits in registers while the current one is consumed),
// two workgroups per CU so one's epilogue (fp32 partial-sum read + bf16 store) overlaps the
// other's main loop.  X is row-major [M, K] (K contiguous): A operands are plain 16-byte LDS
// reads.  W is row-major [K, N] (N contiguous): B operands want 8 consecutive k per lane, which
// the transposing LDS read delivers from the row-major tile.
// The epilogue transposes each wavefront's block through LDS, 16 rows at a time, so that the
// partial sums are read 16 bytes per lane and the bf16 results written 8 bytes per lane in
// 512-byte / 256-byte row runs; all partial-sum loads of a 32-row half are issued before the first
// is used (they stream from HBM: a load-use-load-use loop would be latency bound).
// Block ids are dealt round-robin to the 8 XCDs; each XCD owns a contiguous band of M so the
// X rows it re-reads stay in its L2.
#include "smla_common.h"

#include <stdlib.h>

namespace smla {

typedef __attribute__((ext_vector_type(8))) __bf16 g_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 g_bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 g_bf16x2;
typedef __attribute__((ext_vector_type(4))) short g_short4;
typedef __attribute__((ext_vector_type(16))) float g_f32x16;
typedef __attribute__((ext_vector_type(4))) float g_f32x4;

constexpr int kBM = 128, kBN = 256, kBK = 64;
constexpr int kAStride = kBK * 2 + 16;        // 144 B per X row in LDS: 16 consecutive rows hit 16 distinct bank groups
constexpr int kBStride = kBN * 2 + 64;        // 576 B per W row in LDS: 4 consecutive rows x 64 B cover all 64 banks (transposing reads)
constexpr int kABytes = kBM * kAStride;       // 18432
constexpr int kBBytes = kBK * kBStride;       // 36864
constexpr int kStageFloats = 128 + 8;         // epilogue staging row: 128 fp32 + 32 B pad (rows 4 apart land 32 banks apart)
static_assert(4 * 16 * kStageFloats * 4 <= kBBytes, "epilogue staging (16 rows x 128 fp32 per wavefront) lives in the W buffers");

__device__ __forceinline__ uint32_t g_pack_bf16(float a, float b) {
  g_bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ g_bf16x4 g_read_tr(const uint8_t* p) {
  return hw::lds_read_tr16_b64(p);
}

__global__ __launch_bounds__(256, 2) void gemm_rs_kernel(const uint16_t* __restrict__ x,
                                                         const uint16_t* __restrict__ w,
                                                         const float* __restrict__ partial,
                                                         uint16_t* __restrict__ out, int M, int N, int K,
                                                         int rows_per_chunk, long long chunk_stride) {
  __shared__ __attribute__((aligned(16))) uint8_t s_a[kABytes];     // one buffer each: the next K-step waits in registers
  __shared__ __attribute__((aligned(16))) uint8_t s_b[kBBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;              // wave tile origin (64 * wm, 128 * wn)
  const int g = lane >> 5, c32 = lane & 31, l16 = lane & 15;

  // tile mapping: XCD x owns m-tiles [x * mt/8, (x+1) * mt/8) when mt divides by 8
  const int mt = M / kBM, nt = N / kBN;
  int tile_m, tile_n;
  {
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    if (mt % 8 == 0) {
      const int band = mt / 8;
      tile_m = xcd * band + local % band;
      tile_n = local / band;
    } else {
      tile_m = blockIdx.x % mt;
      tile_n = blockIdx.x / mt;
    }
  }
  if (tile_m >= mt || tile_n >= nt) return;
  const int m0 = tile_m * kBM, n0 = tile_n * kBN;

  // global -> register staging: X tile 128 x 64 = 1024 chunks of 16 B (4 per thread),
  // W tile 64 x 256 = 2048 chunks (8 per thread)
  const int a_row = tid >> 3, a_col = tid & 7;          // rows 0..31 (+32, +64, +96), 8 chunks per row
  const int b_row = tid >> 5, b_col = tid & 31;         // rows 0..7 (+8 * i), 32 chunks per row
  const uint16_t* xa = x + (size_t)(m0 + a_row) * K + a_col * 8;
  const uint16_t* wb = w + (size_t)b_row * N + n0 + b_col * 8;
  // (written as macros over plain locals: staging arrays captured by a closure are left in
  // scratch memory by the compiler once they exceed a few registers)
  typedef __attribute__((ext_vector_type(4))) uint32_t g_u32x4;
  g_u32x4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3, rb4, rb5, rb6, rb7;
#define G_LOAD(k0)                                                                          \
  do {                                                                                      \
    ra0 = *reinterpret_cast<const g_u32x4*>(xa + (k0));                                     \
    ra1 = *reinterpret_cast<const g_u32x4*>(xa + (size_t)32 * K + (k0));                    \
    ra2 = *reinterpret_cast<const g_u32x4*>(xa + (size_t)64 * K + (k0));                    \
    ra3 = *reinterpret_cast<const g_u32x4*>(xa + (size_t)96 * K + (k0));                    \
    rb0 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 0) * N);                   \
    rb1 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 8) * N);                   \
    rb2 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 16) * N);                  \
    rb3 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 24) * N);                  \
    rb4 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 32) * N);                  \
    rb5 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 40) * N);                  \
    rb6 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 48) * N);                  \
    rb7 = *reinterpret_cast<const g_u32x4*>(wb + (size_t)((k0) + 56) * N);                  \
  } while (0)
#define S_STORE()                                                                           \
  do {                                                                                      \
    *reinterpret_cast<g_u32x4*>(s_a + (a_row + 0) * kAStride + a_col * 16) = ra0;           \
    *reinterpret_cast<g_u32x4*>(s_a + (a_row + 32) * kAStride + a_col * 16) = ra1;          \
    *reinterpret_cast<g_u32x4*>(s_a + (a_row + 64) * kAStride + a_col * 16) = ra2;          \
    *reinterpret_cast<g_u32x4*>(s_a + (a_row + 96) * kAStride + a_col * 16) = ra3;          \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 0) * kBStride + b_col * 16) = rb0;           \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 8) * kBStride + b_col * 16) = rb1;           \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 16) * kBStride + b_col * 16) = rb2;          \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 24) * kBStride + b_col * 16) = rb3;          \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 32) * kBStride + b_col * 16) = rb4;          \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 40) * kBStride + b_col * 16) = rb5;          \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 48) * kBStride + b_col * 16) = rb6;          \
    *reinterpret_cast<g_u32x4*>(s_b + (b_row + 56) * kBStride + b_col * 16) = rb7;          \
  } while (0)

  g_f32x16 acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // The next K-step's loads are in flight during the whole compute phase (32 MFMAs per wavefront);
  // they are parked in LDS between two barriers, during which the CU's other workgroup runs.
  G_LOAD(0);
  S_STORE();
  __syncthreads();
  const int n_k = K / kBK;
  const uint8_t* a_base = s_a + (64 * wm + c32) * kAStride + g * 16;
  const uint8_t* b_base = s_b + (8 * g + (l16 >> 2)) * kBStride + (128 * wn + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3)) * 2;
  for (int kt = 0; kt < n_k; ++kt) {
    if (kt + 1 < n_k) G_LOAD((kt + 1) * kBK);
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      g_bf16x8 af[2], bf[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = *reinterpret_cast<const g_bf16x8*>(a_base + 32 * i * kAStride + ks * 32);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t* bp = b_base + (16 * ks) * kBStride + j * 64;
        const g_bf16x4 lo = g_read_tr(bp);
        const g_bf16x4 hi = g_read_tr(bp + 4 * kBStride);      // rows k+4..k+7 of this lane group's 8
        bf[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();                                    // every wavefront is done reading this K-step
    if (kt + 1 < n_k) S_STORE();
    __syncthreads();
  }

  // ---- epilogue.  Accumulator layout: lane owns column lane % 32 of each 32 x 32 tile, register r is
  // row 8*(r/4) + 4*(lane/32) + r%4.  Each wavefront parks 16 rows x 128 columns at a time in LDS
  // (the W buffers are free: the loop ended with a barrier; the staging area is private to the
  // wavefront, whose LDS accesses complete in order) and reads them back two rows per pass, four
  // consecutive columns per lane.
#undef G_LOAD
#undef S_STORE
  float* stage = reinterpret_cast<float*>(s_b) + wave * 16 * kStageFloats;
  const int col4 = 4 * c32;                             // this lane's 4 columns within the wave's 128
  const int n = n0 + 128 * wn + col4;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    g_f32x4 z[16];                                      // partial sums of rows 32*i + 2*p + g, p < 16
#pragma unroll
    for (int p2 = 0; p2 < 16; ++p2) {
      const int m = m0 + 64 * wm + 32 * i + 2 * p2 + g;
      z[p2] = partial ? __builtin_nontemporal_load(reinterpret_cast<const g_f32x4*>(partial + (size_t)m * N + n))
                      : g_f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {                       // rows 16*h .. 16*h+15 of this half: registers 8*h .. 8*h+7
#pragma unroll
      for (int r = 8 * h; r < 8 * h + 8; ++r) {
        const int row = 8 * ((r >> 2) & 1) + 4 * g + (r & 3);
#pragma unroll
        for (int j = 0; j < 4; ++j) stage[row * kStageFloats + 32 * j + c32] = acc[i][j][r];
      }
      hw::wave_lds_order();
#pragma unroll
      for (int p1 = 0; p1 < 8; ++p1) {
        const int row = 2 * p1 + g;                     // within the 16 staged rows
        const int m = m0 + 64 * wm + 32 * i + 16 * h + row;
        const float4 v = *reinterpret_cast<const float4*>(stage + row * kStageFloats + col4);
        const g_f32x4 zz = z[8 * h + p1];
        const int chunk = m / rows_per_chunk;
        uint16_t* o = out + (size_t)chunk * chunk_stride + (size_t)(m - chunk * rows_per_chunk) * N + n;
        uint2 pk;
        pk.x = g_pack_bf16(v.x + zz[0], v.y + zz[1]);
        pk.y = g_pack_bf16(v.z + zz[2], v.w + zz[3]);
        *reinterpret_cast<uint2*>(o) = pk;
      }
      hw::wave_lds_order();
    }
  }
}

// ---------------------------------------------------------------------------------------------
// 256 x 256 output tile per workgroup of 16 wavefronts, one workgroup per CU (M a multiple of 256).
//
// Half the L2 -> CU traffic of the 128 x 256 tiling (1.9 GB against 2.8 GB on the bench shape) and
// four wavefronts per SIMD to hide each other's LDS latencies: wavefront (wm, wn) of the 4 x 4 grid
// owns 64 x 64 (2 x 2 MFMA tiles of 32 x 32, 64 accumulator registers).  The K-steps of 64 go
// global -> LDS by DMA (no staging registers) into two 64 KB buffers, one barrier per K-step: the
// next step's four DMA instructions per wavefront are issued between the MFMAs of the current step,
// right after the barrier that frees their buffer, and the fragments of K-slice ks + 1 are read
// while the MFMAs of slice ks run.
//
// LDS layouts (a DMA instruction writes 1 KB of consecutive LDS, lane l its 16 bytes at 16 l, from
// any global address, so rows cannot be padded; the bank spread comes from where each lane fetches):
//   X tile  256 rows x 128 B: 16-byte chunk c of row r at chunk position c ^ ((r >> 1) & 7).
//           A fragments read chunk (2 ks + lane / 32) of 32 consecutive rows, 16 lanes a pass: 16
//           consecutive rows then cover all 64 banks.
//   W tile  64 rows x 512 B: 64-byte block b of row k at block position b ^ (k & 3).
//           B fragments are transposing reads of 64 B from each of 4 consecutive rows, 32 lanes a
//           pass: the four rows' blocks then cover all 64 banks.
constexpr int kBM2 = 256, kBN2 = 256;
constexpr int kA2Bytes = kBM2 * kBK * 2;      // 32768
constexpr int kB2Bytes = kBK * kBN2 * 2;      // 32768
constexpr int kStage2 = kA2Bytes + kB2Bytes;  // 65536
constexpr int kStage2Floats = 64;             // epilogue staging row of a wavefront: 64 fp32 (a pass reads whole rows: all banks once)
static_assert(16 * 32 * kStage2Floats * 4 <= 2 * kStage2, "epilogue staging (32 rows x 64 fp32 per wavefront) lives in the K-step buffers");

__device__ __forceinline__ g_bf16x8 g_lds_b128(uint32_t a) {
  return hw::lds_read_b128(a);
}
__device__ __forceinline__ g_bf16x4 g_lds_tr(uint32_t a) {
  return hw::lds_read_tr16_b64(a);
}

// What a persistent workgroup carries from one tile to the next (CHAIN): which of the two K-step
// buffers holds, or is receiving, K-step 0 of the current tile, whether the tile before has already
// sent for it, and where the next tile lies, so that this tile can send for the next one's K-step 0
// during its own last K-step.  The next tile's first fetch then runs under this tile's epilogue,
// which for that reason stages through ONE buffer (the one the last K-step was read from), 16 rows
// of a wavefront's block at a time, while the other buffer receives.
struct TileChain {
  int base;
  bool primed, has_next;
  int next_m0, next_n0;
};

// One output tile of 128 MI rows x 256 columns (MI = 2: the full 256 x 256 tile; MI = 1: its upper
// or lower half, used to fill the last, partly occupied round of tiles, see launch_gemm_rs).
// Wavefront (wm, wn) owns rows 32 MI wm .. + 32 MI - 1 and columns 64 wn .. + 63.
template <int MI, bool CHAIN = false>
__device__ __forceinline__ void gemm_big_tile(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                              const float* __restrict__ partial, uint16_t* __restrict__ out, int N, int K,
                                              int rows_per_chunk, long long chunk_stride, int m0, int n0,
                                              uint8_t* s_buf0, TileChain* chain = nullptr) {
  static_assert(!CHAIN || MI == 2, "only whole tiles are chained");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int g = lane >> 5, c32 = lane & 31, l16 = lane & 15;
  const uint32_t lds0 = hw::lds_addr(s_buf0);

  // ---- DMA of one K-step: 16 MI instructions for the X tile (8 rows each) and 32 for the W tile (2
  // rows each), MI + 2 per wavefront.  X instruction i = MI wave + d, W instruction i = 2 wave + d;
  // the swizzles depend on i's parity only, so a lane needs two byte offsets per tile.
  uint32_t a_off[2], b_off[2];
  {
    const int p = lane & 7, rl = lane >> 3;             // X: chunk position, row within the instruction's 8
#pragma unroll
    for (int odd = 0; odd < 2; ++odd) {
      const int c = p ^ ((4 * odd + (rl >> 1)) & 7);    // row r = 8 i + rl: (r >> 1) & 7 = (4 i + rl / 2) & 7
      a_off[odd] = (uint32_t)((rl * K + 8 * c) * 2);
    }
    const int pb = lane & 31, kl = lane >> 5;           // W: chunk position, row within the instruction's 2
#pragma unroll
    for (int odd = 0; odd < 2; ++odd) {
      const int blk = (pb >> 2) ^ ((2 * odd + kl) & 3); // row k = 2 i + kl: k & 3 = (2 i + kl) & 3
      b_off[odd] = (uint32_t)((kl * N + 8 * (4 * blk + (pb & 3))) * 2);
    }
  }
  // DMA slot d = 0..3 of this wavefront for the K-step at k0 of the tile at (tm0, tn0) into buffer buf (0, 1: X, 2, 3: W)
  auto issue_dma_at = [&](int d, int k0, int buf, int tm0, int tn0) {
    const uint32_t dst = lds0 + buf * kStage2;
    if (d < 2) {
      if (d < MI) {
        const int i = MI * wave + d;
        const uint64_t sa = (uint64_t)(uintptr_t)x + ((uint64_t)(tm0 + 8 * i) * K + k0) * 2;
        const uint32_t ma = dst + i * 1024;
        hw::dma_b128(a_off[i & 1], sa, ma);
      }
    } else {
      const int i = 2 * wave + d - 2;
      const uint64_t sb = (uint64_t)(uintptr_t)w + ((uint64_t)(k0 + 2 * i) * N + tn0) * 2;
      const uint32_t mb = dst + kA2Bytes + i * 1024;
      hw::dma_b128(b_off[d & 1], sb, mb);
    }
  };
  auto issue_dma = [&](int d, int k0, int buf) { issue_dma_at(d, k0, buf, m0, n0); };
  const int base = CHAIN ? chain->base : 0;               // the buffer of this tile's K-step 0

  g_f32x16 acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // fragment addresses inside a buffer
  const uint32_t a_lane = (uint32_t)((32 * MI * wm + c32) * 128);         // row of A tile i = 0; + 32 i rows
  const uint32_t a_sw = (uint32_t)((c32 >> 1) & 7);
  const uint32_t b_lane = (uint32_t)(kA2Bytes + (8 * g + (l16 >> 2)) * 512 + 32 * ((lane >> 4) & 1) + 8 * (l16 & 3));
  const uint32_t b_sw = (uint32_t)((l16 >> 2) & 3);

  const int n_k = K / kBK;
  if (!CHAIN || !chain->primed) {
#pragma unroll
    for (int d = 0; d < 4; ++d) issue_dma(d, 0, base);
  }
  auto load_frags = [&](uint32_t buf, int ks, g_bf16x8 (&af)[MI], g_bf16x8 (&bf)[2]) {
#pragma unroll
    for (int i = 0; i < MI; ++i) af[i] = g_lds_b128(buf + a_lane + i * (32 * 128) + (((2 * ks + g) ^ a_sw) << 4));
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t bp = buf + b_lane + (16 * ks) * 512 + (((2 * wn + j) ^ b_sw) << 6);
      const g_bf16x4 lo = g_lds_tr(bp);
      const g_bf16x4 hi = g_lds_tr(bp + 4 * 512);               // rows k+4..k+7 of this lane group's 8
      bf[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  };
  for (int kt = 0; kt < n_k; ++kt) {
    hw::wait_vmcnt<0>();    // this wavefront's share of step kt has landed
    __syncthreads();                                    // ... everyone's has, and everyone is done with step kt - 1
    const uint32_t buf = lds0 + ((base + kt) & 1) * kStage2;
    const bool more = kt + 1 < n_k;
    const int k_next = (kt + 1) * kBK, buf_next = (base + kt + 1) & 1;
    g_bf16x8 af[2][MI], bf[2][2];
    load_frags(buf, 0, af[0], bf[0]);
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      if (ks + 1 < kBK / 16) load_frags(buf, ks + 1, af[(ks + 1) & 1], bf[(ks + 1) & 1]);
      if (more) issue_dma(ks, k_next, buf_next);
      else if (CHAIN && chain->has_next) issue_dma_at(ks, 0, buf_next, chain->next_m0, chain->next_n0);   // the next tile's K-step 0
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][i], bf[ks & 1][j], acc[i][j], 0, 0, 0);
    }
  }
  __syncthreads();                                      // the buffers are free: the epilogue stages through them
                                                        // (CHAIN: the buffer of the last K-step is; the other one is receiving)

  // ---- epilogue: a wavefront parks kRowsStage rows x 64 columns of its MFMA tiles in LDS and
  // reads them back four rows a pass, four consecutive columns per lane
  constexpr int kRowsStage = CHAIN ? 16 : 32;           // rows parked at a time: 32 = a whole row of MFMA tiles
  const int last_buf = (base + n_k - 1) & 1;
  float* stage = CHAIN ? reinterpret_cast<float*>(s_buf0 + last_buf * kStage2) + wave * kRowsStage * kStage2Floats
                       : reinterpret_cast<float*>(s_buf0) + wave * kRowsStage * kStage2Floats;
  static_assert(16 * 16 * kStage2Floats * 4 <= kStage2, "chained tiles stage through one buffer");
  const int col4 = 4 * l16, rsub = lane >> 4;           // this lane's 4 columns within the wave's 64, row within a pass
  const int n = n0 + 64 * wn + col4;
#pragma unroll
  for (int i = 0; i < MI; ++i) {
#pragma unroll
    for (int h = 0; h < 32 / kRowsStage; ++h) {         // the rows 32 i + kRowsStage h .. of the wavefront's block
      constexpr int kPasses = kRowsStage / 4;
      g_f32x4 z[kPasses];                               // partial sums of rows 32 i + kRowsStage h + 4 p + rsub
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const int m = m0 + 32 * MI * wm + 32 * i + kRowsStage * h + 4 * p + rsub;
        z[p] = partial ? __builtin_nontemporal_load(reinterpret_cast<const g_f32x4*>(partial + (size_t)m * N + n))
                       : g_f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * g + (r & 3);
        if ((8 * (r >> 2)) / kRowsStage != h) continue; // (known at compile time: 4 g + r % 4 never crosses a multiple of 8)
#pragma unroll
        // (a row is exactly the 64 banks wide, and a store's two half-wavefronts write rows 4 apart:
        // rows with bit 2 set keep their two 32-float halves swapped, so the halves land on different banks)
        for (int j = 0; j < 2; ++j) stage[(row - kRowsStage * h) * kStage2Floats + ((32 * j + c32) ^ (32 * g))] = acc[i][j][r];
      }
      __builtin_amdgcn_wave_barrier();                  // (the area is the wavefront's own; its LDS operations complete in order)
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const int row = 4 * p + rsub;
        const int m = m0 + 32 * MI * wm + 32 * i + kRowsStage * h + row;
        const float4 v = *reinterpret_cast<const float4*>(stage + row * kStage2Floats + (col4 ^ (32 * ((row >> 2) & 1))));
        const g_f32x4 zz = z[p];
        const int chunk = m / rows_per_chunk;
        uint16_t* o = out + (size_t)chunk * chunk_stride + (size_t)(m - chunk * rows_per_chunk) * N + n;
        uint2 pk;
        pk.x = g_pack_bf16(v.x + zz[0], v.y + zz[1]);
        pk.y = g_pack_bf16(v.z + zz[2], v.w + zz[3]);
        *reinterpret_cast<uint2*>(o) = pk;
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  if constexpr (CHAIN) {                                // hand the buffers on: the next tile's K-step 0 is on its way into the other one
    chain->base = last_buf ^ 1;
    chain->primed = chain->has_next;
  }
}

// Blocks [0, n_full) take whole 256 x 256 tiles; blocks from n_full on take half tiles (128 rows),
// two consecutive blocks of an XCD the two halves of one tile.  The hardware hands out blocks in
// id order, so the half tiles are what runs last.
// Block id -> tile.  XCD x (= id % 8) owns m-tiles [x * mt/8, (x+1) * mt/8) when mt divides by 8.
// Returns false for an id without a tile.
__device__ __forceinline__ bool big_tile_of(int id, int n_full, int mt, int nt, int& tile_m, int& tile_n, int& half, bool& halves) {
  halves = id >= n_full;
  half = 0;
  int xcd = id & 7, local = id >> 3;
  if (halves) {                                         // (only with the banded mapping; n_full is a multiple of 8)
    const int j = id - n_full;
    xcd = j & 7;
    half = (j >> 3) & 1;
    local = (n_full >> 3) + (j >> 4);
  }
  if (mt % 8 == 0) {
    const int band = mt / 8;
    tile_m = xcd * band + local % band;
    tile_n = local / band;
  } else {
    tile_m = id % mt;
    tile_n = id / mt;
  }
  return tile_m < mt && tile_n < nt;
}

__global__ __launch_bounds__(1024)
void gemm_rs_big_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                        const float* __restrict__ partial, uint16_t* __restrict__ out, int M, int N, int K,
                        int rows_per_chunk, long long chunk_stride, int n_full) {
  __shared__ __attribute__((aligned(1024))) uint8_t s_buf[2][kStage2];
  const int mt = M / kBM2, nt = N / kBN2;
  int tile_m, tile_n, half;
  bool halves;
  if (!big_tile_of((int)blockIdx.x, n_full, mt, nt, tile_m, tile_n, half, halves)) return;
  const int n0 = tile_n * kBN2;
  if (halves)
    gemm_big_tile<1>(x, w, partial, out, N, K, rows_per_chunk, chunk_stride, tile_m * kBM2 + 128 * half, n0, &s_buf[0][0]);
  else
    gemm_big_tile<2>(x, w, partial, out, N, K, rows_per_chunk, chunk_stride, tile_m * kBM2, n0, &s_buf[0][0]);
}

// The same tiles by persistent workgroups, one per compute unit (opt-in: FLAGTREE_SMLA_GEMM_CHAIN=1).
// Workgroup b takes the block ids b, b + gridDim.x, ... of the kernel above (gridDim.x a multiple
// of 8, so all of them belong to its own XCD's band); its whole tiles are chained: the moves of the
// next tile's K-step 0 go out during the current tile's last K-step and land while the epilogue
// (partial sums in, bf16 out: traffic that otherwise finds the CU's matrix cores and its LDS
// moves idle) runs.  Its half tiles, which come last, run one by one.
__global__ __launch_bounds__(1024)
void gemm_rs_chain_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                          const float* __restrict__ partial, uint16_t* __restrict__ out, int M, int N, int K,
                          int rows_per_chunk, long long chunk_stride, int n_full, int n_ids) {
  __shared__ __attribute__((aligned(1024))) uint8_t s_buf[2][kStage2];
  const int mt = M / kBM2, nt = N / kBN2;
  const int step = (int)gridDim.x;
  TileChain chain{0, false, false, 0, 0};
  int id = (int)blockIdx.x;
  int tile_m, tile_n, half;
  bool halves;
  // whole tiles (ids below n_full; every such id has a tile when the banded mapping applies, which the launcher checks)
  for (; id < n_full; id += step) {
    big_tile_of(id, n_full, mt, nt, tile_m, tile_n, half, halves);
    const int m0 = tile_m * kBM2, n0 = tile_n * kBN2;
    chain.has_next = id + step < n_full;
    if (chain.has_next) {
      int nm, nn, nh;
      bool nhalves;
      big_tile_of(id + step, n_full, mt, nt, nm, nn, nh, nhalves);
      chain.next_m0 = nm * kBM2;
      chain.next_n0 = nn * kBN2;
    }
    gemm_big_tile<2, true>(x, w, partial, out, N, K, rows_per_chunk, chunk_stride, m0, n0, &s_buf[0][0], &chain);
  }
  for (; id < n_ids; id += step) {
    __syncthreads();                                    // every wavefront is done with the tile before: its staging area is free
    if (!big_tile_of(id, n_full, mt, nt, tile_m, tile_n, half, halves)) continue;
    gemm_big_tile<1>(x, w, partial, out, N, K, rows_per_chunk, chunk_stride, tile_m * kBM2 + 128 * half, tile_n * kBN2, &s_buf[0][0]);
  }
}

// How many of the 256 x 256 tiles are computed whole; the rest, the last and only partly filled
// round of tiles on `n_cu` compute units, is split into half tiles when that fills the round:
// 896 tiles on 256 units are 3 rounds + 128 tiles, which as 256 half tiles keep every unit busy for
// 3/4 of a round (a half tile moves 3/4 of a tile's bytes into LDS) instead of half the units for a
// whole one.
// The kernel's half-tile mapping takes whole tiles in groups of 8 (one per XCD), so the count
// of whole tiles must be a multiple of 8: only a compute-unit count that is one gives that.
int gemm_full_tiles(int mt, int nt, int n_cu) {
  const long long tiles = (long long)mt * nt;
  if (mt % 8 != 0 || n_cu <= 0 || n_cu % 8 != 0) return (int)tiles;
  const long long rest = tiles % n_cu;
  return rest > 0 && 2 * rest <= n_cu ? (int)(tiles - rest) : (int)tiles;
}

int launch_gemm_rs(const void* x, const void* w, const float* partial, void* out, int m, int n, int k,
                   int n_chunks, int64_t chunk_stride, int n_cu, hipStream_t s) {
  if (m % kBM != 0 || n % kBN != 0 || k % kBK != 0) return SMLA_EINVAL_SHAPE;
  // the DMA's per-lane byte offsets are 32-bit
  const bool big = m % kBM2 == 0 && (long long)8 * k * 2 < (1ll << 31) && ((long long)2 * n + n) * 2 < (1ll << 31);
  const int bm = big ? kBM2 : kBM;
  const int mt = m / bm, nt = n / kBN;
  long long blocks = (long long)((mt + 7) / 8 * 8) * nt;
  if (blocks > 0x3fffffffLL) return SMLA_EINVAL_SHAPE;
  if (big) {
    const long long tiles = (long long)mt * nt;
    long long n_full = gemm_full_tiles(mt, nt, n_cu);
    if (n_full < tiles) blocks = n_full + 2 * (tiles - n_full);   // (only with mt a multiple of 8: blocks was mt * nt)
    else n_full = blocks;                                         // no half tiles
    // persistent workgroups (opt-in): needs the banded mapping with every id a tile, and a workgroup count that keeps ids on their XCD
    const char* e = getenv("FLAGTREE_SMLA_GEMM_CHAIN");
    if (e != nullptr && e[0] == '1' && mt % 8 == 0 && n_cu % 8 == 0 && blocks > n_cu) {
      if (n_full == blocks) n_full = tiles;                       // (mt % 8 == 0: blocks == tiles)
      hipLaunchKernelGGL(gemm_rs_chain_kernel, dim3((unsigned)n_cu), dim3(1024), 0, s,
          static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w), partial, static_cast<uint16_t*>(out), m, n, k,
          m / n_chunks, (long long)chunk_stride, (int)n_full, (int)blocks);
      return hip_status(hipGetLastError());
    }
    hipLaunchKernelGGL(gemm_rs_big_kernel, dim3((unsigned)blocks), dim3(1024), 0, s,
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w), partial, static_cast<uint16_t*>(out), m, n, k,
        m / n_chunks, (long long)chunk_stride, (int)n_full);
  } else
    hipLaunchKernelGGL(gemm_rs_kernel, dim3((unsigned)blocks), dim3(256), 0, s, 
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w), partial, static_cast<uint16_t*>(out), m, n, k,
        m / n_chunks, (long long)chunk_stride);
  return hip_status(hipGetLastError());
}

}  // namespace smla
