// fp8 records on the many-heads kernels: raw records into LDS by global -> LDS moves, conversion
// to bf16 tile rows from LDS to LDS.  Shared by the kernels whose tiles are 32 rows of 1 KB bodies
// (16-byte chunks swizzled by a per-row xor) plus a 4 KB RoPE block, filled by 4 wavefronts.
#pragma once
#include "smla_common.h"

namespace smla {
namespace fp8pipe {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
constexpr int kTN = 32;                       // tokens per tile
constexpr int kMainStride = 1024;             // bytes of a tile row's body
constexpr int kRopeBase = kTN * kMainStride;  // size of a tile body
constexpr int kRopeBlock = kTN * 128;         // size of a tile's RoPE block

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

// fp8 records (512 e4m3 values, 4 float scales, 64 bf16 RoPE values = 656 bytes) reach LDS raw,
// by the same global -> LDS moves, and are dequantised from LDS to LDS: no register waits for
// memory.  Wavefront w owns tile rows 8w .. 8w+7 from end to end.  Move j = 0..3 fetches the value
// chunks of its rows 2j and 2j+1 (lane l: row 2j + l/32, chunk l%32) into 1 KB of its raw block,
// move 4 the eight scale chunks (lanes 0..7, one row each) into the 128 bytes behind them, move 5
// the RoPE parts straight into the tile's RoPE block (they are bf16 already).  Later every lane
// turns the four value chunks it fetched itself (raw block byte 16*l + 1024*k) into
// bf16(float(e4m3) * scale) in the tile body.  Only the wavefront's own moves feed its
// conversion, so a wait on its own counter is all the synchronisation the raw data needs, and a
// raw block can be refilled as soon as it is converted.
// LDS: three tile bodies (one being multiplied, one being scored, one being written), three RoPE
// blocks (scored, landed, in flight) and two raw blocks per wavefront (converting, in flight).
struct Pipe {
  static constexpr int kRawWave = 8 * (kFp8ScaleOff + 16);     // 4224 bytes: a wavefront's 8 rows, values then scales
  static constexpr int kRawScales = 8 * kFp8ScaleOff;          // 4096: where the scale chunks start
  static constexpr int kRawSlot = 4 * kRawWave;                // 16896
  static constexpr int kSteps = 6;                             // move instructions per wavefront per tile
  static constexpr int kBodies = 3, kRopes = 3, kRaws = 2;
  static constexpr int kRopeRing = kBodies * kRopeBase;        // byte offsets in the ring area
  static constexpr int kRawRing = kRopeRing + kRopes * kRopeBlock;
  static constexpr int kRingBytes = kRawRing + kRaws * kRawSlot;      // 144384
  const uint8_t* kv;
  uint32_t raw_lds, rope_lds;
  int32_t rid;
  int wave, lane;
  // raw_lds_: this wavefront's raw block, rope_lds_: the tile's RoPE block
  __device__ __forceinline__ void begin(const uint8_t* kv_, const int32_t* rows, int e0, int n_valid,
                                        uint32_t raw_lds_, uint32_t rope_lds_, int wave_, int lane_) {
    kv = kv_; raw_lds = raw_lds_; rope_lds = rope_lds_; wave = wave_; lane = lane_;
    rid = rows[min(e0 + (lane & 31), n_valid - 1)];               // lane l holds the row id of tile row l % 32
  }
  __device__ __forceinline__ void step(int j) const {
    if (j < 4) {
      const int32_t trow = __shfl(rid, 8 * wave + 2 * j + (lane >> 5));
      hw::dma_b128(kv + (size_t)trow * kRowBytesFp8 + (lane & 31) * 16, raw_lds + 1024 * j);
    } else if (j == 4) {
      const int32_t trow = __shfl(rid, 8 * wave + (lane & 7));
      hw::dma_b128_first_lanes<8>(kv + (size_t)trow * kRowBytesFp8 + kFp8ScaleOff, raw_lds + kRawScales);
    } else {
      const int pair = 4 * wave + (lane >> 4);
      const int r = 2 * pair + ((lane >> 3) & 1), c = (lane & 7) ^ (pair & 7);
      const int32_t trow = __shfl(rid, r);
      hw::dma_b128(kv + (size_t)trow * kRowBytesFp8 + kFp8ScaleOff + 16 + c * 16, rope_lds + wave * 1024);
    }
  }
};

// The conversion of one tile is 4 chunks of 16 values per lane: chunk k is column chunk l % 32 of
// the wavefront's row l/32 + 2k.  load / half / store are separate so that a caller can thread
// them through an MFMA stream.  Layout: swz(row) is the kernel's chunk xor of a tile row, and
// store_xor(k) = swz(row0 + 2k) ^ swz(row0) for row0 = 8 * wave + l/32, which for the layouts in
// use does not depend on row0: one per-lane offset then serves all four chunks.
template <typename Layout>
struct Convert {
  hw::u32x4 v;
  float sc;
  uint32_t o[8];
  uint32_t raw_lds;        // this wavefront's raw block
  uint32_t body_lds;       // the tile body being written
  int wave, lane;
  __device__ __forceinline__ void load(int k) {
    v = hw::lds_read_u128(raw_lds + 16 * lane + 1024 * k);
    sc = hw::lds_read_f32(raw_lds + Pipe::kRawScales + 16 * (lane >> 5) + 4 * ((lane & 31) >> 3) + 32 * k);
  }
  // A lane turns 16 codes into the bf16 chunks 2*col and 2*col + 1 of its row, 16 bytes each, stored
  // by two instructions.  A 16-byte store is served 16 lanes at a time, and sixteen EVEN chunks of a
  // row cover only half the banks twice; so the lanes whose column has bit 3 set take their two
  // chunks in the other order (`swap`): every instruction then writes sixteen chunks that differ
  // modulo 16.  half(0) makes the chunk stored first, half(1) the other.
  __device__ __forceinline__ bool swap() const { return (lane & 8) != 0; }
  __device__ __forceinline__ void half(int h) {
    const bool second = (h != 0) != swap();                        // which 8 codes: the first or the second half of the 16
    const uint32_t w[2] = {second ? v[2] : v[0], second ? v[3] : v[1]};
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[k], false);
      const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[k], true);
      o[4 * h + 2 * k] = pack_bf16(lo[0] * sc, lo[1] * sc);
      o[4 * h + 2 * k + 1] = pack_bf16(hi[0] * sc, hi[1] * sc);
    }
  }
  __device__ __forceinline__ void store(int k) {
    // tile row 8*wave + l/32 + 2k, chunks 2*col and 2*col + 1
    const int row0 = 8 * wave + (lane >> 5), col = lane & 31;
    int off = row0 * kMainStride + (((2 * col + (swap() ? 1 : 0)) ^ Layout::swz(row0)) << 4);
    hw::pin(off);                                                  // (worked out here, not kept in four registers from the top of the kernel)
    off = (off ^ (Layout::store_xor(k) << 4)) + 2 * k * kMainStride;
    hw::lds_write_b128(body_lds + off, hw::u32x4{o[0], o[1], o[2], o[3]});
    hw::lds_write_b128(body_lds + (off ^ 16), hw::u32x4{o[4], o[5], o[6], o[7]});
  }
  __device__ __forceinline__ void whole_tile() {     // (one chunk at a time: where this is called, registers are scarce)
#pragma unroll 1
    for (int k = 0; k < 4; ++k) { load(k); half(0); half(1); store(k); }
  }
};

// Compile-time check of what Convert::store relies on: for every row0 = 8 * wave + l/32 the row xor
// of row0 + 2k is that of row0 xor-ed with Layout::store_xor(k).
template <typename Layout>
constexpr bool layout_ok() {
  for (int wave = 0; wave < 4; ++wave)
    for (int g = 0; g < 2; ++g)
      for (int k = 0; k < 4; ++k)
        if (Layout::swz(8 * wave + g + 2 * k) != (Layout::swz(8 * wave + g) ^ Layout::store_xor(k))) return false;
  return true;
}

}  // namespace fp8pipe
}  // namespace smla
