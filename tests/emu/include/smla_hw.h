// CPU-emulator counterpart of flagtree_amd/csrc/smla_hw.h: the same functions with host
// semantics (test infrastructure only; found first on the emulator build's include path).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace smla {
namespace hw {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short short4v;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

inline uint32_t lds_addr(const void* shared_object) { return emu::lds_addr(shared_object); }
inline bf16x8 lds_read_b128(uint32_t a) {
  if (a & 15) emu::fail("ds_read_b128 at unaligned LDS address %u", a);
  emu::lds_account(a, 16, 0);
  bf16x8 v;
  memcpy(&v, emu::lds_ptr(a, 16), 16);
  return v;
}
inline void lds_write_b64(uint32_t a, u32x2 v) {
  if (a & 7) emu::fail("ds_write_b64 at unaligned LDS address %u", a);
  emu::lds_account(a, 8, 2);
  memcpy(emu::lds_ptr(a, 8), &v, 8);
}
inline void lds_write_b128(uint32_t a, u32x4 v) {
  if (a & 15) emu::fail("ds_write_b128 at unaligned LDS address %u", a);
  emu::lds_account(a, 16, 2);
  memcpy(emu::lds_ptr(a, 16), &v, 16);
}
inline u32x4 lds_read_u128(uint32_t a) {
  if (a & 15) emu::fail("ds_read_b128 at unaligned LDS address %u", a);
  emu::lds_account(a, 16, 0);
  u32x4 v;
  memcpy(&v, emu::lds_ptr(a, 16), 16);
  return v;
}
inline float lds_read_f32(uint32_t a) {
  if (a & 3) emu::fail("ds_read_b32 at unaligned LDS address %u", a);
  emu::lds_account(a, 4, 0);
  float v;
  memcpy(&v, emu::lds_ptr(a, 4), 4);
  return v;
}
// ds_read_b64_tr_b16: inside each group of 16 lanes, lane i receives element (i % 4) of the 8-byte
// rows addressed by lanes (i / 4), (i / 4) + 4, (i / 4) + 8, (i / 4) + 12 of the group.
inline bf16x4 lds_read_tr16_b64(uint32_t a) {
  if (a & 7) emu::fail("ds_read_b64_tr_b16 at unaligned LDS address %u", a);
  emu::lds_account(a, 8, 1);
  uint64_t row;
  memcpy(&row, emu::lds_ptr(a, 8), 8);
  const int par = emu::wave_rendezvous(&row, 8, 0x54523136u);
  const int l = emu::self()->lane, base = l & ~15, i = l & 15;
  bf16x4 out;
  for (int j = 0; j < 4; ++j) {
    const int src = base + (i / 4) + 4 * j;
    uint16_t e = 0xffff;                                     // a lane that is gone contributes a NaN pattern
    if (emu::wave_lane_live(src)) memcpy(&e, emu::wave_slot(par, src) + 2 * (i % 4), 2);
    __bf16 b;
    memcpy(&b, &e, 2);
    out[j] = b;
  }
  return out;
}
inline bf16x4 lds_read_tr16_b64(const void* shared_object) { return lds_read_tr16_b64(emu::lds_addr(shared_object)); }

inline int lane_id() { return emu::self()->lane; }
inline void wave_lds_order() { emu::wave_rendezvous(nullptr, 0, 0x4c44534fu); }

inline void dma_b128(const void* lane_src, uint32_t lds_base) {
  emu::dma_issue(lane_src, lds_base + 16u * (uint32_t)emu::self()->lane, 16);
}
template <int N>
inline void dma_b128_first_lanes(const void* lane_src, uint32_t lds_base) {
  if (emu::self()->lane < N) dma_b128(lane_src, lds_base);
  else emu::dma_issue(nullptr, 0, 0);                // the wavefront's instruction still counts for this lane's waits
}
inline void dma_b128(uint32_t lane_off, uint64_t wave_base, uint32_t lds_base) {
  emu::dma_issue(reinterpret_cast<const void*>(wave_base + lane_off), lds_base + 16u * (uint32_t)emu::self()->lane, 16);
}
inline void dma_b32(const void* lane_src, uint32_t lds_base) {
  emu::dma_issue(lane_src, lds_base + 4u * (uint32_t)emu::self()->lane, 4);
}
template <int N>
inline void wait_vmcnt() { emu::dma_wait(N); }

// (the emulator cannot see which moves were issued before the loads in question: it lands all of
// the lane's outstanding moves, which is what the callers' issue order guarantees on hardware)
template <typename... T> inline void wait_for_loads_of(const T&...) { emu::dma_wait(0); }
template <typename... T> inline void pin(T&...) {}
inline void pin_uniform(uint32_t&) {}

inline void shift_in_gt_u32(uint32_t& mask, uint32_t x, uint32_t y) { mask = 2u * mask + (x > y ? 1u : 0u); }
inline void shift_in_eq_u32(uint32_t& mask, uint32_t x, uint32_t y) { mask = 2u * mask + (x == y ? 1u : 0u); }

inline void store_b128_agent(float* p, f32x4 v) { memcpy(p, &v, 16); }

struct buffer_rsrc { const uint8_t* base; };
inline buffer_rsrc make_rsrc(const void* wave_uniform_base) { return buffer_rsrc{static_cast<const uint8_t*>(wave_uniform_base)}; }
inline f32x4 load_b128_agent(buffer_rsrc r, uint32_t byte_off) {
  f32x4 v;
  memcpy(&v, r.base + byte_off, 16);
  return v;
}

}  // namespace hw
}  // namespace smla
