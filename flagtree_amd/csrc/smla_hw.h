// gfx950 instructions the kernels issue that the compiler offers no (or no suitable) builtin for,
// and LDS access by 32-bit LDS address, in one place.  Included as <smla_hw.h>: the CPU emulator
// the kernels are tested on puts a header of the same name, with the same functions, ahead of this
// one on its include path, so the kernel sources themselves carry no conditional code.
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

// ---- LDS by address.  Swizzled layouts build addresses with integer xor, so they are kept as the
// 32-bit LDS addresses the hardware uses.
__device__ __forceinline__ uint32_t lds_addr(const void* shared_object) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t*)shared_object;
}
__device__ __forceinline__ bf16x8 lds_read_b128(uint32_t a) {
  return *(const __attribute__((address_space(3))) bf16x8*)(a);
}
__device__ __forceinline__ void lds_write_b64(uint32_t a, u32x2 v) {
  *(__attribute__((address_space(3))) u32x2*)(a) = v;
}
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
__device__ __forceinline__ void lds_write_b128(uint32_t a, u32x4 v) {
  *(__attribute__((address_space(3))) u32x4*)(a) = v;
}
__device__ __forceinline__ u32x4 lds_read_u128(uint32_t a) {
  return *(const __attribute__((address_space(3))) u32x4*)(a);
}
__device__ __forceinline__ float lds_read_f32(uint32_t a) {
  return *(const __attribute__((address_space(3))) float*)(a);
}
// ds_read_b64_tr_b16: inside each group of 16 lanes, lane i receives element (i % 4) of the 8-byte
// rows addressed by lanes (i / 4), (i / 4) + 4, (i / 4) + 8, (i / 4) + 12.
__device__ __forceinline__ bf16x4 lds_read_tr16_b64(uint32_t a) {
  short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(a));
  return __builtin_bit_cast(bf16x4, v);
}
__device__ __forceinline__ bf16x4 lds_read_tr16_b64(const void* shared_object) {
  short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(shared_object));
  return __builtin_bit_cast(bf16x4, v);
}

// This lane's position in its wavefront, from the hardware's lane counter (two instructions; a
// value the compiler does not connect with threadIdx, so it is recomputed where it is used).
__device__ __forceinline__ int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// Marks a point where lanes of ONE wavefront hand data to each other through LDS (one lane
// writes, another reads, no workgroup barrier in between).  Nothing is needed on the hardware: a
// wavefront's lanes execute an instruction together and its LDS accesses complete in program
// order; the compiler keeps the order because the accesses may alias.  The emulator, whose lanes
// run one after the other, synchronises them here.
__device__ __forceinline__ void wave_lds_order() {}

// ---- global -> LDS moves without staging registers.  Every lane fetches `bytes` from its own
// global address; the wavefront's 64 pieces land in consecutive LDS starting at `lds_base`
// (wave-uniform, goes through M0).  They complete in issue order and are counted by vmcnt like
// any other vector memory operation; nothing orders them against LDS reads but wait_vmcnt and
// a barrier.  Issued from inline assembly (no register output) so that the compiler does not
// serialise them against LDS reads of other ring slots.  The s_nop is the wait state the ISA asks
// for between a scalar write of M0 and a memory instruction that uses it as its LDS base (the
// compiler inserts it in its own code; inside an asm statement nobody does).
__device__ __forceinline__ void dma_b128(const void* lane_src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(lane_src), "s"(lds_base) : "memory", "m0");
}
// A move in which only lanes 0 .. N-1 take part (the others' LDS pieces stay as they are).  The
// execution mask is narrowed and restored around the instruction right here, so that no branch
// cuts the surrounding instruction stream in two; the move counts once for vmcnt like any other.
// Every lane of the wavefront must be active at the call.
template <int N>
__device__ __forceinline__ void dma_b128_first_lanes(const void* lane_src, uint32_t lds_base) {
  static_assert(N > 0 && N < 32, "the mask is written as a 32-bit literal");
  uint64_t saved;
  asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b64 exec, %0"
               : "=&s"(saved) : "v"(lane_src), "s"(lds_base), "n"((1u << N) - 1u) : "memory", "m0");
}
// scalar base + per-lane byte offset
__device__ __forceinline__ void dma_b128(uint32_t lane_off, uint64_t wave_base, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(wave_base), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void dma_b32(const void* lane_src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(lane_src), "s"(lds_base) : "memory", "m0");
}

// s_waitcnt vmcnt(N): at most N of this wavefront's vector memory operations still in flight
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Compiler fences on values (no instruction is emitted).
// wait_for_loads_of: the values are "used" here, so the compiler waits (s_waitcnt) for exactly the
// loads that produce them at this point.  Vector memory operations complete in issue order, so
// every global -> LDS move issued BEFORE those loads has landed as well; callers rely on that.
// pin: the values are "rewritten" here, so the arithmetic that produces them cannot sink below and
// what consumes them cannot rise above -- it keeps a slice of vector work between the two MFMAs
// it was written between.
template <typename... T>
__device__ __forceinline__ void wait_for_loads_of(const T&... v) { (..., [](const auto& x) { asm volatile("" ::"v"(x)); }(v)); }
template <typename... T>
__device__ __forceinline__ void pin(T&... v) { (..., [](auto& x) { asm volatile("" : "+v"(x)); }(v)); }
// the same for a wave-uniform value (it stays in a scalar register).  Also the way to keep what
// is derived from the value from being computed once, far ahead, and held in registers since.
__device__ __forceinline__ void pin_uniform(uint32_t& v) { asm volatile("" : "+s"(v)); }

// mask = 2 * mask + (x > y) / (x == y), unsigned: a compare into vcc and an add with carry-in, two
// vector instructions a bit (the compiler's own lowering takes three and a half); the wait state
// between a vcc write and its use as carry-in is spelled out.
__device__ __forceinline__ void shift_in_gt_u32(uint32_t& mask, uint32_t x, uint32_t y) {
  asm("v_cmp_gt_u32 vcc, %1, %2\n\ts_nop 1\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc" : "+v"(mask) : "v"(x), "v"(y) : "vcc");
}
__device__ __forceinline__ void shift_in_eq_u32(uint32_t& mask, uint32_t x, uint32_t y) {
  asm("v_cmp_eq_u32 vcc, %1, %2\n\ts_nop 1\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc" : "+v"(mask) : "v"(x), "v"(y) : "vcc");
}

// 16-byte store at agent scope (sc1: written through to the L2 every CU of the XCD shares).
// The s_nop covers the two wait states the ISA asks for between a store of more than 8 bytes and
// a vector instruction that overwrites the registers holding its data (the compiler, which would
// insert them for a store of its own, is free to reuse those registers right after the statement).
__device__ __forceinline__ void store_b128_agent(float* p, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

// 16-byte loads at agent scope through a buffer descriptor: loads the compiler can see (it counts
// them in flight and waits where a landing register is first read) that still carry sc1.
typedef __amdgpu_buffer_rsrc_t buffer_rsrc;
__device__ __forceinline__ buffer_rsrc make_rsrc(const void* wave_uniform_base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(wave_uniform_base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ f32x4 load_b128_agent(buffer_rsrc r, uint32_t byte_off) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 16 /* sc1 */));
}

}  // namespace hw
}  // namespace smla
