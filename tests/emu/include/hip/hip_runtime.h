// Stand-in for <hip/hip_runtime.h> when the kernel sources are compiled for the CPU emulator
// (test infrastructure only).  It gives the HIP language extensions, the handful of runtime calls
// and every gfx950 builtin the kernels use a meaning on the host.  Lane semantics follow the
// public CDNA ISA documentation; the register layouts of the matrix instructions and of the
// transposing LDS read are the ones stated in the kernels' own comments.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <type_traits>

#include "../../emu_runtime.h"

// ---- language extensions
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static __attribute__((section("emu_lds")))
#define HIP_KERNEL_NAME(...) __VA_ARGS__
#define __align__(n) __attribute__((aligned(n)))

typedef emu::Dim3 dim3;
#define threadIdx (emu::self()->tid)
#define blockIdx (emu::block_idx())
#define blockDim (emu::block_dim())
#define gridDim (emu::grid_dim())

// ---- runtime calls
typedef void* hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0 };
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2 };
enum { hipDeviceAttributeMultiprocessorCount = 1 };
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* v, int, int) { *v = emu::cu_count(); return hipSuccess; }
inline hipError_t hipMemcpyAsync(void* d, const void* s, size_t n, hipMemcpyKind, hipStream_t) { memcpy(d, s, n); return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emulated HIP error"; }
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
  emu::launch((grid), (block), [&]() { kernel(__VA_ARGS__); })

// ---- vector types
struct uint2 { uint32_t x, y; };
struct uint4 { uint32_t x, y, z, w; };
struct float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
struct ushort4 { uint16_t x, y, z, w; };
struct int2 { int32_t x, y; };
struct alignas(16) int4 { int32_t x, y, z, w; };
inline uint2 make_uint2(uint32_t x, uint32_t y) { return uint2{x, y}; }
inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{x, y, z, w}; }
inline float2 make_float2(float x, float y) { return float2{x, y}; }
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
inline int4 make_int4(int x, int y, int z, int w) { return int4{x, y, z, w}; }

// ---- scalar helpers
using std::max;
using std::min;
inline long long min(long long a, int b) { return a < b ? a : (long long)b; }
inline long long min(int a, long long b) { return a < b ? (long long)a : b; }
inline long min(long a, int b) { return a < b ? a : (long)b; }
inline long min(int a, long b) { return a < b ? (long)a : b; }
inline long long max(long long a, int b) { return a > b ? a : (long long)b; }
inline long long max(int a, long long b) { return a > b ? (long long)a : b; }
inline unsigned min(unsigned a, int b) { return a < (unsigned)b ? a : (unsigned)b; }
inline unsigned min(int a, unsigned b) { return (unsigned)a < b ? (unsigned)a : b; }
inline unsigned max(unsigned a, int b) { return a > (unsigned)b ? a : (unsigned)b; }
inline unsigned max(int a, unsigned b) { return (unsigned)a > b ? (unsigned)a : b; }
inline size_t min(size_t a, int b) { return a < (size_t)b ? a : (size_t)b; }
inline uint32_t __float_as_uint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
inline int __float_as_int(float f) { int u; memcpy(&u, &f, 4); return u; }
inline float __int_as_float(int u) { float f; memcpy(&f, &u, 4); return f; }
inline float __fmul_rn(float a, float b) { return a * b; }     // (built with -ffp-contract=off)
inline float __fadd_rn(float a, float b) { return a + b; }
inline float __fdiv_rn(float a, float b) { return a / b; }
inline float __expf(float x) { return expf(x); }
inline float __logf(float x) { return logf(x); }
inline int __popc(uint32_t v) { return __builtin_popcount(v); }
inline int __popcll(uint64_t v) { return __builtin_popcountll(v); }
inline int __clz(int v) { return v ? __builtin_clz((unsigned)v) : 32; }
inline int __ffs(int v) { return __builtin_ffs(v); }
inline int __ffsll(long long v) { return __builtin_ffsll(v); }

// ---- barriers and scheduling hints
inline void __syncthreads() { emu::block_barrier(); }
#define __builtin_amdgcn_sched_barrier(m) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_s_sleep(n) emu::poll_yield()   /* the kernels sleep only inside loops that poll another workgroup's writes */
#define __builtin_amdgcn_s_setprio(n) ((void)0)
#define __builtin_amdgcn_wave_barrier() ((void)emu::wave_rendezvous(nullptr, 0, 0x57415645u))

// ---- atomics (one OS thread runs everything: plain accesses are atomic)
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __HIP_MEMORY_SCOPE_WORKGROUP 0
#define __HIP_MEMORY_SCOPE_SYSTEM 0
namespace emu {
template <typename T> inline T atomic_load(const T* p) { return *const_cast<const volatile T*>(p); }
template <typename T, typename U> inline void atomic_store(T* p, U v) { *const_cast<volatile T*>(p) = (T)v; }
template <typename T, typename U> inline T atomic_add(T* p, U v) { T o = *p; *p = (T)(o + (T)v); return o; }
template <typename T, typename U> inline T atomic_or(T* p, U v) { T o = *p; *p = (T)(o | (T)v); return o; }
template <typename T, typename U> inline T atomic_max(T* p, U v) { T o = *p; if ((T)v > o) *p = (T)v; return o; }
}  // namespace emu
#define __hip_atomic_load(p, order, scope) emu::atomic_load(p)
#define __hip_atomic_store(p, v, order, scope) emu::atomic_store(p, v)
#define __hip_atomic_fetch_add(p, v, order, scope) emu::atomic_add(p, v)
#define __hip_atomic_fetch_or(p, v, order, scope) emu::atomic_or(p, v)
template <typename T, typename U> inline T atomicAdd(T* p, U v) { return emu::atomic_add(p, v); }
template <typename T, typename U> inline T atomicOr(T* p, U v) { return emu::atomic_or(p, v); }
template <typename T, typename U> inline T atomicMax(T* p, U v) { return emu::atomic_max(p, v); }

// ---- cross-lane operations
namespace emu {
template <typename T>
inline T lane_read(T v, int src, uint32_t tag) {           // every lane posts v, reads lane `src`'s (own value if src is not live)
  static_assert(sizeof(T) <= kSlotBytes && std::is_trivially_copyable<T>::value, "lane_read operand");
  const int par = wave_rendezvous(&v, sizeof(T), tag);
  T r = v;
  if (src >= 0 && src < kWave && wave_lane_live(src)) memcpy(&r, wave_slot(par, src), sizeof(T));
  return r;
}
inline uint64_t ballot(bool pred, uint32_t tag) {
  const uint8_t b = pred ? 1 : 0;
  const int par = wave_rendezvous(&b, 1, tag);
  uint64_t m = 0;
  for (int l = 0; l < kWave; ++l)
    if (wave_lane_live(l) && wave_slot(par, l)[0]) m |= 1ull << l;
  return m;
}
}  // namespace emu
template <typename T> inline T __shfl(T v, int src, int width = 64) {
  const int l = emu::self()->lane;
  return emu::lane_read(v, (l & ~(width - 1)) | (src & (width - 1)), 0x5348464cu);
}
template <typename T> inline T __shfl_xor(T v, int mask, int width = 64) {
  const int l = emu::self()->lane;
  const int src = l ^ mask;
  return emu::lane_read(v, (src & ~(width - 1)) == (l & ~(width - 1)) ? src : l, 0x53485858u);
}
template <typename T> inline T __shfl_up(T v, unsigned delta, int width = 64) {
  const int l = emu::self()->lane;
  const int src = l - (int)delta;
  return emu::lane_read(v, src >= (l & ~(width - 1)) ? src : l, 0x53485550u);
}
template <typename T> inline T __shfl_down(T v, unsigned delta, int width = 64) {
  const int l = emu::self()->lane;
  const int src = l + (int)delta;
  return emu::lane_read(v, src < (l & ~(width - 1)) + width ? src : l, 0x5348444eu);
}
inline uint64_t __ballot(int pred) { return emu::ballot(pred != 0, 0x42414c4cu); }
inline int __any(int pred) { return emu::ballot(pred != 0, 0x414e5920u) != 0; }
inline int __all(int pred) {
  const uint64_t yes = emu::ballot(pred != 0, 0x414c4c20u), live = emu::ballot(true, 0x414c4c21u);
  return yes == live;
}
inline int emu_readlane(int v, int src) { return emu::lane_read(v, src, 0x52444c4eu); }
inline int emu_readfirstlane(int v) {
  const uint64_t live = emu::ballot(true, 0x5246314cu);
  return emu::lane_read(v, __builtin_ctzll(live), 0x5246324cu);
}
#define __builtin_amdgcn_readlane(v, l) emu_readlane((int)(v), (l))
#define __builtin_amdgcn_readfirstlane(v) emu_readfirstlane((int)(v))

// v_mov_b32 with a data-parallel-primitive control: result = the source lane's `src`, or `old`
// where the lane's row / bank is masked off or the source lane does not exist (0 with bound_ctrl).
inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  const int l = emu::self()->lane, row = l >> 4, in_row = l & 15;
  int from = -1;                                             // -1: no source lane
  if (ctrl < 0x100) from = (l & ~3) | ((ctrl >> (2 * (l & 3))) & 3);                 // quad_perm
  else if (ctrl >= 0x101 && ctrl <= 0x10f) { const int s = in_row + (ctrl - 0x100); from = s < 16 ? (row << 4) | s : -1; }   // row_shl
  else if (ctrl >= 0x111 && ctrl <= 0x11f) { const int s = in_row - (ctrl - 0x110); from = s >= 0 ? (row << 4) | s : -1; }   // row_shr
  else if (ctrl >= 0x121 && ctrl <= 0x12f) from = (row << 4) | ((in_row - (ctrl - 0x120)) & 15);                              // row_ror
  else if (ctrl == 0x130) from = l + 1 < 64 ? l + 1 : -1;                            // wave_shl:1
  else if (ctrl == 0x134) from = (l + 1) & 63;                                       // wave_rol:1
  else if (ctrl == 0x138) from = l - 1;                                              // wave_shr:1
  else if (ctrl == 0x13c) from = (l - 1) & 63;                                       // wave_ror:1
  else if (ctrl == 0x140) from = (row << 4) | (15 - in_row);                         // row_mirror
  else if (ctrl == 0x141) from = (l & ~7) | (7 - (l & 7));                           // row_half_mirror
  else if (ctrl == 0x142) from = row > 0 ? ((row - 1) << 4) | 15 : -2;               // row_bcast:15: every lane of a row gets the row below's last lane (-2: keeps old)
  else if (ctrl == 0x143) from = l >= 32 ? 31 : -2;                                  // row_bcast:31: rows 2 and 3 get lane 31
  else emu::fail("update_dpp: control 0x%x is not modelled", ctrl);
  const int par = emu::wave_rendezvous(&src, 4, 0x44505000u | (uint32_t)ctrl);
  const bool enabled = ((row_mask >> row) & 1) && ((bank_mask >> (in_row >> 2)) & 1);
  if (!enabled || from == -2) return old;
  if (from < 0 || !emu::wave_lane_live(from)) return bound_ctrl ? 0 : old;
  int r;
  memcpy(&r, emu::wave_slot(par, from), 4);
  return r;
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) emu_update_dpp((old), (src), (ctrl), (rm), (bm), (bc))

// ---- arithmetic builtins
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)           /* v_log_f32 is the base-2 logarithm */
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_sqrtf(x) sqrtf(x)
#define __builtin_amdgcn_fmed3f(a, b, c) fmaxf(fminf(fmaxf((a), (b)), (c)), fminf((a), (b)))

namespace emu {
typedef __attribute__((ext_vector_type(2))) float v2f;
typedef __attribute__((ext_vector_type(4))) float v4f;
typedef __attribute__((ext_vector_type(16))) float v16f;
typedef __attribute__((ext_vector_type(2))) __bf16 v2bf;
typedef __attribute__((ext_vector_type(8))) __bf16 v8bf;
typedef __attribute__((ext_vector_type(4))) short v4s;

inline float e4m3fn_to_f32(uint32_t c) {                     // OCP e4m3fn: bias 7, no infinities, 0x7f / 0xff = NaN
  const uint32_t e = (c >> 3) & 15u, m = c & 7u;
  float v;
  if (e == 0) v = (float)m * 0x1p-9f;
  else if (e == 15u && m == 7u) v = NAN;
  else v = ldexpf((float)(8 + m), (int)e - 10);
  return (c & 0x80u) ? -v : v;
}
inline uint32_t f32_to_e4m3fn(float x) {                     // round to nearest even, saturating, NaN -> 0x7f
  uint32_t u;
  memcpy(&u, &x, 4);
  const uint32_t sign = (u >> 24) & 0x80u;
  float a = fabsf(x);
  if (a != a) return 0x7fu | sign;
  if (a > 448.f) a = 448.f;
  uint32_t code;
  if (a < 0x1p-6f) code = (uint32_t)lrintf(a * 512.0f);
  else {
    uint32_t b;
    memcpy(&b, &a, 4);
    b += 0x7ffffu + ((b >> 20) & 1u);
    code = (b >> 20) - (120u << 3);
    if (code > 0x7eu) code = 0x7eu;
  }
  return code | sign;
}
inline float bf16_round(float f) { return (float)(__bf16)f; }
inline v2f cvt_pk_f32_fp8(uint32_t w, bool hi) {
  const uint32_t h = hi ? w >> 16 : w;
  return v2f{e4m3fn_to_f32(h & 0xff), e4m3fn_to_f32((h >> 8) & 0xff)};
}
inline v2bf cvt_scalef32_pk_bf16_fp8(uint32_t w, float scale, bool hi) {
  const v2f f = cvt_pk_f32_fp8(w, hi);
  v2bf r;
  r[0] = (__bf16)(f[0] * scale);
  r[1] = (__bf16)(f[1] * scale);
  return r;
}
inline uint32_t cvt_pk_fp8_f32(float a, float b, uint32_t old, bool hi) {
  const uint32_t pk = f32_to_e4m3fn(a) | (f32_to_e4m3fn(b) << 8);
  return hi ? (old & 0x0000ffffu) | (pk << 16) : (old & 0xffff0000u) | pk;
}

// D = A . B + C over the whole wavefront.  Every lane posts its A and B fragments and computes the
// D elements it owns.  A[m][k]: lane m + M * (k / kpl) holds k % kpl; B[k][n] likewise with n.
inline float bf16_bits_as_f32(uint16_t b) { const uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
template <int M, int K, int KPL, int NOUT, typename Frag, typename Acc>
inline Acc mfma(Frag a, Frag b, Acc c, uint32_t tag) {
  static_assert(sizeof(Frag) == 2 * KPL, "fragment = KPL 16-bit values");
  struct Post { Frag a, b; } post{a, b};
  count_mfma(M, K);
  const int par = wave_rendezvous(&post, sizeof(post), tag);
  const int l = self()->lane, n = l % M;
  // column n of B once: K values
  float bcol[K];
  for (int kb = 0; kb < K / KPL; ++kb) {
    uint16_t bits[KPL];
    memcpy(bits, wave_slot(par, n + M * kb) + sizeof(Frag), sizeof(bits));
    for (int j = 0; j < KPL; ++j) bcol[kb * KPL + j] = bf16_bits_as_f32(bits[j]);
  }
  Acc d = c;
  for (int r = 0; r < NOUT; ++r) {
    const int m = M == 32 ? 8 * (r / 4) + 4 * (l / 32) + r % 4 : 4 * (l / 16) + r;
    float sum = 0.f;
    for (int kb = 0; kb < K / KPL; ++kb) {
      uint16_t bits[KPL];
      memcpy(bits, wave_slot(par, m + M * kb), sizeof(bits));
      for (int j = 0; j < KPL; ++j) sum += bf16_bits_as_f32(bits[j]) * bcol[kb * KPL + j];
    }
    d[r] = c[r] + sum;
  }
  return d;
}

// D = A . B + C, 16 x 16 x (4 * BYTES), over fp8 (e4m3fn) operands.  Lane m + 16 g holds BYTES
// values of row m of A (of column n of B).  Which k a (g, byte) pair stands for is the same
// function for A and for B, so the sum over all pairs does not depend on it, and neither does a
// kernel that loads both operands by the same rule.  Products of two e4m3 values are exact in
// fp32; they are summed in fp32 (the hardware's order is its own: results agree to rounding).
// `scaled`: each operand is multiplied by 2^(e - 127), e its lane's scale byte; the model holds
// for scale bytes that are the same in every lane (which lane's byte serves which block of k is
// then immaterial) and refuses anything else.
typedef __attribute__((ext_vector_type(8))) int v8i;
template <int BYTES, typename Frag>
inline v4f mfma16_fp8(Frag a, Frag b, v4f c, bool scaled, uint32_t scale_a, uint32_t scale_b, uint32_t tag) {
  static_assert(sizeof(Frag) == BYTES, "fragment = BYTES fp8 values");
  struct Post { Frag a, b; uint32_t sa, sb; } post{a, b, scale_a & 0xffu, scale_b & 0xffu};
  count_mfma(16, 4 * BYTES);
  const int par = wave_rendezvous(&post, sizeof(post), tag);
  const int l = self()->lane, n = l % 16;
  float factor = 1.f;
  if (scaled) {
    for (int src = 0; src < 64; ++src) {
      if (!wave_lane_live(src)) continue;
      Post other;
      memcpy(&other, wave_slot(par, src), sizeof(other));
      if (other.sa != post.sa || other.sb != post.sb) fail("scaled fp8 MFMA with scale bytes that differ between lanes: not modelled");
    }
    factor = ldexpf(1.f, (int)post.sa - 127 + (int)post.sb - 127);
  }
  float bcol[4 * BYTES];
  for (int g = 0; g < 4; ++g) {
    uint8_t bytes[BYTES];
    memcpy(bytes, wave_slot(par, n + 16 * g) + offsetof(Post, b), BYTES);
    for (int j = 0; j < BYTES; ++j) bcol[g * BYTES + j] = e4m3fn_to_f32(bytes[j]);
  }
  v4f d = c;
  for (int r = 0; r < 4; ++r) {
    const int m = 4 * (l / 16) + r;
    float sum = 0.f;
    for (int g = 0; g < 4; ++g) {
      uint8_t bytes[BYTES];
      memcpy(bytes, wave_slot(par, m + 16 * g), BYTES);
      for (int j = 0; j < BYTES; ++j) sum += e4m3fn_to_f32(bytes[j]) * bcol[g * BYTES + j];
    }
    d[r] = c[r] + factor * sum;
  }
  return d;
}
inline v4f mfma_scale_16x16x128_f8f6f4(v8i a, v8i b, v4f c, int cbsz, int blgp, int opsel_a, int scale_a, int opsel_b, int scale_b) {
  if (cbsz != 0 || blgp != 0) fail("scaled MFMA: only e4m3 operands (cbsz = blgp = 0) are modelled");
  return mfma16_fp8<32, v8i>(a, b, c, true, (uint32_t)scale_a >> (8 * (opsel_a & 3)), (uint32_t)scale_b >> (8 * (opsel_b & 3)), 0x4d463830u);
}
// v_perm_b32: byte i of the result is byte sel[i] of the 8 bytes {b = bytes 0..3, a = bytes 4..7};
// selector 0x0c gives 0x00.  (The sign-replicating selectors 8 .. 11 and 0x0d .. are not modelled.)
inline uint32_t perm_b32(uint32_t a, uint32_t b, uint32_t sel) {
  const uint64_t both = ((uint64_t)a << 32) | b;
  uint32_t out = 0;
  for (int i = 0; i < 4; ++i) {
    const uint32_t s = (sel >> (8 * i)) & 0xffu;
    uint32_t byte;
    if (s < 8) byte = (uint32_t)(both >> (8 * s)) & 0xffu;
    else if (s == 0x0c) byte = 0;
    else fail("v_perm_b32 selector %u is not modelled", s);
    out |= byte << (8 * i);
  }
  return out;
}
}  // namespace emu
#define __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, b, c, x, y, z) \
  emu::mfma16_fp8<8, long>((a), (b), (c), false, 127u, 127u, 0x4d463833u)
#define __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, cbsz, blgp, opa, sa, opb, sb) \
  emu::mfma_scale_16x16x128_f8f6f4((a), (b), (c), (cbsz), (blgp), (opa), (sa), (opb), (sb))
#define __builtin_amdgcn_perm(a, b, sel) emu::perm_b32((a), (b), (sel))
#define __builtin_amdgcn_cvt_pk_f32_fp8(w, hi) emu::cvt_pk_f32_fp8((w), (hi))
#define __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, s, hi) emu::cvt_scalef32_pk_bf16_fp8((w), (s), (hi))
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, hi) emu::cvt_pk_fp8_f32((a), (b), (old), (hi))
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) \
  emu::mfma<16, 32, 8, 4, emu::v8bf, emu::v4f>((a), (b), (c), 0x4d313633u)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) \
  emu::mfma<32, 16, 8, 16, emu::v8bf, emu::v16f>((a), (b), (c), 0x4d333231u)
#define __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, x, y, z) \
  emu::mfma<16, 16, 4, 4, emu::v4s, emu::v4f>((a), (b), (c), 0x4d313631u)
