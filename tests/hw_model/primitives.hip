// Hardware-model probes (test infrastructure; the product never loads this library).
//
// One wavefront executes ONE of the machine-specific primitives the kernels are built from -- a
// matrix instruction, the transposing LDS read, a global -> LDS move, a DPP move, an fp8
// conversion, the agent-scope accesses -- on operands the test hands to every lane, and writes
// back what every lane received.  The same source is built for gfx950 and for the CPU emulator
// (tests/emu); the GPU test runs both on the same bytes and compares the answers, so a place where
// the emulator's model of an instruction differs from the instruction is found by itself, apart
// from any kernel's logic.
//
// Every probe is one workgroup of 64 lanes.  Lane l reads the 256-byte record l of `in` and writes
// the 256-byte record l of `out`; both buffers are exactly 64 records long.  No probe computes an
// address from data it has not range-checked: offsets taken from a record are masked into the
// buffer they index.
#include <hip/hip_runtime.h>
#include <smla_hw.h>
#include <stdint.h>

#include "primitives.h"

namespace {

using namespace smla::hw;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) int i32x8;

constexpr int kRecord = HWM_RECORD_BYTES;
constexpr int kLanes = HWM_LANES;
constexpr int kLdsBytes = 4096;
constexpr uint32_t kDmaLdsBase = 256;          // moves land here, not at the start of the array: the base goes through M0

template <typename T>
__device__ __forceinline__ T get(const uint8_t* p) { return *reinterpret_cast<const T*>(p); }
template <typename T>
__device__ __forceinline__ void put(uint8_t* p, T v) { *reinterpret_cast<T*>(p) = v; }

// every lane writes 64 bytes of LDS, so that the wavefront fills all 4096
__device__ __forceinline__ void fill_lds(uint8_t* s_mem, int lane, const uint8_t* src64) {
#pragma unroll
  for (int i = 0; i < 4; ++i) put<u32x4>(s_mem + 64 * lane + 16 * i, src64 ? get<u32x4>(src64 + 16 * i) : u32x4{0xEEEEEEEEu, 0xEEEEEEEEu, 0xEEEEEEEEu, 0xEEEEEEEEu});
}
// ... and reads the first 2048 back, 32 bytes a lane
__device__ __forceinline__ void dump_lds(const uint8_t* s_mem, int lane, uint8_t* o) {
  put<u32x4>(o, get<u32x4>(s_mem + 32 * lane));
  put<u32x4>(o + 16, get<u32x4>(s_mem + 32 * lane + 16));
}

template <int W>
__global__ __launch_bounds__(64) void probe_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) uint8_t s_mem[kLdsBytes];
  const int lane = threadIdx.x;
  const uint8_t* r = in + kRecord * lane;
  uint8_t* o = out + kRecord * lane;

  if constexpr (W == HWM_MFMA_16X16X32_BF16) {
    put<f32x4>(o, __builtin_amdgcn_mfma_f32_16x16x32_bf16(get<bf16x8>(r), get<bf16x8>(r + 16), get<f32x4>(r + 32), 0, 0, 0));
  } else if constexpr (W == HWM_MFMA_32X32X16_BF16) {
    put<f32x16>(o, __builtin_amdgcn_mfma_f32_32x32x16_bf16(get<bf16x8>(r), get<bf16x8>(r + 16), get<f32x16>(r + 64), 0, 0, 0));
  } else if constexpr (W == HWM_MFMA_16X16X16_BF16) {
    put<f32x4>(o, __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(get<short4v>(r), get<short4v>(r + 8), get<f32x4>(r + 16), 0, 0, 0));
  } else if constexpr (W == HWM_LDS_READ_TR16_B64) {
    fill_lds(s_mem, lane, r);
    __syncthreads();
    const uint32_t a = get<uint32_t>(r + 64) & (kLdsBytes - 8);          // 8-byte aligned, inside the array
    put<bf16x4>(o, lds_read_tr16_b64(lds_addr(s_mem) + a));
  } else if constexpr (W == HWM_DMA_B128 || W == HWM_DMA_B128_FIRST_8_LANES || W == HWM_DMA_B128_BASE_PLUS_OFFSET || W == HWM_DMA_B32) {
    fill_lds(s_mem, lane, nullptr);
    __syncthreads();
    const uint32_t off = get<uint32_t>(r) & (kRecord * kLanes - 16);     // 16-byte aligned, inside `in`
    const uint32_t dst = lds_addr(s_mem) + kDmaLdsBase;
    if constexpr (W == HWM_DMA_B128) dma_b128(in + off, dst);
    if constexpr (W == HWM_DMA_B128_FIRST_8_LANES) dma_b128_first_lanes<8>(in + off, dst);
    if constexpr (W == HWM_DMA_B128_BASE_PLUS_OFFSET) dma_b128(off, (uint64_t)(uintptr_t)in, dst);
    if constexpr (W == HWM_DMA_B32) dma_b32(in + off, dst);
    wait_vmcnt<0>();
    __syncthreads();
    dump_lds(s_mem, lane, o);
  } else if constexpr (W == HWM_DPP_MOVES) {
    const int v = get<int>(r);
    int* d = reinterpret_cast<int*>(o);
    d[0] = __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr 1, 2, 4, 8
    d[1] = __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);
    d[2] = __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);
    d[3] = __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);
    d[4] = __builtin_amdgcn_update_dpp(0, v, 0x121, 0xf, 0xf, false);   // row_ror 1, 2, 4, 8
    d[5] = __builtin_amdgcn_update_dpp(0, v, 0x122, 0xf, 0xf, false);
    d[6] = __builtin_amdgcn_update_dpp(0, v, 0x124, 0xf, 0xf, false);
    d[7] = __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false);
    d[8] = __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast 15 into rows 1 and 3
    d[9] = __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast 31 into rows 2 and 3
    d[10] = __builtin_amdgcn_readlane(v, 37);
    d[11] = __builtin_amdgcn_readfirstlane(v);
    d[12] = lane_id();
    const unsigned long long b = __ballot((v & 1) != 0);
    d[13] = (int)(uint32_t)b;
    d[14] = (int)(uint32_t)(b >> 32);
    d[15] = __shfl_up(v, 1u);
    d[16] = __shfl_xor(v, 21);
  } else if constexpr (W == HWM_FP8_CONVERSIONS) {
    const uint32_t w = get<uint32_t>(r);                                 // four e4m3 codes
    put<f32x2>(o, __builtin_amdgcn_cvt_pk_f32_fp8(w, false));
    put<f32x2>(o + 8, __builtin_amdgcn_cvt_pk_f32_fp8(w, true));
    put<uint32_t>(o + 16, __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false)));
    put<uint32_t>(o + 20, __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)));
    const float a = get<float>(r + 16), b = get<float>(r + 20);          // two floats to e4m3, into either half of a word
    put<uint32_t>(o + 24, (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)0xA5A5A5A5, false));
    put<uint32_t>(o + 28, (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)0xA5A5A5A5, true));
  } else if constexpr (W == HWM_COMPARE_AND_SHIFT_IN) {
    uint32_t gt = get<uint32_t>(r + 8), eq = gt;
    shift_in_gt_u32(gt, get<uint32_t>(r), get<uint32_t>(r + 4));
    shift_in_eq_u32(eq, get<uint32_t>(r), get<uint32_t>(r + 4));
    put<uint32_t>(o, gt);
    put<uint32_t>(o + 4, eq);
  } else if constexpr (W == HWM_AGENT_SCOPE_ACCESSES) {
    store_b128_agent(reinterpret_cast<float*>(o), get<f32x4>(r));
    const buffer_rsrc rsrc = make_rsrc(in);
    put<f32x4>(o + 16, load_b128_agent(rsrc, (uint32_t)(kRecord * lane + 16)));
  } else if constexpr (W == HWM_MFMA_16X16X32_FP8) {
    put<f32x4>(o, __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(get<long>(r), get<long>(r + 8), get<f32x4>(r + 16), 0, 0, 0));
  } else if constexpr (W == HWM_MFMA_SCALE_16X16X128_FP8) {
    // e4m3 operands (format codes 0), scale bytes 2^0 for A and 2^-4 for B, the same in every lane and every byte
    put<f32x4>(o, __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(get<i32x8>(r), get<i32x8>(r + 32), get<f32x4>(r + 64), 0, 0,
                                                                  0, 0x7f7f7f7f, 0, 0x7b7b7b7b));
  } else if constexpr (W == HWM_BYTE_PERMUTE) {
    const uint32_t a = get<uint32_t>(r), b = get<uint32_t>(r + 4);
    put<uint32_t>(o, __builtin_amdgcn_perm(a, b, 0x06040200u));
    put<uint32_t>(o + 4, __builtin_amdgcn_perm(a, b, 0x07050301u));
  } else if constexpr (W == HWM_APPROXIMATE_FUNCTIONS) {
    float* d = reinterpret_cast<float*>(o);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float x = get<float>(r + 4 * i);
      d[i] = __builtin_amdgcn_exp2f(x);
      d[4 + i] = __builtin_amdgcn_logf(fabsf(x) + 1e-3f);
      d[8 + i] = __builtin_amdgcn_rcpf(fabsf(x) + 1e-3f);
    }
  }
}

template <int W>
int launch(const void* in, void* out, hipStream_t s) {
  hipLaunchKernelGGL(HIP_KERNEL_NAME(probe_kernel<W>), dim3(1), dim3(kLanes), 0, s, static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out));
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

extern "C" int hwm_run(int which, const void* in, void* out, void* stream) {
  if (!in || !out) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (which) {
    case HWM_MFMA_16X16X32_BF16: return launch<HWM_MFMA_16X16X32_BF16>(in, out, s);
    case HWM_MFMA_32X32X16_BF16: return launch<HWM_MFMA_32X32X16_BF16>(in, out, s);
    case HWM_MFMA_16X16X16_BF16: return launch<HWM_MFMA_16X16X16_BF16>(in, out, s);
    case HWM_LDS_READ_TR16_B64: return launch<HWM_LDS_READ_TR16_B64>(in, out, s);
    case HWM_DMA_B128: return launch<HWM_DMA_B128>(in, out, s);
    case HWM_DMA_B128_FIRST_8_LANES: return launch<HWM_DMA_B128_FIRST_8_LANES>(in, out, s);
    case HWM_DMA_B128_BASE_PLUS_OFFSET: return launch<HWM_DMA_B128_BASE_PLUS_OFFSET>(in, out, s);
    case HWM_DMA_B32: return launch<HWM_DMA_B32>(in, out, s);
    case HWM_DPP_MOVES: return launch<HWM_DPP_MOVES>(in, out, s);
    case HWM_FP8_CONVERSIONS: return launch<HWM_FP8_CONVERSIONS>(in, out, s);
    case HWM_COMPARE_AND_SHIFT_IN: return launch<HWM_COMPARE_AND_SHIFT_IN>(in, out, s);
    case HWM_AGENT_SCOPE_ACCESSES: return launch<HWM_AGENT_SCOPE_ACCESSES>(in, out, s);
    case HWM_APPROXIMATE_FUNCTIONS: return launch<HWM_APPROXIMATE_FUNCTIONS>(in, out, s);
    case HWM_MFMA_16X16X32_FP8: return launch<HWM_MFMA_16X16X32_FP8>(in, out, s);
    case HWM_MFMA_SCALE_16X16X128_FP8: return launch<HWM_MFMA_SCALE_16X16X128_FP8>(in, out, s);
    case HWM_BYTE_PERMUTE: return launch<HWM_BYTE_PERMUTE>(in, out, s);
    default: return -3;
  }
}

extern "C" int hwm_count(void) { return HWM_COUNT; }
