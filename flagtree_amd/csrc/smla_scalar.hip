// Exact-fp32 scalar sparse-MLA forward, the gather/translate kernel, the split merge and
// the fp8 KV-record writer.  These are the simple, obviously-correct device kernels; the
// MFMA kernels in smla_mfma_*.hip are checked against them at full size.
#include "smla_common.h"

namespace smla {

template <int FMT> struct RowReader;

template <> struct RowReader<SMLA_KV_BF16> {
  static constexpr int kRowBytes = kRowBytesBf16;
  __device__ static float get(const uint8_t* row, int d) {
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(row)[d]);
  }
};
template <> struct RowReader<SMLA_KV_F32> {
  static constexpr int kRowBytes = kDqk * 4;
  __device__ static float get(const uint8_t* row, int d) {
    return reinterpret_cast<const float*>(row)[d];
  }
};
template <> struct RowReader<SMLA_KV_FP8_B128> {
  static constexpr int kRowBytes = kRowBytesFp8;
  __device__ static float get(const uint8_t* row, int d) {
    if (d < kDv) {
      const float scale = reinterpret_cast<const float*>(row + kFp8ScaleOff)[d >> 7];
      return e4m3_to_f32(row[d]) * scale;
    }
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(row + kFp8RopeOff)[d - kDv]);
  }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

constexpr int kScalarThreads = 256;
constexpr int kScalarChunk = 2048;   // top-k entries processed per pass (online softmax across passes)

// One workgroup per (head, token).  Scores in fp32, softmax in fp32, PV in fp32.
template <int FMT, bool QF32>
__global__ __launch_bounds__(kScalarThreads) void fwd_scalar_kernel(Params p) {
  using R = RowReader<FMT>;
  __shared__ float s_q[kDqk];
  __shared__ float s_score[kScalarChunk];
  __shared__ int32_t s_row[kScalarChunk];
  __shared__ float s_red[8];

  const int h = blockIdx.x, t = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int seq = t / p.tokens_per_seq;
  const uint8_t* kv = static_cast<const uint8_t*>(p.kv);

  for (int d = tid; d < kDqk; d += kScalarThreads) {
    const size_t o = ((size_t)t * p.n_heads + h) * kDqk + d;
    s_q[d] = QF32 ? static_cast<const float*>(p.q)[o]
                  : bf16_bits_to_f32(static_cast<const uint16_t*>(p.q)[o]);
  }

  float m_run = -INFINITY, l_run = 0.f;
  float acc0 = 0.f, acc1 = 0.f;   // dv columns tid and tid + 256

  for (int base = 0; base < p.topk; base += kScalarChunk) {
    const int n = min(kScalarChunk, p.topk - base);
    __syncthreads();
    for (int j = tid; j < n; j += kScalarThreads)
      s_row[j] = translate_index(p, seq, list_entry(p, t, seq, base + j));
    __syncthreads();
    // scores: one wave per row, lanes stride the 576 columns
    for (int j = wave; j < n; j += kScalarThreads / 64) {
      const int32_t r = s_row[j];
      float part = 0.f;
      if (r >= 0) {
        const uint8_t* row = kv + (size_t)r * R::kRowBytes;
#pragma unroll
        for (int i = 0; i < kDqk / 64; ++i) part += s_q[lane + 64 * i] * R::get(row, lane + 64 * i);
      }
      part = wave_sum(part);
      if (lane == 0) {
        float sc = part * p.sm_scale;
        if (p.logit_cap > 0.f) sc = p.logit_cap * tanhf(sc / p.logit_cap);
        s_score[j] = r >= 0 ? sc : -INFINITY;
      }
    }
    __syncthreads();
    float m_loc = -INFINITY;
    for (int j = tid; j < n; j += kScalarThreads) m_loc = fmaxf(m_loc, s_score[j]);
    m_loc = wave_max(m_loc);
    if (lane == 0) s_red[wave] = m_loc;
    __syncthreads();
    float m_new = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    m_new = fmaxf(m_new, m_run);
    __syncthreads();
    if (m_new == -INFINITY) continue;            // nothing valid so far
    const float alpha = expf(m_run - m_new);     // exp(-inf) = 0 on the first valid pass
    float l_loc = 0.f;
    for (int j = tid; j < n; j += kScalarThreads) {
      const float pj = s_row[j] >= 0 ? expf(s_score[j] - m_new) : 0.f;
      s_score[j] = pj;
      l_loc += pj;
    }
    l_loc = wave_sum(l_loc);
    if (lane == 0) s_red[4 + wave] = l_loc;
    __syncthreads();
    l_run = l_run * alpha + (s_red[4] + s_red[5] + s_red[6] + s_red[7]);
    m_run = m_new;
    acc0 *= alpha;
    acc1 *= alpha;
    for (int j = 0; j < n; ++j) {
      const int32_t r = s_row[j];
      if (r < 0) continue;
      const float pj = s_score[j];
      const uint8_t* row = kv + (size_t)r * R::kRowBytes;
      acc0 += pj * R::get(row, tid);
      acc1 += pj * R::get(row, tid + 256);
    }
  }

  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  const size_t ob = ((size_t)t * p.n_heads + h) * kDv;
  if (QF32) {
    static_cast<float*>(p.out)[ob + tid] = acc0 * inv;
    static_cast<float*>(p.out)[ob + tid + 256] = acc1 * inv;
  } else {
    static_cast<uint16_t*>(p.out)[ob + tid] = f32_to_bf16_bits(acc0 * inv);
    static_cast<uint16_t*>(p.out)[ob + tid + 256] = f32_to_bf16_bits(acc1 * inv);
  }
  if (tid == 0) p.lse[(size_t)t * p.n_heads + h] = l_run > 0.f ? m_run + logf(l_run) : -INFINITY;
}

int launch_fwd_scalar(int kv_format, const Params& p, hipStream_t s) {
  dim3 grid(p.n_heads, p.n_tokens), block(kScalarThreads);
  switch (kv_format) {
    case SMLA_KV_BF16: hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_scalar_kernel<SMLA_KV_BF16, false>), grid, block, 0, s, p); break;
    case SMLA_KV_FP8_B128: hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_scalar_kernel<SMLA_KV_FP8_B128, false>), grid, block, 0, s, p); break;
    case SMLA_KV_F32: hipLaunchKernelGGL(HIP_KERNEL_NAME(fwd_scalar_kernel<SMLA_KV_F32, true>), grid, block, 0, s, p); break;
    default: return SMLA_EINVAL_SHAPE;
  }
  return hip_status(hipGetLastError());
}

// ---------------------------------------------------------------------------------------
// translate + mask + gather: one wave per top-k entry, 16-byte chunks across lanes.
__global__ __launch_bounds__(256) void gather_kernel(Params p, int row_bytes, int32_t* phys_out,
                                                     uint8_t* rows_out) {
  const int t = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (j >= p.topk) return;
  const int seq = t / p.tokens_per_seq;
  const size_t e = (size_t)t * p.topk + j;
  const int32_t r = translate_index(p, seq, list_entry(p, t, seq, j));
  if (lane == 0) phys_out[e] = r;
  if (rows_out == nullptr) return;
  const int n_chunks = row_bytes >> 4;
  const uint4* src = reinterpret_cast<const uint4*>(static_cast<const uint8_t*>(p.kv) +
                                                    (size_t)(r >= 0 ? r : 0) * row_bytes);
  uint4* dst = reinterpret_cast<uint4*>(rows_out + e * row_bytes);
  for (int c = lane; c < n_chunks; c += 64) dst[c] = r >= 0 ? src[c] : make_uint4(0, 0, 0, 0);
}

int launch_gather(const Params& p, int row_bytes, int32_t* phys_out, void* rows_out, hipStream_t s) {
  dim3 grid((p.topk + 3) / 4, p.n_tokens), block(256);
  hipLaunchKernelGGL(gather_kernel, grid, block, 0, s, p, row_bytes, phys_out, static_cast<uint8_t*>(rows_out));
  return hip_status(hipGetLastError());
}

// ---------------------------------------------------------------------------------------
// merge of split partials: one workgroup of 128 lanes per (token, head); 4 dv columns per lane.
// (PART16: the partial sums are bf16, packed at the start of the same area: the head-group kernel's)
template <bool PART16>
__global__ __launch_bounds__(128) void merge_kernel(const float* __restrict__ part_out,
                                                    const float* __restrict__ part_lse,
                                                    uint16_t* __restrict__ out, float* __restrict__ lse,
                                                    int n_heads, int n_splits) {
  const int h = blockIdx.x % n_heads, t = blockIdx.x / n_heads;
  float m = -INFINITY;
  for (int i = 0; i < n_splits; ++i)
    m = fmaxf(m, part_lse[((size_t)t * n_splits + i) * n_heads + h]);
  const float m_safe = m == -INFINITY ? 0.f : m;
  float tot = 0.f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int i = 0; i < n_splits; ++i) {
    const float w = expf(part_lse[((size_t)t * n_splits + i) * n_heads + h] - m_safe);
    if (w == 0.f) continue;    // also skips partials of empty splits (their out is 0, lse -inf)
    tot += w;
    float4 v;
    if constexpr (PART16) {
      const uint2 b = reinterpret_cast<const uint2*>(
          reinterpret_cast<const uint16_t*>(part_out) + (((size_t)t * n_splits + i) * n_heads + h) * kDv)[threadIdx.x];
      v = make_float4(__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xffff0000u), __uint_as_float(b.y << 16),
                      __uint_as_float(b.y & 0xffff0000u));
    } else {
      v = reinterpret_cast<const float4*>(part_out + (((size_t)t * n_splits + i) * n_heads + h) * kDv)[threadIdx.x];
    }
    acc.x += w * v.x; acc.y += w * v.y; acc.z += w * v.z; acc.w += w * v.w;
  }
  const float inv = tot > 0.f ? 1.f / tot : 0.f;
  ushort4 o;
  o.x = f32_to_bf16_bits(acc.x * inv); o.y = f32_to_bf16_bits(acc.y * inv);
  o.z = f32_to_bf16_bits(acc.z * inv); o.w = f32_to_bf16_bits(acc.w * inv);
  reinterpret_cast<ushort4*>(out + ((size_t)t * n_heads + h) * kDv)[threadIdx.x] = o;
  if (threadIdx.x == 0) lse[(size_t)t * n_heads + h] = tot > 0.f ? m_safe + logf(tot) : -INFINITY;
}

int launch_merge(const float* part_out, const float* part_lse, void* out, float* lse, int n_tokens,
                 int n_heads, int d_v, int n_splits, bool partials_bf16, hipStream_t s) {
  if (d_v != kDv) return SMLA_EINVAL_SHAPE;
  dim3 grid((unsigned)n_heads * (unsigned)n_tokens), block(128);
  if (partials_bf16)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(merge_kernel<true>), grid, block, 0, s, part_out, part_lse, static_cast<uint16_t*>(out), lse,
                       n_heads, n_splits);
  else
    hipLaunchKernelGGL(HIP_KERNEL_NAME(merge_kernel<false>), grid, block, 0, s, part_out, part_lse, static_cast<uint16_t*>(out), lse,
                       n_heads, n_splits);
  return hip_status(hipGetLastError());
}

// ---------------------------------------------------------------------------------------
// KV-cache writers: one wavefront per latent row, addressed through the slot mapping
// (slot = page * page_size + offset, negative or past the pool = skip).
// fp8 records: lane owns 8 consecutive NoPE values; 16 lanes = one 128-column block.  The
// quotients x / scale are converted by v_cvt_pk_fp8_f32 (round to nearest even; |x / scale| never
// exceeds 448 by more than a rounding, so nothing saturates); a row that holds a NaN anywhere
// takes the bit-level routine instead, which pins NaN to the code 0x7f.
//
// The kernel is bound by instructions, and eight IEEE divisions a lane were most of them.  The
// code of a quotient only changes where the quotient crosses the midpoint of two fp8 values, so
// x * (1 / scale) gives the same code as the correctly rounded x / scale unless it lies next to
// such a midpoint: with 1 / scale good to one unit in the last place the product is within 3.5
// units of the quotient, and a normal-range midpoint is the bit pattern 0x80000 in the low 20
// bits of the fp32 mantissa (three mantissa bits kept, the fourth set, nothing below).  Lanes
// with a product within 5 units of that pattern, or with a value small enough for an fp8
// subnormal (other midpoints), divide.
// a 64-bit value that every lane of the wavefront holds alike, moved to scalar registers
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

constexpr int kRowsPerWave = 4;                    // rows a wavefront has in flight: one row a wavefront leaves the
                                                   // memory pipe half empty (36 KB of loads per CU against ~64 KB of latency x bandwidth)

// x / 448 correctly rounded, for x >= 2^-126 * 448 and finite, in three operations instead of the
// dozen of an IEEE division: q0 = x * RN(1/448) is within a unit of the quotient, the residual
// x - 448 q0 is exact in one fused operation, and q0 + residual * RN(1/448) rounds to the nearest
// float of the true quotient (448 = 1.75 * 2^8: its reciprocal's rounding error is far from the
// half-unit cases where this correction can fail).  Infinity and NaN come out as NaN, as the
// quotients of such a block do anyway.
__device__ __forceinline__ float div_by_448(float x) {
  constexpr float r = 1.0f / 448.0f;
  const float q0 = x * r;
  return __builtin_fmaf(__builtin_fmaf(-q0, 448.0f, x), r, q0);
}

// quantises one latent row held as (raw = this lane's 8 NoPE values, rope = lanes 0..7: the RoPE tail) into rec
__device__ __forceinline__ void quantize_row(const uint4 raw, const uint4 rope, uint8_t* rec, int lane) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  float v[8];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    amax = fmaxf(amax, fmaxf(fabsf(v[2 * i]), fabsf(v[2 * i + 1])));
  }
  // 16 lanes = one 128-block = one row of the data-parallel-primitive moves: rotate by 1, 2, 4, 8
  amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0x121, 0xf, 0xf, false)));
  amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0x122, 0xf, 0xf, false)));
  amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0x124, 0xf, 0xf, false)));
  amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0x128, 0xf, 0xf, false)));
  const float scale = div_by_448(fmaxf(amax, 0x1p-126f * 448.0f));
  const float r0 = __builtin_amdgcn_rcpf(scale);
  const float inv = __builtin_fmaf(r0, __builtin_fmaf(-scale, r0, 1.0f), r0);    // one Newton step: 1 / scale to one unit
  const float small = scale * 0x1.02p-6f;            // below this a quotient may be an fp8 subnormal
  float qv[8];
  uint32_t nearest = 0xffffffffu;                    // smallest distance code of the eight: one compare for all
  float least = INFINITY;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    qv[i] = v[i] * inv;
    nearest = min(nearest, (__float_as_uint(qv[i]) - (0x80000u - 5u)) & 0xfffffu);
    least = fminf(least, fabsf(v[i]));
  }
  if (nearest <= 10u || least < small) {
#pragma unroll
    for (int i = 0; i < 8; ++i) qv[i] = __fdiv_rn(v[i], scale);
  }
  bool odd = false;                                  // a NaN quotient (NaN or infinite input)
#pragma unroll
  for (int i = 0; i < 8; ++i) odd |= qv[i] != qv[i];
  uint32_t lo = 0, hi = 0;
  if (!__any(odd)) {
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(qv[0], qv[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(qv[2], qv[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(qv[4], qv[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(qv[6], qv[7], hi, true);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo |= f32_to_e4m3(qv[i]) << (8 * i);
      hi |= f32_to_e4m3(qv[4 + i]) << (8 * i);
    }
  }
  reinterpret_cast<uint2*>(rec)[lane] = make_uint2(lo, hi);
  if ((lane & 15) == 0) reinterpret_cast<float*>(rec + kFp8ScaleOff)[lane >> 4] = scale;
  if (lane < 8) reinterpret_cast<uint4*>(rec + kFp8RopeOff)[lane] = rope;
}

__global__ __launch_bounds__(256) void quantize_kernel(const uint16_t* __restrict__ src,
                                                       const int64_t* __restrict__ slot,
                                                       uint8_t* __restrict__ records, int64_t n_rows,
                                                       int64_t record_rows) {
  const int lane = threadIdx.x & 63;
  const int64_t first = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * kRowsPerWave;
  uint4 raw[kRowsPerWave], rope[kRowsPerWave];
  int64_t dst[kRowsPerWave];
#pragma unroll
  for (int j = 0; j < kRowsPerWave; ++j) {          // every row's loads are issued before the first is used
    const int64_t r = min(first + j, n_rows - 1);
    const uint16_t* row = src + r * kDqk;
    raw[j] = reinterpret_cast<const uint4*>(row)[lane];
    rope[j] = reinterpret_cast<const uint4*>(row + kDv)[lane & 7];
    dst[j] = first + j < n_rows ? (slot ? slot[r] : r) : -1;
  }
#pragma unroll
  for (int j = 0; j < kRowsPerWave; ++j) {
    const int64_t d = wave_uniform(dst[j]);                      // the same in every lane: the record's address is scalar work
    if (d < 0 || d >= record_rows) continue;
    quantize_row(raw[j], rope[j], records + d * kRowBytesFp8, lane);
  }
}

int launch_quantize(const void* src, const int64_t* slot, void* records, int64_t n_rows,
                    int64_t record_rows, hipStream_t s) {
  if (n_rows == 0) return SMLA_OK;
  dim3 grid((unsigned)((n_rows + 4 * kRowsPerWave - 1) / (4 * kRowsPerWave))), block(256);
  hipLaunchKernelGGL(quantize_kernel, grid, block, 0, s, static_cast<const uint16_t*>(src), slot,
                                         static_cast<uint8_t*>(records), n_rows, record_rows);
  return hip_status(hipGetLastError());
}

// bf16 rows: a 1152-byte copy per row (72 lanes' worth of 16 bytes: the first 8 lanes take a second chunk)
__global__ __launch_bounds__(256) void kv_copy_kernel(const uint4* __restrict__ src, const int64_t* __restrict__ slot,
                                                      uint4* __restrict__ pool, int64_t n_rows, int64_t pool_rows) {
  const int lane = threadIdx.x & 63;
  const int64_t first = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * kRowsPerWave;
  constexpr int kChunks = kRowBytesBf16 / 16;        // 72
  uint4 a[kRowsPerWave], b[kRowsPerWave];
  int64_t dst[kRowsPerWave];
#pragma unroll
  for (int j = 0; j < kRowsPerWave; ++j) {          // every row's loads are issued before the first store
    const int64_t r = min(first + j, n_rows - 1);
    const uint4* in = src + r * kChunks;
    a[j] = in[lane];
    b[j] = in[64 + (lane & 7)];
    dst[j] = first + j < n_rows ? (slot ? slot[r] : r) : -1;
  }
#pragma unroll
  for (int j = 0; j < kRowsPerWave; ++j) {
    if (dst[j] < 0 || dst[j] >= pool_rows) continue;              // (wave-uniform)
    uint4* out = pool + dst[j] * kChunks;
    out[lane] = a[j];
    if (lane < kChunks - 64) out[64 + lane] = b[j];
  }
}

int launch_kv_copy(const void* src, const int64_t* slot, void* pool, int64_t n_rows, int64_t pool_rows, hipStream_t s) {
  if (n_rows == 0) return SMLA_OK;
  dim3 grid((unsigned)((n_rows + 4 * kRowsPerWave - 1) / (4 * kRowsPerWave))), block(256);
  hipLaunchKernelGGL(kv_copy_kernel, grid, block, 0, s, static_cast<const uint4*>(src), slot, static_cast<uint4*>(pool), n_rows, pool_rows);
  return hip_status(hipGetLastError());
}

// ---------------------------------------------------------------------------------------
// plain fill kernel (used instead of a memset node so callers may capture it in a graph)
__global__ __launch_bounds__(256) void zero_kernel(uint4* __restrict__ p, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256)
    p[i] = make_uint4(0, 0, 0, 0);
}

int launch_zero(void* ptr, size_t bytes, hipStream_t s) {
  const size_t n16 = bytes / 16;
  if (n16 == 0) return SMLA_OK;
  const unsigned blocks = (unsigned)((n16 + 255) / 256 > 1024 ? 1024 : (n16 + 255) / 256);
  hipLaunchKernelGGL(zero_kernel, dim3(blocks), dim3(256), 0, s, static_cast<uint4*>(ptr), n16);
  return hip_status(hipGetLastError());
}

// zeroes the arrival words of a workspace and writes its header (same reason for a kernel)
__global__ __launch_bounds__(256) void workspace_init_kernel(uint4* __restrict__ p) {
  constexpr size_t kWords16 = SMLA_WS_COUNTER_BYTES / 16, kHeader16 = SMLA_WS_HEADER_OFFSET / 16;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < kWords16; i += (size_t)gridDim.x * 256)
    p[i] = i == kHeader16 ? make_uint4(SMLA_WS_MAGIC, 0u, SMLA_WS_SPIN_LIMIT_DEFAULT, 0u) : make_uint4(0, 0, 0, 0);
}

int launch_workspace_init(void* workspace, hipStream_t s) {
  hipLaunchKernelGGL(workspace_init_kernel, dim3(64), dim3(256), 0, s, static_cast<uint4*>(workspace));
  return hip_status(hipGetLastError());
}

}  // namespace smla
