/* Probe numbers and buffer geometry of the hardware-model probes (primitives.hip); the Python
 * side reads this file for the same numbers. */
#pragma once

#define HWM_LANES 64
#define HWM_RECORD_BYTES 256 /* per lane, in `in` and in `out` */

enum {
  HWM_MFMA_16X16X32_BF16 = 0,      /* in: A 16 B, B 16 B, C 16 B at 0/16/32;  out: D 16 B */
  HWM_MFMA_32X32X16_BF16 = 1,      /* in: A, B at 0/16, C 64 B at 64;  out: D 64 B */
  HWM_MFMA_16X16X16_BF16 = 2,      /* in: A 8 B, B 8 B, C 16 B at 0/8/16;  out: D 16 B */
  HWM_LDS_READ_TR16_B64 = 3,       /* in: 64 B of LDS contents, u32 LDS offset at 64;  out: 8 B */
  HWM_DMA_B128 = 4,                /* in: u32 byte offset into `in` of the 16 B this lane moves;  out: LDS bytes 32 l .. 32 l + 31 */
  HWM_DMA_B128_FIRST_8_LANES = 5,  /* the same, lanes 0 .. 7 only */
  HWM_DMA_B128_BASE_PLUS_OFFSET = 6,
  HWM_DMA_B32 = 7,                 /* 4 B a lane */
  HWM_DPP_MOVES = 8,               /* in: i32;  out: 17 i32 (DPP controls the kernels use, readlane, ballot, shuffles) */
  HWM_FP8_CONVERSIONS = 9,         /* in: 4 e4m3 codes at 0, two floats at 16;  out: 32 B */
  HWM_COMPARE_AND_SHIFT_IN = 10,   /* in: x, y, mask (u32);  out: mask after shift_in_gt, after shift_in_eq */
  HWM_AGENT_SCOPE_ACCESSES = 11,   /* in: 16 B at 0 (stored), 16 B at 16 (loaded);  out: both */
  HWM_APPROXIMATE_FUNCTIONS = 12,  /* in: 4 floats;  out: exp2, log2(|x| + 1e-3), 1 / (|x| + 1e-3) of each */
  HWM_MFMA_16X16X32_FP8 = 13,      /* in: A 8 B, B 8 B, C 16 B at 0/8/16 (e4m3 codes);  out: D 16 B */
  HWM_MFMA_SCALE_16X16X128_FP8 = 14, /* in: A 32 B, B 32 B, C 16 B at 0/32/64; scale bytes 127 (A) and 123 (B) in every lane;  out: D 16 B */
  HWM_BYTE_PERMUTE = 15,           /* in: a, b (u32);  out: v_perm_b32 with the two selectors the fp8 V operand is put together with */
  HWM_COUNT = 16
};

#ifdef __cplusplus
extern "C" {
#endif
/* Runs probe `which` on one wavefront.  `in` and `out`: HWM_LANES * HWM_RECORD_BYTES bytes each,
 * 256-byte aligned, on the device.  0 on success. */
int hwm_run(int which, const void* in, void* out, void* stream);
int hwm_count(void);
#ifdef __cplusplus
}
#endif
