"""Inputs for the hardware-model probes (tests/hw_model/primitives.hip) and statements of what each
instruction is documented to do, in numpy, written from the instruction descriptions and not from
the emulator's code.  Test infrastructure."""
import ctypes
import os
import re

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LANES, RECORD = 64, 256
GPU_LIB_PATH = os.path.join(HERE, "libhw_model.so")


def _probe_numbers():
    text = open(os.path.join(HERE, "primitives.h")).read()
    return {m.group(1): int(m.group(2)) for m in re.finditer(r"HWM_([A-Z0-9_]+) = (\d+)", text)}


PROBES = _probe_numbers()
PROBE_NAMES = [n for n in PROBES if n != "COUNT"]


def bind(lib):
    lib.hwm_run.restype = ctypes.c_int
    lib.hwm_run.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.hwm_count.restype = ctypes.c_int
    return lib


def gpu_lib():
    """The gfx950 build; built on the CPU beforehand (build_hw_model.py), never inside a GPU run."""
    if not os.path.exists(GPU_LIB_PATH):
        raise RuntimeError(f"{GPU_LIB_PATH} is missing: run python tests/hw_model/build_hw_model.py")
    return bind(ctypes.CDLL(GPU_LIB_PATH))


def bf16_bits(x):
    """float32 array of values that bf16 holds exactly -> their 16-bit patterns."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    assert not (u & 0xFFFF).any(), "not exactly representable in bf16"
    return (u >> 16).astype(np.uint16)


def bf16_value(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def make_input(name, seed):
    """64 records of 256 bytes (uint8 array [64, 256]) for probe `name`."""
    g = np.random.default_rng(1000 * PROBES[name] + seed)
    rec = g.integers(0, 256, size=(LANES, RECORD), dtype=np.uint8)
    u32 = rec.view(np.uint32)
    f32 = rec.view(np.float32)
    u16 = rec.view(np.uint16)
    if name in ("MFMA_16X16X32_FP8", "MFMA_SCALE_16X16X128_FP8"):
        # e4m3 codes of small integers: every product and partial sum is exact in fp32, whatever the order
        import oracle
        n_ab = 16 if name == "MFMA_16X16X32_FP8" else 64
        rec[:, :n_ab] = oracle.e4m3_encode(g.integers(-4, 5, size=(LANES, n_ab)).astype(np.float32))
        c0 = n_ab // 4
        f32[:, c0:c0 + 4] = g.integers(-8, 9, size=(LANES, 4)).astype(np.float32)
    elif name.startswith("MFMA"):
        # small integers: every product and every partial sum is exact in fp32, whatever the order
        n_ab = 8 if name == "MFMA_16X16X16_BF16" else 16
        u16[:, :n_ab] = bf16_bits(g.integers(-4, 5, size=(LANES, n_ab)).astype(np.float32))
        c0, nc = {"MFMA_16X16X32_BF16": (8, 4), "MFMA_32X32X16_BF16": (16, 16), "MFMA_16X16X16_BF16": (4, 4)}[name]
        f32[:, c0:c0 + nc] = g.integers(-8, 9, size=(LANES, nc)).astype(np.float32)
    elif name == "LDS_READ_TR16_B64":
        u32[:, 16] = g.integers(0, 4096 // 8, size=LANES).astype(np.uint32) * 8
    elif name.startswith("DMA"):
        u32[:, 0] = g.integers(0, LANES * RECORD // 16, size=LANES).astype(np.uint32) * 16
    elif name == "FP8_CONVERSIONS":
        rec[:, :4] = (4 * np.arange(LANES)[:, None] + np.arange(4)[None, :]).astype(np.uint8)      # all 256 codes
        edge = np.array([0.0, -0.0, 448.0, -448.0, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9, 2.5 * 2.0 ** -9, 0.9 * 2.0 ** -10,
                         17.0, 18.0, 19.0, 20.0, 21.0, 22.0, 23.0, 0.0146484375, 1e-10, -1e-10, 447.9, 431.9, 432.0, 432.1],
                        dtype=np.float32)
        vals = (g.standard_normal((LANES, 2)) * np.array([1.0, 150.0])[g.integers(0, 2, size=(LANES, 1))]).astype(np.float32)
        vals = np.clip(vals, -448.0, 448.0)            # the quantiser never hands the instruction more
        k = min(len(edge), LANES) if seed == 0 else 0
        vals[:k, 0] = edge[:k]
        vals[:k, 1] = -edge[:k][::-1]
        f32[:, 4:6] = vals
    elif name == "COMPARE_AND_SHIFT_IN":
        same = g.random(LANES) < 0.3
        u32[same, 1] = u32[same, 0]
    elif name == "APPROXIMATE_FUNCTIONS":
        f32[:, :4] = (g.random((LANES, 4)) * 40.0 - 20.0).astype(np.float32)
    return rec


# ---- what the instructions are documented to do ------------------------------------------------

def _mfma_operands(rec, m, k, kpl):
    """Fragments -> matrices.  A[i][kk] sits in lane i + m * (kk // kpl), element kk % kpl; B[kk][j]
    in lane j + m * (kk // kpl), element kk % kpl."""
    a = np.zeros((m, k), np.float32)
    b = np.zeros((k, m), np.float32)
    u16 = rec.view(np.uint16)
    for lane in range(LANES):
        i, blk = lane % m, lane // m
        a[i, kpl * blk:kpl * (blk + 1)] = bf16_value(u16[lane, :kpl])
        b[kpl * blk:kpl * (blk + 1), i] = bf16_value(u16[lane, kpl:2 * kpl])
    return a, b


def expect(name, rec):
    """Expected [64, 256] output bytes (0xCD where a probe writes nothing), or for the approximate
    functions the float32 values to be matched within a tolerance."""
    out = np.full((LANES, RECORD), 0xCD, dtype=np.uint8)
    o32, of32 = out.view(np.uint32), out.view(np.float32)
    u32, f32 = rec.view(np.uint32), rec.view(np.float32)
    if name in ("MFMA_16X16X32_BF16", "MFMA_16X16X16_BF16"):
        k, kpl, c0 = (32, 8, 8) if name == "MFMA_16X16X32_BF16" else (16, 4, 4)
        a, b = _mfma_operands(rec, 16, k, kpl)
        d = a @ b
        for lane in range(LANES):                     # C/D: lane holds column lane % 16, rows 4 * (lane // 16) + 0..3
            for r in range(4):
                of32[lane, r] = d[4 * (lane // 16) + r, lane % 16] + f32[lane, c0 + r]
    elif name in ("MFMA_16X16X32_FP8", "MFMA_SCALE_16X16X128_FP8"):
        # Lane m + 16 g holds `nb` values of row m of A and, behind them, of column m of B.  A (g, byte)
        # pair stands for the same k in both operands, so the sum over all pairs is the product
        # whatever that k is.  The scaled form multiplies by 2^(127 - 127) * 2^(123 - 127).
        import oracle
        nb = 8 if name == "MFMA_16X16X32_FP8" else 32
        a = oracle.e4m3_decode(rec[:, :nb]).astype(np.float64).reshape(4, 16, nb)          # [g, m, byte]
        b = oracle.e4m3_decode(rec[:, nb:2 * nb]).astype(np.float64).reshape(4, 16, nb)     # [g, n, byte]
        d = np.einsum("gmj,gnj->mn", a, b) * (1.0 if name == "MFMA_16X16X32_FP8" else 2.0 ** -4)
        c0 = nb // 2
        for lane in range(LANES):
            for r in range(4):
                of32[lane, r] = d[4 * (lane // 16) + r, lane % 16] + f32[lane, c0 + r]
    elif name == "BYTE_PERMUTE":
        both = rec[:, [4, 5, 6, 7, 0, 1, 2, 3]]           # bytes 0..3 = b (the second operand), 4..7 = a
        out[:, 0:4] = both[:, [0, 2, 4, 6]]
        out[:, 4:8] = both[:, [1, 3, 5, 7]]
    elif name == "MFMA_32X32X16_BF16":
        a, b = _mfma_operands(rec, 32, 16, 8)
        d = a @ b
        for lane in range(LANES):                     # column lane % 32, rows 8 * (r // 4) + 4 * (lane // 32) + r % 4
            for r in range(16):
                of32[lane, r] = d[8 * (r // 4) + 4 * (lane // 32) + r % 4, lane % 32] + f32[lane, 16 + r]
    elif name == "LDS_READ_TR16_B64":
        lds = rec[:, :64].reshape(-1)
        addr = u32[:, 16] & (4096 - 8)
        o16 = out.view(np.uint16)
        for lane in range(LANES):
            grp, i = lane - lane % 16, lane % 16
            for e in range(4):                        # element i % 4 of the rows of lanes i // 4 + 4 e of the group
                src = int(addr[grp + i // 4 + 4 * e]) + 2 * (i % 4)
                o16[lane, e] = lds[src:src + 2].view(np.uint16)[0]
    elif name.startswith("DMA"):
        flat = rec.reshape(-1)
        lds = np.full(4096, 0xEE, dtype=np.uint8)
        width = 4 if name == "DMA_B32" else 16
        lanes = 8 if name == "DMA_B128_FIRST_8_LANES" else LANES
        for lane in range(lanes):                     # lane's piece lands at base + width * lane
            off = int(u32[lane, 0]) & (LANES * RECORD - 16)
            lds[256 + width * lane:256 + width * (lane + 1)] = flat[off:off + width]
        out[:, :32] = lds[:2048].reshape(LANES, 32)
    elif name == "DPP_MOVES":
        v = rec.view(np.int32)[:, 0]
        d = np.zeros((LANES, 17), np.int32)
        for lane in range(LANES):
            row, i = lane // 16, lane % 16
            for j, s in enumerate((1, 2, 4, 8)):
                d[lane, j] = v[16 * row + i - s] if i >= s else 0           # row_shr: lanes without a source keep `old` (0)
                d[lane, 4 + j] = v[16 * row + (i - s) % 16]                 # row_ror
            d[lane, 8] = v[16 * row - 1] if row in (1, 3) else 0            # row_bcast 15, rows 1 and 3 enabled
            d[lane, 9] = v[31] if row in (2, 3) else 0                      # row_bcast 31, rows 2 and 3 enabled
            d[lane, 10], d[lane, 11], d[lane, 12] = v[37], v[0], lane
            d[lane, 15] = v[lane - 1] if lane >= 1 else v[lane]
            d[lane, 16] = v[lane ^ 21]
        ballot = sum((int(v[l]) & 1) << l for l in range(LANES))
        d[:, 13] = np.uint32(ballot & 0xFFFFFFFF).view(np.int32)
        d[:, 14] = np.uint32(ballot >> 32).view(np.int32)
        out.view(np.int32)[:, :17] = d
    elif name == "FP8_CONVERSIONS":
        import oracle
        codes = rec[:, :4]
        val = oracle.e4m3_decode(codes)               # [64, 4] float32 (NaN for 0x7f / 0xff)
        of32[:, 0:4] = val
        out.view(np.uint16)[:, 8:12] = (val.view(np.uint32) >> 16).astype(np.uint16)     # every e4m3 value is exact in bf16
        q = oracle.e4m3_encode(f32[:, 4:6])           # [64, 2] uint8
        pair = q[:, 0].astype(np.uint32) | (q[:, 1].astype(np.uint32) << 8)
        o32[:, 6] = (0xA5A50000 | pair)
        o32[:, 7] = (0x0000A5A5 | (pair << 16))
    elif name == "COMPARE_AND_SHIFT_IN":
        x, y, m = u32[:, 0], u32[:, 1], u32[:, 2]
        o32[:, 0] = (m << np.uint32(1)) + (x > y)
        o32[:, 1] = (m << np.uint32(1)) + (x == y)
    elif name == "AGENT_SCOPE_ACCESSES":
        out[:, :32] = rec[:, :32]
    elif name == "APPROXIMATE_FUNCTIONS":
        x = f32[:, :4]
        arg = (np.abs(x) + np.float32(1e-3)).astype(np.float64)          # the probe forms the argument in fp32
        return np.concatenate([np.exp2(x.astype(np.float64)), np.log2(arg), 1.0 / arg], axis=1).astype(np.float32)
    return out


def differences(name, got, want):
    """Compares a probe's output [64, 256] uint8 with another run's, or with expect()'s answer.
    Bit for bit, except: NaN compares equal to NaN whatever its payload (fp8 conversions of the two
    NaN codes), and the approximate functions are matched to 2e-6 relative + 2e-7 absolute (1 ulp
    instructions against libm).  Returns a list of messages, empty when they agree."""
    got = np.asarray(got, dtype=np.uint8).reshape(LANES, RECORD)
    if name == "APPROXIMATE_FUNCTIONS":
        g = got.view(np.float32)[:, :12]
        w = want if want.dtype == np.float32 and want.shape == (LANES, 12) else np.asarray(want, np.uint8).reshape(LANES, RECORD).view(np.float32)[:, :12]
        bad = ~(np.abs(g.astype(np.float64) - w) <= 2e-6 * np.abs(w) + 2e-7)       # (absolute part: log2 near 1)
        untouched = (got[:, 48:] == 0xCD).all()
        return [f"lane {l} value {c}: {g[l, c]!r} against {w[l, c]!r}" for l, c in zip(*np.nonzero(bad))][:8] + ([] if untouched else ["bytes past the results were written"])
    want = np.asarray(want, dtype=np.uint8).reshape(LANES, RECORD)
    g, w = got.copy(), want.copy()
    if name == "FP8_CONVERSIONS":
        gf, wf = g.view(np.float32)[:, :4], w.view(np.float32)[:, :4]
        both = np.isnan(gf) & np.isnan(wf)
        gf[both] = 0.0
        wf[both] = 0.0
        gb, wb = g.view(np.uint16)[:, 8:12], w.view(np.uint16)[:, 8:12]
        both = np.isnan(bf16_value(gb)) & np.isnan(bf16_value(wb))
        gb[both] = 0
        wb[both] = 0
    bad = np.nonzero(g != w)
    return [f"lane {l} byte {b}: {got[l, b]:#04x} against {want[l, b]:#04x}" for l, b in zip(*bad)][:8]
