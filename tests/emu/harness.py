"""Calls into the emulator build of the kernel sources (tests only).

The emulated library exports the same C ABI as the product library; here it is given CPU tensors,
whose memory the emulated kernels read and write directly."""
import ctypes
import importlib.util
import math
import os

import torch

from flagtree_amd import _lib as product_lib

HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None
_keep_alive = []
# compute units the stand-in device reports: small, so that small shapes reach the planning corner
# cases (FLAGTREE_EMU_CUS=256 makes the planners choose what they choose on the real device)
EMU_CUS = int(os.environ.get("FLAGTREE_EMU_CUS", "16"))


def lib():
    global _lib
    if _lib is None:
        spec = importlib.util.spec_from_file_location("build_emu", os.path.join(HERE, "build_emu.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        path = mod.build()
        l = ctypes.CDLL(path)
        for name, (res, args) in product_lib.SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        l.emu_set_dma_mode.argtypes = [ctypes.c_int]
        l.emu_set_block_order.argtypes = [ctypes.c_uint]
        l.emu_set_wave_skew.argtypes = [ctypes.c_uint]
        l.emu_set_concurrent_blocks.argtypes = [ctypes.c_uint, ctypes.c_uint]
        l.emu_launch_count.restype = ctypes.c_ulonglong
        l.emu_block_count.restype = ctypes.c_ulonglong
        l.emu_poll_count.restype = ctypes.c_ulonglong
        l.emu_set_cu_count.argtypes = [ctypes.c_int]
        l.emu_set_lds_profile.argtypes = [ctypes.c_int]
        l.emu_lds_profile.argtypes = [ctypes.POINTER(ctypes.c_ulonglong)]
        l.emu_work_counts.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.c_int]
        l.emu_set_cu_count(EMU_CUS)                      # before the library's first (cached) query
        l.emu_set_wave_skew(DEFAULT_WAVE_SKEW)
        _lib = l
    return _lib


DEFAULT_WAVE_SKEW = int(os.environ.get("FLAGTREE_EMU_WAVE_SKEW", "0"))   # schedule of runs that do not choose one (a rehearsal)


def configure(dma_eager=False, block_order_seed=0, wave_skew_seed=None, concurrent_blocks=0, concurrent_seed=0):
    l = lib()
    l.emu_set_concurrent_blocks(concurrent_blocks, concurrent_seed)
    l.emu_set_dma_mode(1 if dma_eager else 0)
    l.emu_set_block_order(block_order_seed)
    l.emu_set_wave_skew(DEFAULT_WAVE_SKEW if wave_skew_seed is None else wave_skew_seed)


def lds_profile_start():
    """Count bank passes of the kernels' addressed LDS accesses from now on (slower)."""
    lib().emu_set_lds_profile(1)


def lds_profile_stop():
    """{'read' | 'read_tr' | 'write': (wavefront instructions, passes taken, passes without conflicts)}"""
    out = (ctypes.c_ulonglong * 9)()
    lib().emu_lds_profile(out)
    lib().emu_set_lds_profile(0)
    return {k: tuple(int(out[3 * i + j]) for j in range(3)) for i, k in enumerate(("read", "read_tr", "write"))}


def work_counts(reset=True):
    """What the emulated kernels have done since the last reset: MFMA wavefront instructions and
    flops, LDS bytes read / written by address, bytes moved global -> LDS and the wavefront
    instructions that moved them, workgroup barriers (times wavefronts)."""
    out = (ctypes.c_double * 7)()
    lib().emu_work_counts(out, 1 if reset else 0)
    keys = ("mfma", "mfma_flops", "lds_read_bytes", "lds_write_bytes", "dma_bytes", "dma_instr", "barriers_x_waves")
    return dict(zip(keys, (float(v) for v in out)))


_FORMATS = {"bf16": 0, "fp8_e4m3_b128": 1, "f32": 2}


def make_workspace(n_bytes):
    ws = torch.empty(max(int(n_bytes), product_lib.SMLA_WS_COUNTER_BYTES), dtype=torch.uint8)
    ws.fill_(0xA5)
    rc = lib().smla_workspace_init(ws.data_ptr(), ws.numel(), None)
    assert rc == 0, rc
    return ws


def workspace_status(ws):
    status = ctypes.c_uint32(0)
    rc = lib().smla_workspace_status(ws.data_ptr(), ws.numel(), None, ctypes.byref(status))
    return rc, status.value


def forward(cfg, n_splits=1, workspace=None, dense_lens=None, scalar=False, logit_cap=0.0, guard_outputs=None):
    """cfg as flagtree_amd.workloads builds it, on the CPU.  Returns (out [T, H, 512], lse [T, H], rc)."""
    l = lib()
    q = cfg["q"]
    H, D = q.shape[-2], q.shape[-1]
    q3 = q.reshape(-1, H, D).contiguous()
    T = q3.shape[0]
    bt = cfg.get("block_table")
    B = q.shape[0] if q.dim() == 4 else (bt.shape[0] if bt is not None else 1)
    S = T // B
    kvc = cfg["kv_cache"]
    kv2 = kvc.reshape(-1, kvc.shape[-1]).contiguous()
    stride = 0
    if bt is None and kvc.dim() >= 3 and kvc.shape[0] == B and B > 1:
        stride = kvc[0].numel() // kvc.shape[-1]
    fmt = _FORMATS[cfg["kv_format"]]
    out = torch.full((T, H, 512), float("nan"), dtype=q.dtype)
    lse = torch.full((T, H), float("nan"), dtype=torch.float32)
    if guard_outputs is not None:                       # outputs between inaccessible pages (kept alive by the tensors' buffers)
        g_out, g_lse = Guarded(out, guard_outputs), Guarded(lse, guard_outputs)
        out, lse = g_out.tensor, g_lse.tensor
        _keep_alive.extend([g_out, g_lse])
    btc = bt.contiguous() if bt is not None else None
    bt_ptr = btc.data_ptr() if btc is not None else None
    bt_stride = btc.shape[1] if btc is not None else 0
    sm = float(cfg.get("sm_scale", 1.0 / math.sqrt(576)))
    if scalar:
        idx = cfg["indices"].reshape(T, -1).to(torch.int32).contiguous()
        rc = l.smla_fwd_scalar(fmt, q3.data_ptr(), kv2.data_ptr(), idx.data_ptr(), bt_ptr, out.data_ptr(), lse.data_ptr(),
                               T, S, H, idx.shape[1], 576, 512, cfg["page_size"], bt_stride, stride, kv2.shape[0], sm, None)
        return out, lse, rc
    ws_bytes = l.smla_workspace_bytes(T, H, 512, n_splits)
    if ws_bytes and workspace is None:
        workspace = make_workspace(ws_bytes)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_n = workspace.numel() if workspace is not None else 0
    if dense_lens is not None:
        lens = dense_lens.to(torch.int32).contiguous()
        rc = l.smla_decode_dense(fmt, q3.data_ptr(), kv2.data_ptr(), lens.data_ptr(), bt_ptr, out.data_ptr(), lse.data_ptr(),
                                 T, S, H, bt_stride * cfg["page_size"], 576, 512, cfg["page_size"], bt_stride, stride,
                                 kv2.shape[0], sm, float(logit_cap), n_splits, ws_ptr, ws_n, None)
    else:
        idx = cfg["indices"].reshape(T, -1).to(torch.int32).contiguous()
        rc = l.smla_fwd(fmt, q3.data_ptr(), kv2.data_ptr(), idx.data_ptr(), bt_ptr, out.data_ptr(), lse.data_ptr(),
                        T, S, H, idx.shape[1], 576, 512, cfg["page_size"], bt_stride, stride, kv2.shape[0], sm,
                        n_splits, ws_ptr, ws_n, None)
    return out, lse, rc


# ---- guarded buffers: memory the emulated kernels must not step outside of -------------------
import mmap as _mmap

_PAGE = _mmap.PAGESIZE
_libc = ctypes.CDLL(None, use_errno=True)
_libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]


class Guarded:
    """A copy of `tensor` whose last byte sits right before an inaccessible page (``end=True``) or
    whose first byte right after one: an emulated kernel that reads or writes past that edge of
    the buffer dies with SIGSEGV instead of silently touching a neighbour.  (A real GPU would take
    a memory access fault, or worse, not take one.)"""

    def __init__(self, tensor, end=True):
        t = tensor.contiguous()
        n = t.numel() * t.element_size()
        body = (n + _PAGE - 1) // _PAGE * _PAGE
        self._map = _mmap.mmap(-1, body + 2 * _PAGE)
        base = ctypes.addressof(ctypes.c_char.from_buffer(self._map))
        for off in (0, _PAGE + body):
            if _libc.mprotect(base + off, _PAGE, 0) != 0:
                raise OSError(ctypes.get_errno(), "mprotect")
        start = _PAGE + (body - n if end else 0)
        if end and (base + start) % 16:                   # keep the 16-byte alignment the C ABI asks for
            start -= (base + start) % 16
        self._buf = (ctypes.c_char * n).from_buffer(self._map, start)
        self.tensor = torch.frombuffer(self._buf, dtype=torch.uint8).view(t.dtype).view(t.shape)
        self.tensor.copy_(t)

    def close(self):
        """Drop this object's references; the mapping goes away with the last tensor that views it."""
        self.tensor = None
        self._buf = None
