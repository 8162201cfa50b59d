"""ctypes binding of libflagtree_smla.so (the C ABI declared in include/flagtree_smla.h)."""
import ctypes
import os

from .build import LIB_PATH

_c = ctypes
_i32, _i64, _f32, _vp, _sz = _c.c_int32, _c.c_int64, _c.c_float, _c.c_void_p, _c.c_size_t

SMLA_KV_BF16, SMLA_KV_FP8_B128, SMLA_KV_F32 = 0, 1, 2
SMLA_MAX_SPLITS = 32
SMLA_WS_COUNTER_BYTES = 262144
SMLA_WS_HEADER_OFFSET = SMLA_WS_COUNTER_BYTES - 64
SMLA_WS_MAGIC = 0x414C4D53
SMLA_EWORKSPACE_STATE = -8
WS_STATUS_BITS = {1: "never initialised", 2: "arrival word in an illegal state", 4: "split merge timed out"}
FP8_RECORD_BYTES = 656

# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "smla_strerror": (_c.c_char_p, [_c.c_int]),
    "smla_abi_version": (_c.c_int, []),
    "smla_fwd": (_c.c_int, [_c.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32,
                            _i32, _i32, _i64, _i64, _f32, _i32, _vp, _sz, _vp]),
    "smla_decode_dense": (_c.c_int, [_c.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32,
                                     _i32, _i32, _i64, _i64, _f32, _f32, _i32, _vp, _sz, _vp]),
    "smla_fwd_scalar": (_c.c_int, [_c.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                   _i32, _i32, _i32, _i64, _i64, _f32, _vp]),
    "smla_plan_splits": (_c.c_int, [_c.c_int, _i32, _i32, _i32]),
    "smla_merge_in_launch": (_c.c_int, []),
    "smla_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32]),
    "smla_workspace_init": (_c.c_int, [_vp, _sz, _vp]),
    "smla_workspace_status": (_c.c_int, [_vp, _sz, _vp, _c.POINTER(_c.c_uint32)]),
    "smla_gather_rows": (_c.c_int, [_vp, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i64,
                                    _i64, _vp]),
    "smla_merge_splits": (_c.c_int, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp]),
    "smla_kv_quantize_fp8": (_c.c_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "smla_kv_write": (_c.c_int, [_c.c_int, _vp, _vp, _vp, _i64, _i64, _vp]),
    "smla_topk_indices": (_c.c_int, [_vp, _vp, _vp, _c.c_int32, _c.c_int32, _i64, _c.c_int32, _vp, _sz, _vp]),
    "smla_topk_rows": (_c.c_int, [_vp, _vp, _vp, _vp, _i32, _i32, _i64, _i32, _i32, _i32, _i32, _i64, _vp, _sz, _vp]),
    "smla_topk_workspace_bytes": (_sz, [_i32, _i32, _i32]),
    "smla_gemm_rs_local": (_c.c_int, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i64, _vp]),
}

_lib = None


def load():
    """Load the in-tree library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    path = LIB_PATH
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: build it with `python -m flagtree_amd.build` "
            "(flagtree_amd has no non-HIP fallback)")
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def strerror(rc):
    return load().smla_strerror(rc).decode()


def check(rc, what):
    if rc == 0:
        return
    msg = f"{what}: {strerror(rc)} (status {rc})"
    if -10 < rc < 0:
        raise ValueError(msg)
    raise RuntimeError(msg)


def on_device(t):
    """True for a tensor in GPU memory.  The one place the wrappers ask (there is no CPU path)."""
    return t.is_cuda


def stream_handle(device):
    """The caller's current stream on `device` as the hipStream_t the C ABI takes."""
    import torch
    return torch.cuda.current_stream(device).cuda_stream

