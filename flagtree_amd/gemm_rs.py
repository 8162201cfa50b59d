"""Host side of the local GEMM of GEMM + reduce-scatter (single GPU, chunked-output epilogue).

Mirrors the calling style of the reference's matmul operator: a plain callable over tensors
that allocates and returns its output (/root/reference/python/triton/ops/matmul.py:162-228).
"""
import torch

from . import _lib


def gemm_rs_local(x, w, partial=None, n_chunks=8, out=None):
    """out[r] = bf16(X[r-th row chunk] @ W + partial[r-th row chunk]), r < n_chunks.

    x [M, K] bf16, w [K, N] bf16, partial [M, N] fp32 or None.  Returns a bf16 tensor
    [n_chunks, M // n_chunks, N]: chunk r is what rank r receives from the reduce-scatter.
    """
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ValueError("x and w must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[0]:
        raise ValueError("x must be [M, K] and w [K, N]")
    if not _lib.on_device(x):
        raise ValueError("gemm_rs_local needs device tensors (there is no CPU path)")
    M, K = x.shape
    N = w.shape[1]
    if M % n_chunks != 0:
        raise ValueError("M must be divisible by n_chunks")
    x, w = x.contiguous(), w.contiguous()
    if partial is not None:
        if partial.dtype != torch.float32 or tuple(partial.shape) != (M, N):
            raise ValueError("partial must be fp32 [M, N]")
        partial = partial.contiguous()
    if out is None:
        out = torch.empty((n_chunks, M // n_chunks, N), dtype=torch.bfloat16, device=x.device)
    elif out.dtype != torch.bfloat16 or tuple(out.shape) != (n_chunks, M // n_chunks, N) or not out.is_contiguous():
        raise ValueError("out must be a contiguous bf16 [n_chunks, M/n_chunks, N] tensor")
    lib = _lib.load()
    rc = lib.smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr() if partial is not None else None,
                                out.data_ptr(), M, N, K, n_chunks, (M // n_chunks) * N,
                                _lib.stream_handle(x.device))
    _lib.check(rc, "smla_gemm_rs_local")
    return out
