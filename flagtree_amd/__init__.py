"""flagtree_amd: MI355X-native sparse MLA forward (hand-written HIP behind a C ABI).

Public surface mirrors the operator FlagTree ships as a Triton/TLE kernel:
``sparse_mla_fwd(q, kv_cache, indices, sm_scale, d_v) -> (out, lse)``.
"""
from .sparse_mla import (sparse_mla_fwd, sparse_mla_fwd_scalar, gather_rows, merge_splits, plan_splits, quantize_kv_fp8,
                         make_workspace, workspace_status, reshape_and_cache, topk_indices, topk_workspace_bytes,
                         decode_attention_fwd)
from .gemm_rs import gemm_rs_local

__all__ = ["sparse_mla_fwd", "sparse_mla_fwd_scalar", "gather_rows", "merge_splits", "plan_splits",
           "quantize_kv_fp8", "reshape_and_cache", "topk_indices", "topk_workspace_bytes", "decode_attention_fwd", "make_workspace", "workspace_status",
           "gemm_rs_local"]
