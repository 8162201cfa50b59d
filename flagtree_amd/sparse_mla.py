"""Host side of the sparse MLA forward operator.

Mirrors how the reference exposes an attention operator: a plain Python callable over
``torch.Tensor`` that validates shapes, allocates the outputs, and launches on the caller's
current stream (/root/reference/python/triton/ops/flash_attention.py:375-416; MLA decode
wrapper /root/reference/third_party/mthreads/python/test/wmma/test_accuracy_musa_vllm_mla.py:571-620).
The launch itself goes through the C ABI of ``libflagtree_smla.so``; there is no fallback
implementation: without the built library, or with CPU tensors, the call raises.
"""
import math

import torch

from . import _lib

D_QK = 576
D_V = 512
_FORMATS = {"bf16": _lib.SMLA_KV_BF16, "fp8_e4m3_b128": _lib.SMLA_KV_FP8_B128, "f32": _lib.SMLA_KV_F32}


def _stream(t):
    return _lib.stream_handle(t.device)


_I32_MAX = 2 ** 31 - 1


def _indices_i32(idx2):
    """int64 -> int32 without wrapping: anything past int32 is past every cache (at most 2^31 - 1
    rows), so it is clamped to a value the kernels mask; negatives stay negative."""
    if idx2.dtype == torch.int32:
        return idx2
    return idx2.clamp(min=-1, max=_I32_MAX).to(torch.int32)


def _normalise(q, kv_cache, indices, d_v, block_table, kv_format, per_sequence=None):
    """Shape / dtype validation shared by the MFMA and scalar entry points.
    Returns (q3, kv2, idx2, B, S, H, K, fmt, kv_seq_stride, block_table, out_shape, lse_shape).
    ``per_sequence`` (only without a block table): True = kv_cache[b] is sequence b's own rows and
    indices address them, False = one shared pool addressed by row number, None = per-sequence
    exactly when kv_cache has a leading dim equal to the batch and the batch is larger than 1."""
    if q.dim() == 4:
        B, S, H, D = q.shape
    elif q.dim() == 3:
        T, H, D = q.shape
        B, S = (block_table.shape[0], T // max(block_table.shape[0], 1)) if block_table is not None else (1, T)
        if B * S != T:
            raise ValueError("q [T, H, D]: T must be a multiple of the number of block-table rows")
    else:
        raise ValueError("q must be [B, S, H, 576] or [T, H, 576]")
    if D != D_QK or d_v != D_V:
        raise ValueError(f"only d_qk = {D_QK} (512 NoPE + 64 RoPE) and d_v = {D_V} are supported")
    T = B * S
    if kv_format is None:
        kv_format = {torch.bfloat16: "bf16", torch.uint8: "fp8_e4m3_b128", torch.float32: "f32"}.get(kv_cache.dtype)
    if kv_format not in _FORMATS:
        raise ValueError(f"kv_format must be one of {sorted(_FORMATS)}")
    fmt = _FORMATS[kv_format]
    want_kv = {"bf16": (torch.bfloat16, D_QK), "fp8_e4m3_b128": (torch.uint8, _lib.FP8_RECORD_BYTES),
               "f32": (torch.float32, D_QK)}[kv_format]
    if kv_cache.dtype != want_kv[0] or kv_cache.shape[-1] != want_kv[1]:
        raise ValueError(f"kv_cache for format {kv_format} must be {want_kv[0]} with last dim {want_kv[1]}")
    want_q = torch.float32 if kv_format == "f32" else torch.bfloat16
    if q.dtype != want_q:
        raise ValueError(f"q must be {want_q} for kv format {kv_format}")
    if indices.dim() == 4 and indices.shape[2] == 1:
        indices = indices[:, :, 0]
    if indices.dim() == 3:
        if tuple(indices.shape[:2]) != (B, S):
            raise ValueError("indices must be [B, S, topk]")
    elif indices.dim() == 2:
        if indices.shape[0] != T:
            raise ValueError("indices must be [T, topk]")
    else:
        raise ValueError("indices must be [B, S, topk], [B, S, 1, topk] or [T, topk]")
    K = indices.shape[-1]
    if indices.dtype not in (torch.int32, torch.int64):
        raise ValueError("indices must be int32 or int64")
    for name, t in (("q", q), ("kv_cache", kv_cache), ("indices", indices)):
        if not _lib.on_device(t):
            raise ValueError(f"{name} must be a device tensor (there is no CPU path)")
    idx2 = _indices_i32(indices.reshape(T, K))
    if not idx2.is_contiguous():
        idx2 = idx2.contiguous()
    q3 = q.reshape(T, H, D)
    if not q3.is_contiguous():
        q3 = q3.contiguous()
    kv_seq_stride = 0
    if block_table is not None:
        if per_sequence:
            raise ValueError("per_sequence addressing and a block table exclude each other")
    else:
        if per_sequence is None:
            per_sequence = kv_cache.dim() >= 3 and kv_cache.shape[0] == B and B > 1
        if per_sequence:
            if kv_cache.dim() < 3 or kv_cache.shape[0] != B:
                raise ValueError("per_sequence=True needs kv_cache [B, rows per sequence, ..., D]")
            kv_seq_stride = kv_cache[0].numel() // kv_cache.shape[-1]      # rows per sequence
    kv2 = kv_cache.reshape(-1, kv_cache.shape[-1])
    if not kv2.is_contiguous():
        kv2 = kv2.contiguous()
    if block_table is not None:
        if block_table.dim() != 2 or block_table.shape[0] != B:
            raise ValueError("block_table must be [B, max_pages]")
        if block_table.dtype != torch.int32 or not _lib.on_device(block_table):
            raise ValueError("block_table must be an int32 device tensor")
        block_table = block_table.contiguous()
    out_shape = (B, S, H, D_V) if q.dim() == 4 else (T, H, D_V)
    lse_shape = out_shape[:-1]
    return q3, kv2, idx2, B, S, H, K, fmt, kv_seq_stride, block_table, out_shape, lse_shape


_workspaces = {}    # (device, stream) -> initialised workspace tensor (grown on demand)


def make_workspace(n_bytes, device):
    """Allocate a split workspace, zero its arrival words and write its header (once per allocation).
    Calls that share a workspace must not overlap: give every stream its own."""
    ws = torch.empty(max(int(n_bytes), _lib.SMLA_WS_COUNTER_BYTES), dtype=torch.uint8, device=device)
    rc = _lib.load().smla_workspace_init(ws.data_ptr(), ws.numel(), _stream(ws))
    _lib.check(rc, "smla_workspace_init")
    return ws


def workspace_status(workspace=None, device=None):
    """Wait for the current stream and report what the split launches left in ``workspace``'s header.
    Returns 0 when healthy; otherwise raises RuntimeError naming the SMLA_WS_STATUS bits, after the
    library has initialised the workspace again.

    ``workspace=None`` checks the workspace ``sparse_mla_fwd`` / ``decode_attention_fwd`` keep for
    the current stream of ``device`` (default: the current device); 0 when no split launch has
    needed one yet.  A launch whose merge gave up marks its rows with a NaN LSE and flags the
    workspace, and every later split launch on that workspace gives up too until this function has
    run: a serving loop calls it wherever it synchronises anyway (it waits for the stream)."""
    if workspace is None:
        device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if device.type == "cuda" and device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        workspace = _workspaces.get((device, _lib.stream_handle(device)))
        if workspace is None:
            return 0
    _check_workspace(workspace, 0, workspace.device)
    import ctypes
    status = ctypes.c_uint32(0)
    rc = _lib.load().smla_workspace_status(workspace.data_ptr(), workspace.numel(), _stream(workspace),
                                           ctypes.byref(status))
    if rc == _lib.SMLA_EWORKSPACE_STATE:
        what = ", ".join(name for bit, name in _lib.WS_STATUS_BITS.items() if status.value & bit)
        raise RuntimeError(f"split workspace flagged by a launch: {what} (status {status.value})")
    _lib.check(rc, "smla_workspace_status")
    return 0


def _check_workspace(workspace, need, device):
    if not isinstance(workspace, torch.Tensor) or not _lib.on_device(workspace) or workspace.device != device:
        raise ValueError("workspace must be a tensor on the inputs' device (see make_workspace)")
    if workspace.dtype != torch.uint8 or not workspace.is_contiguous():
        raise ValueError("workspace must be a contiguous uint8 tensor (see make_workspace)")
    if workspace.numel() < max(need, _lib.SMLA_WS_COUNTER_BYTES):
        raise ValueError(f"workspace too small: {max(need, _lib.SMLA_WS_COUNTER_BYTES)} bytes needed (see make_workspace)")


def _default_workspace(n_bytes, device):
    # One workspace per (device, stream): launches on one stream run in order, so they may share
    # the arrival words and partials; launches on different streams may overlap and must not.
    # A workspace that has to grow is replaced; the old tensor goes back to torch's allocator,
    # which keeps it away from other streams until this stream's queued work is done.
    key = (device, _lib.stream_handle(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < n_bytes:
        ws = make_workspace(n_bytes, device)
        _workspaces[key] = ws
    return ws


def _resolve_workspace(workspace, ws_bytes, device):
    """(pointer, size) of the workspace a split launch uses: the caller's (validated) or the stream's own."""
    if not ws_bytes:
        return None, 0
    if workspace is None:
        workspace = _default_workspace(ws_bytes, device)
    else:
        _check_workspace(workspace, ws_bytes, device)
    return workspace.data_ptr(), workspace.numel()


def plan_splits(n_tokens, n_heads, topk, kv_format="bf16"):
    """Split count ``sparse_mla_fwd`` uses when ``n_splits`` is None."""
    return _lib.load().smla_plan_splits(_FORMATS[kv_format], n_tokens, n_heads, topk)


def sparse_mla_fwd(q, kv_cache, indices, sm_scale=None, d_v=D_V, *, block_table=None, page_size=64,
                   kv_format=None, n_splits=None, lse_base2=False, workspace=None, per_sequence=None):
    """Sparse MLA forward: attend each query token to its top-k latent KV rows.

    q         [B, S, H, 576] (or [T, H, 576]) bf16; fp32 for the fp32 plumbing format
    kv_cache  latent rows, last dim 576 (bf16 / fp32) or 656 (uint8 fp8 records); leading dims
              are flattened: [pages, page_size, 576], [B, S_kv, 1, 576], [N, 576] ...
    indices   [B, S, topk] int32; -1 = padding.  With ``block_table`` [B, max_pages] they are
              logical positions translated through the table (page_size tokens per page);
              without it they address kv_cache rows of the token's own sequence
              (``per_sequence=True``; the default when kv_cache has a leading batch dim and
              B > 1) or rows of one shared pool (``per_sequence=False``).  int64 is accepted;
              values past int32 are masked like any index past the cache.
    workspace only for split launches: a tensor from ``make_workspace``; default = one per
              (device, stream), since launches that share a workspace must not overlap.
    Returns (out [B, S, H, 512] in q's dtype, lse [B, S, H] fp32, natural log unless lse_base2).
    """
    q3, kv2, idx2, B, S, H, K, fmt, kv_seq_stride, block_table, out_shape, lse_shape = _normalise(
        q, kv_cache, indices, d_v, block_table, kv_format, per_sequence)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D_QK)
    lib = _lib.load()
    T = B * S
    out = torch.empty((T, H, D_V), dtype=q.dtype, device=q.device)
    lse = torch.empty((T, H), dtype=torch.float32, device=q.device)
    ns = 0 if n_splits is None else int(n_splits)
    if ns < 0 or ns > _lib.SMLA_MAX_SPLITS:
        raise ValueError(f"n_splits must be in [1, {_lib.SMLA_MAX_SPLITS}]")
    eff = ns if ns else lib.smla_plan_splits(fmt, T, H, K)
    ws_bytes = lib.smla_workspace_bytes(T, H, D_V, eff)
    ws_ptr, ws_bytes = _resolve_workspace(workspace, ws_bytes, q.device)
    rc = lib.smla_fwd(fmt, q3.data_ptr(), kv2.data_ptr(), idx2.data_ptr(),
                      block_table.data_ptr() if block_table is not None else None,
                      out.data_ptr(), lse.data_ptr(), T, S, H, K, D_QK, D_V, page_size,
                      block_table.shape[1] if block_table is not None else 0,
                      kv_seq_stride, kv2.shape[0], float(sm_scale), eff, ws_ptr, ws_bytes, _stream(q))
    _lib.check(rc, "smla_fwd")
    if lse_base2:
        lse = lse * math.log2(math.e)
    return out.view(out_shape), lse.view(lse_shape)


def sparse_mla_fwd_scalar(q, kv_cache, indices, sm_scale=None, d_v=D_V, *, block_table=None,
                          page_size=64, kv_format=None, per_sequence=None):
    """Same operator on the exact-fp32 scalar device kernel (slow; cross-check for the MFMA path)."""
    q3, kv2, idx2, B, S, H, K, fmt, kv_seq_stride, block_table, out_shape, lse_shape = _normalise(
        q, kv_cache, indices, d_v, block_table, kv_format, per_sequence)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D_QK)
    lib = _lib.load()
    T = B * S
    out = torch.empty((T, H, D_V), dtype=q.dtype, device=q.device)
    lse = torch.empty((T, H), dtype=torch.float32, device=q.device)
    rc = lib.smla_fwd_scalar(fmt, q3.data_ptr(), kv2.data_ptr(), idx2.data_ptr(),
                             block_table.data_ptr() if block_table is not None else None,
                             out.data_ptr(), lse.data_ptr(), T, S, H, K, D_QK, D_V, page_size,
                             block_table.shape[1] if block_table is not None else 0,
                             kv_seq_stride, kv2.shape[0], float(sm_scale), _stream(q))
    _lib.check(rc, "smla_fwd_scalar")
    return out.view(out_shape), lse.view(lse_shape)


def gather_rows(kv_cache, indices, *, block_table=None, page_size=64, tokens_per_seq=1,
                kv_seq_stride=0, with_rows=True):
    """Translate + mask + gather only.  kv_cache [..., W] any dtype (row = W elements, a multiple
    of 16 bytes); indices [T, topk].  Returns (phys int32 [T, topk] with -1 = masked,
    rows [T, topk, W] with zero rows where masked, or None)."""
    if not _lib.on_device(kv_cache) or not _lib.on_device(indices):
        raise ValueError("gather_rows needs device tensors (there is no CPU path)")
    kv2 = kv_cache.reshape(-1, kv_cache.shape[-1]).contiguous()
    if indices.dtype not in (torch.int32, torch.int64):
        raise ValueError("indices must be int32 or int64")
    idx2 = _indices_i32(indices.reshape(-1, indices.shape[-1])).contiguous()
    T, K = idx2.shape
    row_bytes = kv2.shape[1] * kv2.element_size()
    phys = torch.empty((T, K), dtype=torch.int32, device=kv2.device)
    rows = torch.empty((T, K, kv2.shape[1]), dtype=kv2.dtype, device=kv2.device) if with_rows else None
    if block_table is not None:
        if block_table.dtype != torch.int32 or not _lib.on_device(block_table):
            raise ValueError("block_table must be an int32 device tensor")
        block_table = block_table.contiguous()
    lib = _lib.load()
    rc = lib.smla_gather_rows(kv2.data_ptr(), row_bytes, idx2.data_ptr(),
                              block_table.data_ptr() if block_table is not None else None,
                              phys.data_ptr(), rows.data_ptr() if rows is not None else None,
                              T, tokens_per_seq, K, page_size,
                              block_table.shape[1] if block_table is not None else 0,
                              kv_seq_stride, kv2.shape[0], _stream(kv2))
    _lib.check(rc, "smla_gather_rows")
    return phys, rows


def merge_splits(part_out, part_lse):
    """part_out fp32 [T, n_splits, H, 512], part_lse fp32 [T, n_splits, H] -> (out bf16 [T, H, 512], lse [T, H])."""
    if not _lib.on_device(part_out):
        raise ValueError("merge_splits needs device tensors (there is no CPU path)")
    T, ns, H, dv = part_out.shape
    part_out = part_out.contiguous().float()
    part_lse = part_lse.contiguous().float()
    out = torch.empty((T, H, dv), dtype=torch.bfloat16, device=part_out.device)
    lse = torch.empty((T, H), dtype=torch.float32, device=part_out.device)
    rc = _lib.load().smla_merge_splits(part_out.data_ptr(), part_lse.data_ptr(), out.data_ptr(),
                                       lse.data_ptr(), T, H, dv, ns, _stream(part_out))
    _lib.check(rc, "smla_merge_splits")
    return out, lse


def quantize_kv_fp8(latent, records=None, slot=None):
    """KV-cache writer for the fp8 format: latent bf16 [N, 576] -> uint8 records [rows, 656].
    ``slot`` int64 [N] names the destination row of each latent row (negative = skip)."""
    if not _lib.on_device(latent):
        raise ValueError("quantize_kv_fp8 needs device tensors (there is no CPU path)")
    if latent.dtype != torch.bfloat16 or latent.shape[-1] != D_QK:
        raise ValueError("latent must be bf16 [..., 576]")
    src = latent.reshape(-1, D_QK).contiguous()
    n = src.shape[0]
    if records is None:
        if slot is not None:
            raise ValueError("slot needs an existing records buffer")
        records = torch.empty((n, _lib.FP8_RECORD_BYTES), dtype=torch.uint8, device=src.device)
    rec2 = records.view(-1, _lib.FP8_RECORD_BYTES)
    if slot is not None:
        slot = slot.to(torch.int64).contiguous()
    rc = _lib.load().smla_kv_quantize_fp8(src.data_ptr(), slot.data_ptr() if slot is not None else None,
                                          rec2.data_ptr(), n, rec2.shape[0], _stream(src))
    _lib.check(rc, "smla_kv_quantize_fp8")
    return records


def reshape_and_cache(latent, kv_cache, slot_mapping, kv_format="bf16"):
    """KV-cache writer: ``kv_cache[slot_mapping[i]] = latent[i]`` in the cache's row format.

    Mirrors the reference's ``reshape_and_cache(key, value, key_cache, value_cache, slot_mapping, ...)``
    (/root/reference/third_party/cambricon/python/triton/ops/reshape_and_cache.py:48-75) for a cache
    that holds one latent row per token: ``latent`` bf16 [num_tokens, 576]; ``kv_cache`` bf16
    [..., 576] ("bf16") or uint8 [..., 656] records ("fp8_e4m3_b128", quantised on the way in);
    ``slot_mapping`` int64 [num_tokens] = page * page_size + offset, negative = skip.  Returns None,
    like the reference (the cache is updated in place)."""
    if not _lib.on_device(latent) or not _lib.on_device(kv_cache) or not _lib.on_device(slot_mapping):
        raise ValueError("reshape_and_cache needs device tensors (there is no CPU path)")
    if latent.dtype != torch.bfloat16 or latent.shape[-1] != D_QK:
        raise ValueError("latent must be bf16 [..., 576]")
    if kv_format == "bf16":
        if kv_cache.dtype != torch.bfloat16 or kv_cache.shape[-1] != D_QK:
            raise ValueError("a bf16 cache has rows of 576 bf16")
    elif kv_format == "fp8_e4m3_b128":
        if kv_cache.dtype != torch.uint8 or kv_cache.shape[-1] != _lib.FP8_RECORD_BYTES:
            raise ValueError("an fp8 cache has rows of 656 bytes")
    else:
        raise ValueError(f"unknown kv_format {kv_format!r}")
    if not kv_cache.is_contiguous():
        raise ValueError("kv_cache must be contiguous")
    src = latent.reshape(-1, D_QK).contiguous()
    slot = slot_mapping.reshape(-1)
    if slot.dtype != torch.int64 or not slot.is_contiguous():
        slot = slot.to(torch.int64).contiguous()
    if slot.shape[0] != src.shape[0]:
        raise ValueError("slot_mapping needs one entry per latent row")
    rows = kv_cache.numel() // kv_cache.shape[-1]
    rc = _lib.load().smla_kv_write(_FORMATS[kv_format], src.data_ptr(), slot.data_ptr(), kv_cache.data_ptr(),
                                   src.shape[0], rows, _stream(src))
    _lib.check(rc, "smla_kv_write")


def topk_indices(scores, k, context_lens=None, workspace=None, *, block_table=None, page_size=64, kv_rows=None,
                 rows_per_seq=1):
    """Top-k index producer: int32 [..., k] indices of the k largest entries of each row of ``scores``
    (f32 [..., N]) among its first ``context_lens[row]`` entries (default N), ascending, -1 padded.
    Ties at the k-th value go to the lower index.  The reference only has ``topk`` as a language
    primitive returning values (/root/reference/third_party/metax/python/triton/language/standard.py:443).
    Few long rows are cut into parts, one workgroup each, through a scratch buffer: ``workspace``
    (a uint8 device tensor of ``topk_workspace_bytes`` bytes, e.g. kept by a serving loop), or one
    allocated here for the call; ``workspace=False`` keeps one workgroup per row.  Same result
    every way.

    With ``block_table`` [n_seqs, max_pages] (int32, row r belongs to sequence r // rows_per_seq) the
    selected positions are written as physical rows of the paged cache of ``kv_rows`` rows
    (``page_size`` positions a page; -1 where the table masks a position): a list to hand to
    ``sparse_mla_fwd(..., block_table=None, per_sequence=False)``, which then skips its own
    page-table look-up."""
    if not _lib.on_device(scores):
        raise ValueError("topk_indices needs device tensors (there is no CPU path)")
    if scores.dtype != torch.float32:
        raise ValueError("scores must be float32")
    if k <= 0:
        raise ValueError("k must be positive")
    lead, n = scores.shape[:-1], scores.shape[-1]
    s2 = scores.reshape(-1, n)
    if s2.stride(-1) != 1:
        s2 = s2.contiguous()
    rows = s2.shape[0]
    cl = None
    if context_lens is not None:
        cl = context_lens.reshape(-1).to(torch.int32).contiguous()
        if cl.shape[0] != rows or not _lib.on_device(cl):
            raise ValueError("context_lens needs one device entry per row")
    out = torch.empty((rows, k), dtype=torch.int32, device=scores.device)
    lib = _lib.load()
    need = lib.smla_topk_workspace_bytes(rows, n, k)
    if workspace is False:
        workspace = None
    elif workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=scores.device)
    elif workspace is not None:
        if workspace.dtype != torch.uint8 or not workspace.is_contiguous() or not _lib.on_device(workspace):
            raise ValueError("workspace must be a contiguous uint8 device tensor")
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_len = workspace.numel() if workspace is not None else 0
    if block_table is None:
        rc = lib.smla_topk_indices(s2.data_ptr(), cl.data_ptr() if cl is not None else None, out.data_ptr(),
                                   rows, n, s2.stride(0) if rows > 1 else n, k, ws_ptr, ws_len, _stream(s2))
        _lib.check(rc, "smla_topk_indices")
        return out.reshape(*lead, k)
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or not _lib.on_device(block_table):
        raise ValueError("block_table must be an int32 device tensor [n_seqs, max_pages]")
    if kv_rows is None or rows_per_seq <= 0 or rows % rows_per_seq != 0 or block_table.shape[0] != rows // rows_per_seq:
        raise ValueError("with block_table: kv_rows, and one table row per rows_per_seq score rows")
    bt = block_table.contiguous()
    rc = lib.smla_topk_rows(s2.data_ptr(), cl.data_ptr() if cl is not None else None, bt.data_ptr(), out.data_ptr(),
                            rows, n, s2.stride(0) if rows > 1 else n, k, rows_per_seq, page_size, bt.shape[1], int(kv_rows),
                            ws_ptr, ws_len, _stream(s2))
    _lib.check(rc, "smla_topk_rows")
    return out.reshape(*lead, k)


def topk_workspace_bytes(n_rows, n_cols, k):
    """Bytes of scratch with which ``topk_indices`` cuts rows of this shape into parts (0: it would not)."""
    return _lib.load().smla_topk_workspace_bytes(n_rows, n_cols, k)


def decode_attention_fwd(q, k_buffer, v_buffer, o, req_to_token, b_seq_len, attn_logits=None, num_kv_splits=None,
                         sm_scale=None, page_size=1, logit_cap=0.0, en_wmma=True, *, kv_format=None, workspace=None):
    """Dense MLA decode over the whole paged context of every sequence (no index list).

    Mirrors the reference's ``decode_attention_fwd(q, k_buffer, v_buffer, o, req_to_token, b_seq_len,
    attn_logits, num_kv_splits, sm_scale, page_size, logit_cap)``
    (/root/reference/third_party/mthreads/python/test/wmma/test_accuracy_musa_vllm_mla.py:571-620)
    for the latent cache of MLA, where the values are the first 512 columns of the keys:
      q            [B, H, 576] bf16, one new token per sequence
      k_buffer     latent cache, [rows, 576] / [pages, page_size, 576] / [rows, 1, 576] bf16, or uint8
                   [..., 656] fp8 records
      v_buffer     None, or the view ``k_buffer[..., :512]`` (the reference passes both buffers)
      o            [B, H, 512] output in q's dtype, written in place (None = allocate)
      req_to_token [B, max_pages] int32 page numbers: position p of sequence b lives in cache row
                   ``req_to_token[b, p // page_size] * page_size + p % page_size`` (reference :278-283)
      b_seq_len    [B] int32 context lengths; a length past ``max_pages * page_size`` attends to
                   the positions the table covers
      en_wmma      the reference's switch between its matrix-core and plain kernels; accepted and
                   ignored (there is one kernel)
      attn_logits  the reference's split scratch [B, H, splits, 513]; accepted and ignored (the
                   library's own workspace holds the split partials)
      logit_cap    > 0: every scaled score s becomes ``logit_cap * tanh(s / logit_cap)`` before the
                   softmax (reference :299-302); 0 = off
    Returns (o, lse) with lse [B, H] fp32, natural log."""
    if not (0.0 <= float(logit_cap) < float("inf")):
        raise ValueError("logit_cap must be non-negative and finite (0 = off)")
    if q.dim() != 3 or q.shape[-1] != D_QK:
        raise ValueError("q must be [B, H, 576]")
    for name, t in (("q", q), ("k_buffer", k_buffer), ("req_to_token", req_to_token), ("b_seq_len", b_seq_len)):
        if not _lib.on_device(t):
            raise ValueError(f"{name} must be a device tensor (there is no CPU path)")
    if v_buffer is not None and (v_buffer.data_ptr() != k_buffer.data_ptr() or v_buffer.shape[-1] != D_V or
                                 v_buffer.dtype != k_buffer.dtype or v_buffer.dim() != k_buffer.dim() or
                                 tuple(v_buffer.shape[:-1]) != tuple(k_buffer.shape[:-1]) or
                                 v_buffer.stride() != k_buffer.stride()):
        raise ValueError("v_buffer must be k_buffer[..., :512]: the latent cache holds keys and values in one row")
    B, H, _ = q.shape
    if kv_format is None:
        kv_format = {torch.bfloat16: "bf16", torch.uint8: "fp8_e4m3_b128"}.get(k_buffer.dtype)
    if kv_format not in ("bf16", "fp8_e4m3_b128"):
        raise ValueError("k_buffer must be a bf16 latent cache or uint8 fp8 records")
    row = D_QK if kv_format == "bf16" else _lib.FP8_RECORD_BYTES
    if k_buffer.shape[-1] != row or not k_buffer.is_contiguous():
        raise ValueError(f"k_buffer must be contiguous with rows of {row}")
    if q.dtype != torch.bfloat16:
        raise ValueError("q must be bf16")
    if req_to_token.dim() != 2 or req_to_token.shape[0] != B or req_to_token.dtype != torch.int32:
        raise ValueError("req_to_token must be int32 [B, max_pages]")
    if b_seq_len.shape != (B,):
        raise ValueError("b_seq_len must be [B]")
    seq = b_seq_len.to(torch.int32).contiguous()
    bt = req_to_token.contiguous()
    max_len = bt.shape[1] * int(page_size)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D_QK)
    if o is None:
        o = torch.empty((B, H, D_V), dtype=q.dtype, device=q.device)
    elif o.shape != (B, H, D_V) or o.dtype != q.dtype or not o.is_contiguous():
        raise ValueError("o must be a contiguous [B, H, 512] tensor of q's dtype")
    lse = torch.empty((B, H), dtype=torch.float32, device=q.device)
    lib = _lib.load()
    fmt = _FORMATS[kv_format]
    ns = 0 if not num_kv_splits else int(num_kv_splits)
    if ns < 0 or ns > _lib.SMLA_MAX_SPLITS:
        raise ValueError(f"num_kv_splits must be in [1, {_lib.SMLA_MAX_SPLITS}]")
    eff = ns if ns else lib.smla_plan_splits(fmt, B, H, max_len)
    ws_bytes = lib.smla_workspace_bytes(B, H, D_V, eff)
    ws_ptr, ws_bytes = _resolve_workspace(workspace, ws_bytes, q.device)
    q3 = q.contiguous()
    kv_rows = k_buffer.numel() // row
    rc = lib.smla_decode_dense(fmt, q3.data_ptr(), k_buffer.data_ptr(), seq.data_ptr(), bt.data_ptr(), o.data_ptr(),
                               lse.data_ptr(), B, 1, H, max_len, D_QK, D_V, int(page_size), bt.shape[1], 0, kv_rows,
                               float(sm_scale), float(logit_cap), eff, ws_ptr, ws_bytes, _stream(q))
    _lib.check(rc, "smla_decode_dense")
    return o, lse
