"""Oracle: sparse MLA forward (page translation, top-k gather, softmax, PV, LSE, split merge).

TEST INFRASTRUCTURE ONLY (see package docstring).

Semantics: for every query token t and head h, with I = indices[t, :],
V = {j : I[j] names a valid row},
    score_j = sm_scale * <q[t,h,:], kv[I[j], :]>
    lse     = log sum_{j in V} exp(score_j)                    (natural log)
    out     = sum_{j in V} exp(score_j - lse) * kv[I[j], :d_v]
A token with no valid index yields out = 0, lse = -inf.  Duplicated indices
count once per occurrence.  Non-negative indices that fall outside the cache
are treated as invalid.

Conventions followed (the operator itself is absent from the checkout):
  * 576 = 512 NoPE + 64 RoPE split, one latent KV row shared by all heads,
    scores scaled after the dot product, masked entries excluded, and
    LSE = max + log(sum) in natural log:
    /root/reference/third_party/mthreads/python/test/wmma/test_accuracy_musa_vllm_mla.py:290-299, :313-320, :333-337
  * page translation phys = page_number * PAGE_SIZE + pos % PAGE_SIZE:
    same file :278-283; block-table layout [num_seqs, max_pages]:
    /root/reference/third_party/cambricon/python/triton/ops/paged_attention.py:33-53
  * split merge with exp(lse_i - max) weights: same mthreads file :426-477.

Pinned by (tests/test_oracle_mla.py): dense special case == softmax attention
computed by torch.nn.functional.scaled_dot_product_attention and by
scipy.special.logsumexp/softmax; sum_j p_j == 1; permutation invariance;
padding invariance; K=1 closed form; equal-keys closed form; split/merge
identity; brute-force scalar loops on tiny inputs; translation against a
per-element python loop.  "Parity unpinned -- fixed by decision": LSE base,
fully-masked rows, duplicates, out-of-range handling, tensor ranks.
"""
import numpy as np


def translate_indices(indices, block_table=None, page_size=64, kv_rows=None,
                      tokens_per_seq=1, kv_seq_stride=0):
    """Logical top-k positions -> physical row ids (int64), -1 where invalid.

    indices      [T, K] integers, T = batch * tokens_per_seq, token t belongs to
                 sequence t // tokens_per_seq.
    block_table  [B, max_pages] physical page numbers or None.
    With a block table: phys = block_table[b, i // P] * P + i % P, valid iff
    0 <= i < max_pages*P, the page entry is >= 0 and phys < kv_rows.
    Without: phys = b * kv_seq_stride + i, valid iff 0 <= i < (kv_seq_stride or kv_rows).
    """
    idx = np.asarray(indices).astype(np.int64)
    T, K = idx.shape
    seq = (np.arange(T) // tokens_per_seq)[:, None]
    if block_table is not None:
        bt = np.asarray(block_table).astype(np.int64)
        cap = bt.shape[1] * page_size
        ok = (idx >= 0) & (idx < cap)
        safe = np.where(ok, idx, 0)
        page = bt[seq, safe // page_size]
        phys = page * page_size + safe % page_size
        ok &= page >= 0
    else:
        lim = kv_seq_stride if kv_seq_stride else kv_rows
        ok = idx >= 0
        if lim is not None:
            ok &= idx < lim
        phys = seq * kv_seq_stride + np.where(ok, idx, 0)
    if kv_rows is not None:
        ok &= phys < kv_rows
    return np.where(ok, phys, -1)


def gather_rows(rows, phys):
    """rows [N, W] (any dtype, compared as raw bytes) and phys [T, K] -> [T, K, W];
    invalid entries (phys < 0) give all-zero rows."""
    rows = np.asarray(rows)
    phys = np.asarray(phys)
    out = rows[np.where(phys >= 0, phys, 0)]
    out[phys < 0] = 0
    return out


def sparse_mla_fwd(q, kv, phys, sm_scale, d_v=512, dtype=np.float64, logit_cap=0.0):
    """q [T, H, D], kv [N, D] (already dequantised values), phys [T, K] physical
    row ids with -1 = invalid  ->  (out [T, H, d_v], lse [T, H]) in ``dtype``.

    ``logit_cap`` > 0 squashes every scaled score before the mask and the maximum, as the
    reference's MLA decode kernels do: ``qk = logit_cap * tanh(qk / logit_cap)`` after
    ``qk *= sm_scale`` (/root/reference/third_party/mthreads/python/test/wmma/
    test_accuracy_musa_vllm_mla.py:299-302, :109-111).  Pinned by tests/test_oracle_mla.py: a
    per-element loop with math.tanh, the equal-keys closed form lse = cap tanh(s / cap) + log n,
    the bound lse <= cap + log n, and the limit cap -> infinity (no cap)."""
    q = np.asarray(q, dtype=dtype)
    kv = np.asarray(kv, dtype=dtype)
    phys = np.asarray(phys)
    T, H, D = q.shape
    out = np.zeros((T, H, d_v), dtype=dtype)
    lse = np.full((T, H), -np.inf, dtype=dtype)
    for t in range(T):
        sel = phys[t][phys[t] >= 0]
        if sel.size == 0:
            continue
        rows = kv[sel]                                   # [n, D]
        s = (q[t] @ rows.T) * dtype(sm_scale)            # [H, n]
        if logit_cap > 0:
            s = dtype(logit_cap) * np.tanh(s / dtype(logit_cap))
        m = s.max(axis=1, keepdims=True)
        e = np.exp(s - m)
        l = e.sum(axis=1, keepdims=True)
        lse[t] = (m + np.log(l))[:, 0]
        out[t] = (e / l) @ rows[:, :d_v]
    return out, lse


def split_partials(q, kv, phys, sm_scale, d_v, n_splits, dtype=np.float64):
    """Partials of a split top-k list: split i covers a contiguous slice of the K axis.
    Returns (out_i [n_splits, T, H, d_v], lse_i [n_splits, T, H])."""
    K = phys.shape[1]
    per = -(-K // n_splits)
    outs, lses = [], []
    for i in range(n_splits):
        o, l = sparse_mla_fwd(q, kv, phys[:, i * per:(i + 1) * per], sm_scale, d_v, dtype)
        outs.append(o)
        lses.append(l)
    return np.stack(outs), np.stack(lses)


def merge_splits(out_i, lse_i):
    """Merge normalised partials: w_i = exp(lse_i - lse*) / sum, lse = lse* + log sum exp(lse_i - lse*).
    Splits with lse_i = -inf contribute nothing; all -inf gives out = 0, lse = -inf."""
    out_i = np.asarray(out_i)
    lse_i = np.asarray(lse_i)
    m = lse_i.max(axis=0)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    w = np.exp(lse_i - m_safe)                            # exp(-inf) = 0
    tot = w.sum(axis=0)
    with np.errstate(divide="ignore", invalid="ignore"):
        lse = np.where(tot > 0, m_safe + np.log(tot), -np.inf)
        wn = np.where(tot > 0, w / np.where(tot > 0, tot, 1.0), 0.0)
    out = (wn[..., None] * out_i).sum(axis=0)
    return out, lse


def topk_indices(scores, k, context_lens=None):
    """Indices of the k largest entries of each row among its first context_lens[row] entries,
    ascending, padded with -1; ties at the k-th value go to the lower index; NaN counts as -inf.

    The reference offers the selection only as ``topk`` returning the k largest values
    (/root/reference/third_party/metax/python/triton/language/standard.py:443-444); index output,
    order and tie rule are fixed by decision ("parity unpinned" against the reference).  Pinned by
    tests/test_oracle_mla.py: against a selection written as repeated "take the current maximum,
    lowest index first", and through its values against a descending sort (what the reference's
    ``topk`` returns)."""
    scores = np.asarray(scores, dtype=np.float32)
    lead, n = scores.shape[:-1], scores.shape[-1]
    s2 = scores.reshape(-1, n)
    out = np.full((s2.shape[0], k), -1, dtype=np.int32)
    for r in range(s2.shape[0]):
        m = n if context_lens is None else int(np.clip(np.asarray(context_lens).reshape(-1)[r], 0, n))
        row = s2[r, :m].astype(np.float64)
        row = np.where(np.isnan(row), -np.inf, row)
        # stable sort on value descending: lower index first among equals
        order = np.lexsort((np.arange(m), -row))
        sel = np.sort(order[:min(k, m)])
        out[r, :sel.size] = sel
    return out.reshape(*lead, k)
