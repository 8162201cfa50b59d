"""CPU checks that pin the attention part of the oracle (oracle/sparse_mla.py): library routines,
closed forms, invariants and brute force, chosen so that a dropped scale, a wrong axis, a
mis-translated page or a mishandled -1 fails at least one of them."""
import os

import numpy as np
import pytest
import scipy.special
import torch

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _rand(shape, seed, scale=0.3):
    return (np.random.default_rng(seed).standard_normal(shape) * scale)


def test_golden_small_case():
    z = np.load(os.path.join(GOLDEN, "sparse_mla_small.npz"))
    q = oracle.bf16_bits_to_f32(z["q_bf16_bits"])
    kv = oracle.bf16_bits_to_f32(z["kv_bf16_bits"])
    phys = oracle.translate_indices(z["indices"], z["block_table"], int(z["page_size"]), kv_rows=kv.shape[0])
    out, lse = oracle.sparse_mla_fwd(q, kv, phys, float(z["sm_scale"]), 512)
    assert np.abs(out - z["out"]).max() <= 2e-6
    assert np.abs(lse - z["lse"]).max() <= 2e-6


def test_dense_case_equals_library_attention():
    T, H, N = 3, 4, 37
    q, kv = _rand((T, H, 576), 0), _rand((N, 576), 1)
    phys = np.tile(np.arange(N), (T, 1))
    scale = 576 ** -0.5
    out, lse = oracle.sparse_mla_fwd(q, kv, phys, scale, 512)
    tq = torch.from_numpy(q).permute(1, 0, 2)[None]                       # [1, H, T, D]
    tk = torch.from_numpy(kv)[None, None].expand(1, H, N, 576)
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tk[..., :512], scale=scale)
    assert np.abs(out - ref[0].permute(1, 0, 2).numpy()).max() <= 1e-12
    s = np.einsum("thd,nd->thn", q, kv) * scale
    assert np.abs(lse - scipy.special.logsumexp(s, axis=2)).max() <= 1e-12
    assert np.abs(out - np.einsum("thn,nd->thd", scipy.special.softmax(s, axis=2), kv[:, :512])).max() <= 1e-12


def test_probabilities_sum_to_one_and_only_first_dv_columns_are_values():
    q, kv = _rand((2, 3, 576), 2), _rand((50, 576), 3)
    kv[:, :512] = 1.0
    phys = np.array([[4, 9, -1, 30], [-1, -1, 7, 7]])
    out, _ = oracle.sparse_mla_fwd(q, kv, phys, 0.7, 512)
    assert np.abs(out - 1.0).max() <= 1e-12
    kv2 = kv.copy()
    kv2[:, 512:] += 5.0                                                    # rope part moves scores, never values
    out2, lse2 = oracle.sparse_mla_fwd(q, kv2, phys, 0.7, 512)
    assert np.abs(out2 - 1.0).max() <= 1e-12


def test_permutation_and_padding_invariance():
    q, kv = _rand((2, 5, 576), 4), _rand((64, 576), 5)
    rng = np.random.default_rng(6)
    phys = np.stack([rng.permutation(64)[:20] for _ in range(2)])
    o1, l1 = oracle.sparse_mla_fwd(q, kv, phys, 0.2, 512)
    perm = rng.permutation(20)
    o2, l2 = oracle.sparse_mla_fwd(q, kv, phys[:, perm], 0.2, 512)
    padded = np.full((2, 31), -1)
    padded[:, ::2][:, :16] = phys[:, :16]
    padded[:, 1::2][:, :4] = phys[:, 16:]
    o3, l3 = oracle.sparse_mla_fwd(q, kv, padded, 0.2, 512)
    for o, l in ((o2, l2), (o3, l3)):
        assert np.abs(o - o1).max() <= 1e-13 and np.abs(l - l1).max() <= 1e-13


def test_closed_forms_single_key_equal_keys_duplicates_empty():
    q, kv = _rand((1, 4, 576), 7), _rand((10, 576), 8)
    out, lse = oracle.sparse_mla_fwd(q, kv, np.array([[-1, 6, -1]]), 0.3, 512)
    assert np.allclose(out[0], np.broadcast_to(kv[6, :512], (4, 512)), atol=1e-15)
    assert np.allclose(lse[0], 0.3 * q[0] @ kv[6], atol=1e-13)
    kv_eq = np.tile(kv[3], (10, 1))
    out, lse = oracle.sparse_mla_fwd(q, kv_eq, np.array([[0, 1, 2, 5, 9]]), 0.3, 512)
    assert np.allclose(out[0], np.broadcast_to(kv[3, :512], (4, 512)), atol=1e-14)
    assert np.allclose(lse[0], 0.3 * q[0] @ kv[3] + np.log(5), atol=1e-13)
    # a duplicated index counts once per occurrence: [a, a, b] == weights 2:1
    o_dup, l_dup = oracle.sparse_mla_fwd(q, kv, np.array([[1, 1, 2]]), 0.3, 512)
    s = 0.3 * q[0] @ kv[[1, 2]].T
    w = np.exp(s) * np.array([2.0, 1.0])
    assert np.allclose(o_dup[0], (w / w.sum(1, keepdims=True)) @ kv[[1, 2], :512], atol=1e-13)
    assert np.allclose(l_dup[0], np.log(w.sum(1)), atol=1e-13)
    out, lse = oracle.sparse_mla_fwd(q, kv, np.array([[-1, -1]]), 0.3, 512)
    assert (out == 0).all() and np.isneginf(lse).all()


def test_brute_force_scalar_loops():
    T, H, N, K = 2, 2, 9, 5
    q, kv = _rand((T, H, 576), 9), _rand((N, 576), 10)
    phys = np.array([[0, 3, -1, 8, 2], [-1, 1, 1, 4, -1]])
    out, lse = oracle.sparse_mla_fwd(q, kv, phys, 0.11, 512)
    for t in range(T):
        for h in range(H):
            sc = [sum(q[t, h, d] * kv[j, d] for d in range(576)) * 0.11 for j in phys[t] if j >= 0]
            tot = sum(np.exp(x) for x in sc)
            assert abs(lse[t, h] - np.log(tot)) <= 1e-12
            rows = [j for j in phys[t] if j >= 0]
            for d in (0, 17, 511):
                want = sum(np.exp(x) / tot * kv[j, d] for x, j in zip(sc, rows))
                assert abs(out[t, h, d] - want) <= 1e-12


def test_split_merge_identity():
    q, kv = _rand((3, 4, 576), 11), _rand((80, 576), 12)
    rng = np.random.default_rng(13)
    phys = np.stack([rng.permutation(80)[:40] for _ in range(3)])
    phys[0, 10:25] = -1
    phys[1, :20] = -1                                    # an entirely empty split
    full_o, full_l = oracle.sparse_mla_fwd(q, kv, phys, 0.25, 512)
    for ns in (2, 3, 8):
        po, pl = oracle.split_partials(q, kv, phys, 0.25, 512, ns)
        mo, ml = oracle.merge_splits(po, pl)
        assert np.abs(mo - full_o).max() <= 1e-13 and np.abs(ml - full_l).max() <= 1e-13
    mo, ml = oracle.merge_splits(np.zeros((2, 1, 1, 512)), np.full((2, 1, 1), -np.inf))
    assert (mo == 0).all() and np.isneginf(ml).all()


def test_translate_indices_against_python_loop():
    rng = np.random.default_rng(14)
    B, S, pages, P, K = 3, 2, 5, 8, 30
    bt = rng.permutation(B * pages).reshape(B, pages).astype(np.int32)
    bt[1, 2] = -1                                        # an unmapped page
    idx = rng.integers(-2, pages * P + 3, size=(B * S, K)).astype(np.int32)
    kv_rows = B * pages * P - 5                          # a few physical rows fall off the end
    got = oracle.translate_indices(idx, bt, P, kv_rows=kv_rows, tokens_per_seq=S)
    for t in range(B * S):
        for j in range(K):
            i, b = int(idx[t, j]), t // S
            want = -1
            if 0 <= i < pages * P and bt[b, i // P] >= 0:
                phys = int(bt[b, i // P]) * P + i % P
                want = phys if phys < kv_rows else -1
            assert got[t, j] == want
    # no block table: shared pool, and per-sequence stride
    idx2 = np.array([[0, 5, 9, 10, -1], [3, 9, 10, 11, 2]])
    assert np.array_equal(oracle.translate_indices(idx2, None, 64, kv_rows=10), [[0, 5, 9, -1, -1], [3, 9, -1, -1, 2]])
    assert np.array_equal(oracle.translate_indices(idx2, None, 64, kv_rows=24, tokens_per_seq=1, kv_seq_stride=12),
                          [[0, 5, 9, 10, -1], [15, 21, 22, 23, 14]])


def test_gather_rows_zero_fills_masked():
    rows = np.arange(40, dtype=np.int16).reshape(10, 4)
    got = oracle.gather_rows(rows, np.array([[3, -1, 0]]))
    assert np.array_equal(got, [[[12, 13, 14, 15], [0, 0, 0, 0], [0, 1, 2, 3]]])


def test_topk_indices_against_repeated_maximum():
    """Selection restated as: k times, take the largest remaining value, lowest index first."""
    rng = np.random.default_rng(41)
    for n, k, quant in ((1, 1, 0), (7, 3, 0), (50, 50, 0), (64, 70, 0), (200, 16, 4), (333, 128, 2)):
        x = rng.standard_normal((3, n)).astype(np.float32)
        if quant:
            x = np.round(x * quant) / quant                       # many ties
        if n > 5:
            x[0, 2] = np.nan; x[1, 4] = -np.inf; x[2, 1] = np.inf; x[0, 0] = -0.0; x[0, 1] = 0.0
        lens = np.array([n, max(1, n // 2), n], dtype=np.int32)
        got = oracle.topk_indices(x, k, lens)
        for r in range(3):
            m = int(lens[r])
            vals = [(-np.inf if np.isnan(v) else float(v), False) for v in x[r, :m]]
            left = set(range(m))
            picked = []
            for _ in range(min(k, m)):
                best = None
                for i in sorted(left):
                    vi, ni = vals[i]
                    if best is None:
                        best = i
                        continue
                    vb, nb = vals[best]
                    if (nb and not ni) or (nb == ni and vi > vb):
                        best = i
                picked.append(best)
                left.remove(best)
            want = sorted(picked) + [-1] * (k - len(picked))
            assert got[r].tolist() == want, (n, k, r)
    # the values at the selected indices are what a descending sort keeps (the reference's topk)
    x = rng.standard_normal((4, 500)).astype(np.float32)
    idx = oracle.topk_indices(x, 32)
    for r in range(4):
        assert np.array_equal(np.sort(x[r, idx[r]])[::-1], np.sort(x[r])[::-1][:32])


def test_logit_cap_closed_forms_and_loop():
    """cap * tanh(score / cap) before the softmax (reference test_accuracy_musa_vllm_mla.py:299-302)."""
    import math
    rng = np.random.default_rng(5)
    T, H, D, N, K = 2, 3, 576, 40, 17
    q = rng.standard_normal((T, H, D)) * 2.0
    kv = rng.standard_normal((N, D)) * 2.0
    phys = np.stack([rng.permutation(N)[:K] for _ in range(T)])
    phys[0, 3] = -1
    scale, cap = 576 ** -0.5, 1.5                        # raw scores reach +-8: the cap bites
    out, lse = oracle.sparse_mla_fwd(q, kv, phys, scale, 512, logit_cap=cap)
    # element-by-element restatement with math.tanh
    for t in range(T):
        for h in range(H):
            sc, rows = [], []
            for j in range(K):
                if phys[t, j] < 0:
                    continue
                dot = sum(float(q[t, h, d]) * float(kv[phys[t, j], d]) for d in range(D)) * scale
                sc.append(cap * math.tanh(dot / cap))
                rows.append(kv[phys[t, j], :512])
            m = max(sc)
            w = [math.exp(x - m) for x in sc]
            tot = sum(w)
            assert abs(lse[t, h] - (m + math.log(tot))) < 1e-12
            want = sum(wi / tot * r for wi, r in zip(w, rows))
            assert np.abs(out[t, h] - want).max() < 1e-12
    assert (lse <= cap + math.log(K) + 1e-12).all()       # every capped score is below cap
    raw_out, raw_lse = oracle.sparse_mla_fwd(q, kv, phys, scale, 512)
    assert np.abs(lse - raw_lse).max() > 0.5              # ... and the cap changed the result
    big_out, big_lse = oracle.sparse_mla_fwd(q, kv, phys, scale, 512, logit_cap=1e6)
    assert np.abs(big_lse - raw_lse).max() < 1e-9 and np.abs(big_out - raw_out).max() < 1e-9
    # all keys equal: every score is s, so lse = cap tanh(s / cap) + log n and out = v
    kv_same = np.tile(kv[:1], (N, 1))
    o2, l2 = oracle.sparse_mla_fwd(q, kv_same, phys[:, :8].clip(min=0), scale, 512, logit_cap=cap)
    s_raw = (q @ kv_same[0]) * scale
    assert np.abs(l2 - (cap * np.tanh(s_raw / cap) + math.log(8))).max() < 1e-12
    assert np.abs(o2 - kv_same[0, :512]).max() < 1e-12
