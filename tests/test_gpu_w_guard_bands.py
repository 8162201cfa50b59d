"""GPU check that no entry point writes outside the buffers it is given.

Every output lives in the middle of a larger buffer filled with a byte pattern, 64 KB of it on
either side; after the call through the C ABI the pattern must be intact and the output must be
bit-identical to what the Python wrapper (whose results the parity tests check) returns for the
same inputs.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

GUARD = 1 << 16
PATTERN = 0xA5


class Banded:
    """`nbytes` of device memory with guard bands; `view(dtype, shape)` is the caller's buffer."""

    def __init__(self, nbytes, dev, fill=None):
        self.buf = torch.full((GUARD + nbytes + GUARD + 256,), PATTERN, dtype=torch.uint8, device=dev)
        self.off = GUARD + (-(self.buf.data_ptr() + GUARD)) % 256
        self.nbytes = nbytes
        if fill is not None:
            self.buf[self.off:self.off + nbytes] = fill

    def view(self, dtype, shape):
        return self.buf[self.off:self.off + self.nbytes].view(dtype).view(shape)

    def ptr(self):
        return self.buf.data_ptr() + self.off

    def intact(self):
        lo = self.buf[:self.off]
        hi = self.buf[self.off + self.nbytes:]
        return bool((lo == PATTERN).all().item() and (hi == PATTERN).all().item())


def _stream(dev):
    from flagtree_amd import _lib
    return _lib.stream_handle(dev)


def _forward_banded(cfg, n_splits, dev):
    import flagtree_amd as ft
    from flagtree_amd import _lib, sparse_mla
    lib = _lib.load()
    q3, kv2, idx2, B, S, H, K, fmt, kv_seq_stride, bt, out_shape, lse_shape = sparse_mla._normalise(
        cfg["q"], cfg["kv_cache"], cfg["indices"], 512, cfg["block_table"], cfg["kv_format"])
    T = B * S
    esz = cfg["q"].element_size()
    out_b = Banded(T * H * 512 * esz, dev)
    lse_b = Banded(T * H * 4, dev)
    eff = n_splits if n_splits else lib.smla_plan_splits(fmt, T, H, K)
    ws_bytes = lib.smla_workspace_bytes(T, H, 512, eff)
    ws_b = None
    if ws_bytes:
        ws_b = Banded(ws_bytes, dev, fill=0)
        _lib.check(lib.smla_workspace_init(ws_b.ptr(), ws_bytes, _stream(dev)), "smla_workspace_init")
    rc = lib.smla_fwd(fmt, q3.data_ptr(), kv2.data_ptr(), idx2.data_ptr(), bt.data_ptr() if bt is not None else None,
                      out_b.ptr(), lse_b.ptr(), T, S, H, K, 576, 512, cfg["page_size"],
                      bt.shape[1] if bt is not None else 0, kv_seq_stride, kv2.shape[0], float(cfg["sm_scale"]),
                      eff, ws_b.ptr() if ws_b else None, ws_bytes, _stream(dev))
    _lib.check(rc, "smla_fwd")
    torch.cuda.synchronize()
    ref_out, ref_lse = ft.sparse_mla_fwd(cfg["q"], cfg["kv_cache"], cfg["indices"], cfg["sm_scale"], 512,
                                         block_table=cfg["block_table"], page_size=cfg["page_size"],
                                         kv_format=cfg["kv_format"], n_splits=eff)
    assert out_b.intact() and lse_b.intact() and (ws_b is None or ws_b.intact())
    got_out = out_b.view(cfg["q"].dtype, (T, H, 512))
    got_lse = lse_b.view(torch.float32, (T, H))
    assert torch.equal(got_out.view(torch.int16 if esz == 2 else torch.int32),
                       ref_out.reshape(T, H, 512).view(torch.int16 if esz == 2 else torch.int32))
    assert torch.equal(got_lse, ref_lse.reshape(T, H))


@pytest.mark.parametrize("heads", [128, 96, 16, 8])
@pytest.mark.parametrize("n_splits", [1, 3])
def test_forward_bf16_stays_inside_its_buffers(dev, heads, n_splits):
    from flagtree_amd import workloads
    cfg = workloads.decode_bf16(dev, batch=3, heads=heads, pages_per_seq=48, topk=520, pad_frac=0.07)
    _forward_banded(cfg, n_splits, dev)


@pytest.mark.parametrize("heads", [128, 16])
@pytest.mark.parametrize("n_splits", [1, 2])
def test_forward_fp8_stays_inside_its_buffers(dev, heads, n_splits):
    from flagtree_amd import workloads
    cfg = workloads.decode_fp8(dev, batch=3, heads=heads, pages_per_seq=40, topk=300)
    _forward_banded(cfg, n_splits, dev)


def test_forward_f32_plumbing_stays_inside_its_buffers(dev):
    from flagtree_amd import workloads
    _forward_banded(workloads.plumbing_f32(dev), 1, dev)


@pytest.mark.parametrize("rows,n,k", [(5, 4097, 2048), (3, 1000, 64), (2, 70000, 2048), (1100, 520, 128), (7, 33, 40)])
def test_topk_indices_stays_inside_its_buffer(dev, rows, n, k):
    import flagtree_amd as ft
    from flagtree_amd import _lib
    g = torch.Generator(device=dev).manual_seed(rows * 131 + n)
    scores = torch.randn((rows, n), generator=g, device=dev)
    lens = torch.randint(0, n + 1, (rows,), generator=g, device=dev, dtype=torch.int32)
    out_b = Banded(rows * k * 4, dev)
    rc = _lib.load().smla_topk_indices(scores.data_ptr(), lens.data_ptr(), out_b.ptr(), rows, n, n, k, None, 0, _stream(dev))
    _lib.check(rc, "smla_topk_indices")
    torch.cuda.synchronize()
    ref = ft.topk_indices(scores, k, context_lens=lens)
    assert out_b.intact()
    assert torch.equal(out_b.view(torch.int32, (rows, k)), ref)


@pytest.mark.parametrize("fmt,row_bytes", [("bf16", 1152), ("fp8_e4m3_b128", 656)])
def test_cache_writer_stays_inside_the_cache(dev, fmt, row_bytes):
    import flagtree_amd as ft
    from flagtree_amd import _lib
    g = torch.Generator(device=dev).manual_seed(17)
    n_tok, cache_rows = 290, 257
    latent = (torch.randn((n_tok, 576), generator=g, device=dev) * 0.3).to(torch.bfloat16)
    slots = torch.randperm(cache_rows + 40, generator=g, device=dev)[:n_tok].to(torch.int64) - 20   # some negative, some past the pool
    cache_b = Banded(cache_rows * row_bytes, dev, fill=0)
    code = {"bf16": _lib.SMLA_KV_BF16, "fp8_e4m3_b128": _lib.SMLA_KV_FP8_B128}[fmt]
    rc = _lib.load().smla_kv_write(code, latent.data_ptr(), slots.data_ptr(), cache_b.ptr(), n_tok, cache_rows, _stream(dev))
    _lib.check(rc, "smla_kv_write")
    torch.cuda.synchronize()
    if fmt == "bf16":
        ref = torch.zeros((cache_rows, 576), dtype=torch.bfloat16, device=dev)
    else:
        ref = torch.zeros((cache_rows, 656), dtype=torch.uint8, device=dev)
    ft.reshape_and_cache(latent, ref, slots, kv_format=fmt)
    assert cache_b.intact()
    assert torch.equal(cache_b.view(torch.uint8, (cache_rows, row_bytes)), ref.view(torch.uint8).view(cache_rows, row_bytes))


@pytest.mark.parametrize("m,n,k,chunks", [(256, 256, 64, 2), (384, 512, 192, 3), (128, 256, 64, 1)])
def test_local_gemm_stays_inside_its_buffer(dev, m, n, k, chunks):
    import flagtree_amd as ft
    from flagtree_amd import _lib
    g = torch.Generator(device=dev).manual_seed(m + n + k)
    x = (torch.randn((m, k), generator=g, device=dev) * 0.1).to(torch.bfloat16)
    w = (torch.randn((k, n), generator=g, device=dev) * 0.1).to(torch.bfloat16)
    partial = torch.randn((m, n), generator=g, device=dev)
    out_b = Banded(m * n * 2, dev)
    rc = _lib.load().smla_gemm_rs_local(x.data_ptr(), w.data_ptr(), partial.data_ptr(), out_b.ptr(), m, n, k, chunks,
                                        (m // chunks) * n, _stream(dev))
    _lib.check(rc, "smla_gemm_rs_local")
    torch.cuda.synchronize()
    ref = ft.gemm_rs_local(x, w, partial, n_chunks=chunks)
    assert out_b.intact()
    assert torch.equal(out_b.view(torch.int16, (chunks, m // chunks, n)), ref.view(torch.int16))
