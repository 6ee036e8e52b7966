"""GPU parity of every libvtdge operator against the CPU oracle, through the C ABI.

Integer outputs (gate indices, query counts, patch descriptors) are compared bit-exactly;
floating point within the tolerances stated in tests/util.py.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import dge_oracle as orc
from oracle import torch_ref
from util import BF16_ABS, SPLITS, abs_err, assert_close, bf16_round, randn, random_indices, rel_err, rng

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _t(a, dev, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    return t if dtype is None else t.to(dtype)


# ------------------------------------------------------------------ index -> patch
@pytest.mark.parametrize("B,Hr,Wr,extra,splits", [
    (8, 4, 4, 1, [4, 2, 1]),      # config 1 geometry
    (1, 1, 1, 1, [4, 2, 1]),
    (3, 2, 3, 0, [4, 2, 1]),      # non-square, no extra token (PVT-like)
    (5, 8, 8, 2, [4, 2, 1]),      # 512 px geometry, distilled-style 2 extra tokens
    (33, 4, 4, 1, [2, 1]),
    (7, 4, 4, 1, [1]),
    (2, 20, 20, 1, [4, 2, 1]),    # > 256 regions per sample: several passes of the LDS scan
    (1500, 4, 4, 1, [4, 2, 1]),   # count kernel + a write kernel that sums the lengths before its sample
    (256, 14, 14, 0, [4, 2, 1]),  # PVT stage 1 at batch 256: 50176 regions, the same two kernels
    (4097, 2, 2, 1, [4, 2, 1]),   # > 4096 samples: the one-workgroup count-and-scan in several passes, then the write
    (256, 4, 4, 1, [4, 2, 1]),    # the headline batch: one launch, every sample sums the counts before it
    (64, 8, 8, 1, [4, 2, 1]),
    (300, 8, 8, 0, [4, 2, 1]),    # 19200 regions: just past the single-launch limit (count kernel + write)
])
def test_index_to_patch_bit_exact(dev, B, Hr, Wr, extra, splits):
    from vtpack_amd import _C
    R = max(splits)
    idx = random_indices(B * 7 + Hr, B, Hr, Wr, S=len(splits))
    want_p, want_l = orc.index_to_patch(idx, splits, R, extra)
    got_p, got_l = _C.grained_sample_index_to_patch(_t(idx, dev), _t(np.array(splits, dtype=np.int64), dev), R, extra)
    assert got_l.device.type == "cpu" and got_l.dtype == torch.int64
    assert np.array_equal(got_l.numpy(), want_l)
    assert got_p.shape == want_p.shape
    assert np.array_equal(got_p.cpu().numpy(), want_p)


def test_index_to_patch_uniform_gates(dev):
    from vtpack_amd import _C
    sp = _t(np.array(SPLITS, dtype=np.int64), dev)
    for g in range(3):
        idx = np.full((4, 4, 4), g, dtype=np.int64)
        want_p, want_l = orc.index_to_patch(idx, SPLITS, 4, 1)
        got_p, got_l = _C.grained_sample_index_to_patch(_t(idx, dev), sp, 4, 1)
        assert np.array_equal(got_p.cpu().numpy(), want_p) and np.array_equal(got_l.numpy(), want_l)


def test_index_to_patch_dense(dev):
    from vtpack_amd import _C
    idx = random_indices(3, 3, 4, 4)
    want_p, want_l = orc.index_to_patch_dense(idx, SPLITS, 4, 1)
    got_p, got_l = _C.grained_sample_index_to_patch_dense(_t(idx, dev), _t(np.array(SPLITS, dtype=np.int64), dev), 4, 1)
    assert np.array_equal(got_p.cpu().numpy(), want_p) and np.array_equal(got_l.numpy(), want_l)


# ------------------------------------------------------------------ compress / decompress
GEOMS = [(8, 16, 16, 1, 192), (2, 32, 32, 1, 384), (3, 8, 12, 0, 64), (2, 16, 16, 2, 768)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,W,extra,C", GEOMS)
def test_compress_bit_exact(dev, dtype, B, H, W, extra, C):
    from vtpack_amd import _C
    idx = random_indices(B + C, B, H // 4, W // 4)
    patches, _ = orc.index_to_patch(idx, SPLITS, 4, extra)
    x = randn(C + 1, B, extra + H * W, C)
    if dtype == torch.bfloat16:
        x = bf16_round(x)
    want = orc.compress(x, patches, H, W, extra)
    got = _C.grained_sample_compress(_t(x, dev, dtype), _t(patches, dev), H, W, extra)
    assert got.dtype == dtype and tuple(got.shape) == want.shape
    want_t = torch.from_numpy(want).to(dtype)       # one round-to-nearest-even on store
    assert torch.equal(got.cpu(), want_t), f"max diff {rel_err(got.float(), want_t.float()):.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("with_counts", [False, True])
@pytest.mark.parametrize("B,H,W,extra,C,p", [(8, 16, 16, 1, 384, None), (2, 32, 32, 1, 384, None), (3, 8, 12, 0, 264, None),
                                              (2, 16, 16, 2, 512, None), (300, 16, 16, 1, 384, [.6, .3, .1]),
                                              (5, 4, 4, 1, 384, [0, 0, 1]), (4, 16, 16, 1, 384, [1, 0, 0]),
                                              (64, 32, 32, 1, 384, [.2, .3, .5])])
def test_compress_regions_bit_exact(dev, dtype, with_counts, B, H, W, extra, C, p):
    """index->patch and compress as one kernel that works by region: the packed rows, descriptors, offsets and lengths
    are those of the two operators (the oracle's), bit for bit, whether the rows before a region are added up from the
    per-region count bytes or from the gate indices; the bytes themselves are checked where they come from (the
    scatter-back that routes the next block)."""
    from vtpack_amd import ops
    if dtype == torch.float32:
        C = C // 2                          # the same 16-byte vectors per row
    idx = random_indices(B + C, B, H // 4, W // 4, p=p)
    patches, lengths = orc.index_to_patch(idx, SPLITS, 4, extra)
    x = randn(C + 1, B, extra + H * W, C)
    x[0, 0, :8] = -0.0                      # 0 + (-0) = +0 in a window mean, -0 stays in a copied extra token
    x[-1, -1, :8] = -0.0
    if dtype == torch.bfloat16:
        x = bf16_round(x)
    want = torch.from_numpy(orc.compress(x, patches, H, W, extra)).to(dtype)
    L = patches.shape[0]
    counts = None
    if with_counts:
        counts = ops.region_counts_buffer(B, (H // 4) * (W // 4), dev)
        counts.fill_(255)
        counts[:idx.size] = torch.from_numpy((np.array(SPLITS)[idx.reshape(-1)] ** 2).astype(np.uint8)).to(dev)
    sp = _t(np.array(SPLITS, dtype=np.int64), dev)
    assert ops.fits_compress_regions(_t(x, dev, dtype), H, W, 4, SPLITS)
    comp, rec, got_p, offsets, got_l = ops.compress_regions(_t(x, dev, dtype), _t(idx, dev), sp, H, W, 4, counts=counts)
    assert rec is None and comp.dtype == dtype
    assert torch.equal(got_l.cpu(), torch.from_numpy(lengths))
    assert torch.equal(offsets.cpu(), torch.from_numpy(np.concatenate([[0], np.cumsum(lengths)])))
    got_p, want_p = got_p[:L].cpu().numpy(), patches.copy()
    ext = want_p[:, 1] < 0                  # column 2 of an extra token's row is unwritten in the reference: 0 here
    assert np.array_equal(got_p[:, [0, 1, 3]], want_p[:, [0, 1, 3]]) and np.array_equal(got_p[~ext, 2], want_p[~ext, 2])
    assert bool((got_p[ext, 2] == 0).all())
    assert torch.equal(comp[:L].cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       want.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    # and the two-kernel path of this library
    p2, o2, l2 = ops.index_to_patch(_t(idx, dev), sp, 4, extra, capacity=B * (extra + H * W))
    c2 = ops.compress(_t(x, dev, dtype), p2, W, extra, rows_dev=o2[B:], rows=B * (extra + H * W))
    assert torch.equal(c2[:L], comp[:L]) and torch.equal(p2[:L], torch.from_numpy(got_p).to(dev))


@pytest.mark.parametrize("B,H,W,extra,C", [(8, 16, 16, 1, 384), (2, 32, 32, 2, 512), (3, 8, 12, 0, 264)])
def test_compress_regions_records(dev, B, H, W, extra, C):
    """The statistics records of the packed rows as stored, for the q Linear with norm1 folded in."""
    from vtpack_amd import ops
    idx = random_indices(B, B, H // 4, W // 4)
    g = torch.Generator().manual_seed(C)
    x = (torch.randn(B, extra + H * W, C, generator=g) * 2 + 5 * torch.randn(B, extra + H * W, 1, generator=g))
    x = x.bfloat16().to(dev)
    sp = _t(np.array(SPLITS, dtype=np.int64), dev)
    plain = ops.compress_regions(x, _t(idx, dev), sp, H, W, 4)
    comp, rec, patches, offsets, lengths = ops.compress_regions(x, _t(idx, dev), sp, H, W, 4, stats_eps=1e-6)
    L = int(offsets[-1])
    assert torch.equal(comp[:L], plain[0][:L]) and torch.equal(patches[:L], plain[2][:L])
    r = rec[:L].float()
    mean, sigma = r[:, 0] + r[:, 2] + r[:, 5], r[:, 6] + r[:, 7]
    cd = comp[:L].double()
    m_ref, s_ref = cd.mean(1), (cd.var(1, unbiased=False) + 1e-6).sqrt()
    assert bool((r[:, 0] == r[:, 1]).all() and (r[:, 0] == r[:, 3]).all() and (r[:, 2] == r[:, 4]).all())
    assert bool((r[:, 6] == r[:, 8]).all() and (r[:, 7] == r[:, 9]).all() and (r[:, 10:] == 0).all())
    assert float((mean.double() - m_ref).abs().max()) < 5e-6 * float(cd.abs().max())
    assert float(((sigma.double() - s_ref) / s_ref).abs().max()) < 3e-5


def test_compress_regions_refuses_what_it_cannot_do(dev):
    from vtpack_amd import ops
    from vtpack_amd._lib import VtdgeError
    x = torch.zeros(2, 65, 768, dtype=torch.bfloat16, device=dev)         # 96 vectors per row
    idx = torch.zeros(2, 2, 2, dtype=torch.int64, device=dev)
    sp = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    assert not ops.fits_compress_regions(x, 8, 8, 4, SPLITS)
    assert not ops.fits_compress_regions(x[..., :384], 8, 8, 2, [2, 1])
    assert not ops.fits_compress_regions(x[..., :64].contiguous(), 8, 8, 4, SPLITS)      # narrow rows: row-wise kernels
    with pytest.raises(VtdgeError):
        ops.compress_regions(x, idx, sp, 8, 8, 4)
    with pytest.raises(TypeError):
        ops.compress_regions(x[..., :384].float().contiguous(), idx, sp, 8, 8, 4, stats_eps=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("add_ref", [True, False])
@pytest.mark.parametrize("B,H,W,extra,C", GEOMS)
def test_decompress_bit_exact(dev, dtype, add_ref, B, H, W, extra, C):
    from vtpack_amd import _C
    idx = random_indices(B + C + 5, B, H // 4, W // 4)
    patches, _ = orc.index_to_patch(idx, SPLITS, 4, extra)
    d = randn(C + 2, patches.shape[0], C)
    ref = randn(C + 3, B, extra + H * W, C)
    if dtype == torch.bfloat16:
        d, ref = bf16_round(d), bf16_round(ref)
    want = torch.from_numpy(orc.decompress(d, patches, ref, H, W, extra, add_ref)).to(dtype)
    got = _C.grained_sample_decompress(_t(d, dev, dtype), _t(patches, dev), _t(ref, dev, dtype), H, W, extra, add_ref)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decompress_fused_subtract(dev, dtype):
    """out = (q - comp) + ref in one kernel == DynamicGrainedEncoder.decompress (dge.py:88 + scatter)."""
    from vtpack_amd import ops
    B, H, W, extra, C = 4, 16, 16, 1, 192
    idx = random_indices(11, B, 4, 4)
    patches, _ = orc.index_to_patch(idx, SPLITS, 4, extra)
    q, comp = randn(1, patches.shape[0], C), randn(2, patches.shape[0], C)
    ref = randn(3, B, extra + H * W, C)
    if dtype == torch.bfloat16:
        q, comp, ref = bf16_round(q), bf16_round(comp), bf16_round(ref)
    delta = torch.from_numpy(q - comp).to(dtype).float().numpy()      # the reference rounds the difference
    want = torch.from_numpy(orc.decompress(delta, patches, ref, H, W, extra, True)).to(dtype)
    got = ops.decompress(_t(q, dev, dtype), _t(patches, dev), _t(ref, dev, dtype), W, extra, add_ref=True,
                         sub=_t(comp, dev, dtype))
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,W,extra,C", [(4, 16, 16, 1, 192), (2, 32, 32, 1, 384), (3, 8, 12, 0, 64), (2, 8, 8, 2, 256)])
def test_decompress_with_layernorm(dev, dtype, B, H, W, extra, C):
    """The scatter-back that also writes the next block's first LayerNorm: `out` is bit for bit the plain
    scatter-back, and the second output is LayerNorm of `out` as stored."""
    from vtpack_amd import ops
    if C * (2 if dtype == torch.bfloat16 else 4) > 1024:
        pytest.skip("rows longer than 64 vectors go through the separate kernels")
    idx = random_indices(B + C + 1, B, H // 4, W // 4)
    patches, _ = orc.index_to_patch(idx, SPLITS, 4, extra)
    q, comp = randn(C + 4, patches.shape[0], C), randn(C + 5, patches.shape[0], C)
    ref = randn(C + 6, B, extra + H * W, C)
    w, b = randn(C + 7, C) * 0.2 + 1, randn(C + 8, C) * 0.1
    if dtype == torch.bfloat16:
        q, comp, ref, w, b = bf16_round(q), bf16_round(comp), bf16_round(ref), bf16_round(w), bf16_round(b)
    delta = torch.from_numpy(q - comp).to(dtype).float().numpy()
    want = torch.from_numpy(orc.decompress(delta, patches, ref, H, W, extra, True)).to(dtype)
    want_ln = torch.nn.functional.layer_norm(want.float(), (C,), torch.from_numpy(w), torch.from_numpy(b), 1e-6)
    got, got_ln = ops.decompress_layernorm(_t(q, dev, dtype), _t(patches, dev), _t(ref, dev, dtype), W, extra,
                                           _t(w, dev, dtype), _t(b, dev, dtype), 1e-6, sub=_t(comp, dev, dtype))
    assert torch.equal(got.cpu(), want)
    assert_close(got_ln.float(), want_ln, dtype, "decompress + layernorm")
    # the separate LayerNorm kernel on the same tokens gives the same numbers
    sep = ops.layernorm(got, _t(w, dev, dtype), _t(b, dev, dtype), 1e-6)
    assert abs_err(got_ln, sep) <= (1e-6 if dtype == torch.float32 else 2 ** -6)


def test_decompress_with_layernorm_refuses_long_rows(dev):
    from vtpack_amd import ops
    from vtpack_amd._lib import VtdgeError
    B, H, W, C = 1, 4, 4, 1024
    patches, _ = orc.index_to_patch(np.zeros((B, 1, 1), dtype=np.int64), SPLITS, 4, 0)
    z = torch.zeros(patches.shape[0], C, device=dev, dtype=torch.bfloat16)
    ref = torch.zeros(B, H * W, C, device=dev, dtype=torch.bfloat16)
    g = torch.ones(C, device=dev, dtype=torch.bfloat16)
    assert not ops.fits_decompress_layernorm(ref)
    with pytest.raises(VtdgeError):
        ops.decompress_layernorm(z, _t(patches, dev), ref, W, 0, g, g, 1e-6)


def test_device_side_row_count(dev):
    """Packed kernels stop at the row count held in device memory, not at the buffer capacity."""
    from vtpack_amd import ops
    B, H, W, extra, C = 4, 16, 16, 1, 192
    idx = random_indices(5, B, 4, 4)
    want_p, want_l = orc.index_to_patch(idx, SPLITS, 4, extra)
    cap = B * (extra + H * W)
    patches, offsets, lengths = ops.index_to_patch(_t(idx, dev), _t(np.array(SPLITS, dtype=np.int64), dev), 4, extra,
                                                   capacity=cap)
    L = int(want_l.sum())
    assert np.array_equal(offsets.cpu().numpy(), np.concatenate([[0], np.cumsum(want_l)]))
    assert np.array_equal(patches[:L].cpu().numpy(), want_p)
    x = randn(9, B, extra + H * W, C)
    sentinel = 12345.0
    out = torch.full((cap, C), sentinel, device=dev)
    from vtpack_amd._lib import call, ptr, stream_ptr, F32
    call("vtdge_compress", ptr(_t(x, dev)), ptr(patches), ptr(offsets[B:]), cap, ptr(out), 0, 0, 0, 0.0, B,
         extra + H * W, C, W, extra, F32, stream_ptr())
    assert torch.equal(out[:L].cpu(), torch.from_numpy(orc.compress(x, want_p, H, W, extra)))
    assert bool((out[L:] == sentinel).all())


# ------------------------------------------------------------------ router
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,W,extra,C", [(8, 16, 16, 1, 192), (4, 32, 32, 1, 384), (3, 8, 12, 0, 64)])
def test_router_gate_and_indices(dev, dtype, B, H, W, extra, C):
    from vtpack_amd import ops
    x = randn(21, B, extra + H * W, C)
    w = randn(22, 3, C) * 0.3
    b = randn(23, 3) * 0.1
    if dtype == torch.bfloat16:
        x, w, b = bf16_round(x), bf16_round(w), bf16_round(b)
    want = torch_ref.router_gate(torch.from_numpy(x), H, W, torch.from_numpy(w), torch.from_numpy(b), 4)
    gate, indices = ops.router(_t(x, dev, dtype), _t(w, dev, dtype), _t(b, dev, dtype), H, W, 4)
    assert_close(gate.float(), want, dtype, "gate logits")
    # gate choices must be identical wherever the decision is not a numerical tie of the oracle's own logits
    top2 = want.topk(2, dim=-1).values
    margin = (top2[..., 0] - top2[..., 1])
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    decided = margin > tol
    assert decided.float().mean() > 0.9
    assert torch.equal(indices.cpu()[decided], want.argmax(-1)[decided])
    # and the kernel's indices are exactly the argmax of the kernel's own (rounded) logits, lowest index on ties
    assert torch.equal(indices.cpu(), gate.float().cpu().argmax(-1))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,W,extra,C,R", [(8, 16, 16, 1, 192, 4), (3, 8, 12, 0, 64, 4), (5, 16, 16, 2, 384, 4),
                                             (2, 32, 32, 1, 384, 4), (4, 8, 8, 1, 128, 2), (2, 4, 4, 1, 512, 4),
                                             (3, 4, 8, 0, 256, 2)])
def test_router_with_layernorm(dev, dtype, B, H, W, extra, C, R):
    """One pass over x gives the router's outputs and LayerNorm of every token: bit for bit what the two separate
    kernels give, and the LayerNorm within tolerance of the library routine."""
    from vtpack_amd import ops
    if dtype == torch.float32 and C > 256:
        pytest.skip("one 16-byte vector per lane and row: at most 256 fp32 channels")
    x = randn(121, B, extra + H * W, C) * 1.5 + 0.3
    w, b = randn(122, 3, C) * 0.3, randn(123, 3) * 0.1
    lw, lb = randn(124, C) * 0.2 + 1, randn(125, C) * 0.1
    if dtype == torch.bfloat16:
        x, w, b, lw, lb = (bf16_round(t) for t in (x, w, b, lw, lb))
    xd, wd, bd, lwd, lbd = (_t(t, dev, dtype) for t in (x, w, b, lw, lb))
    assert ops.fits_router_layernorm(xd, R)
    gate, indices, x_ln = ops.router_layernorm(xd, wd, bd, H, W, R, lwd, lbd, 1e-6)
    gate0, indices0 = ops.router(xd, wd, bd, H, W, R)
    assert torch.equal(gate, gate0) and torch.equal(indices, indices0)
    assert torch.equal(x_ln, ops.layernorm(xd, lwd, lbd, 1e-6))
    want = torch.nn.functional.layer_norm(torch.from_numpy(x), (C,), torch.from_numpy(lw), torch.from_numpy(lb), 1e-6)
    assert_close(x_ln.float(), want, dtype, "router + layernorm")


def test_router_with_layernorm_refuses_what_it_cannot_do(dev):
    from vtpack_amd import ops
    from vtpack_amd._lib import VtdgeError
    x = torch.zeros(2, 1 + 64, 768, device=dev, dtype=torch.bfloat16)
    w, b = torch.zeros(3, 768, device=dev, dtype=torch.bfloat16), torch.zeros(3, device=dev, dtype=torch.bfloat16)
    lw = torch.ones(768, device=dev, dtype=torch.bfloat16)
    assert not ops.fits_router_layernorm(x, 4)
    with pytest.raises(VtdgeError):
        ops.router_layernorm(x, w, b, 8, 8, 4, lw, lw, 1e-6)
    x = torch.zeros(2, 1 + 64, 384, device=dev, dtype=torch.bfloat16)
    assert not ops.fits_router_layernorm(x, 8)
    with pytest.raises(VtdgeError):
        ops.router_layernorm(x, w[:, :384].contiguous(), b, 8, 8, 8, lw[:384].contiguous(), lw[:384].contiguous(), 1e-6)


# ------------------------------------------------------------------ layernorm / linear
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,C", [(1, 192), (257, 384), (1000, 768), (33, 64)])
def test_layernorm(dev, dtype, rows, C):
    from vtpack_amd import ops
    x, w, b = randn(31, rows, C) * 2 + 0.5, randn(32, C) * 0.2 + 1, randn(33, C) * 0.1
    if dtype == torch.bfloat16:
        x, w, b = bf16_round(x), bf16_round(w), bf16_round(b)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x), (C,), torch.from_numpy(w), torch.from_numpy(b), 1e-6)
    got = ops.layernorm(_t(x, dev, dtype), _t(w, dev, dtype), _t(b, dev, dtype), 1e-6)
    assert_close(got.float(), want, dtype, "layernorm")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,period,C", [(4096, 1024, 64), (1537, 29, 384), (640, 64, 512), (300, 300, 768)])
def test_layernorm_with_rows_added(dev, dtype, rows, period, C):
    """LayerNorm followed by `+ pos_embed` in one pass: bit for bit the LayerNorm kernel's result plus the addend
    (rounded in between as the two modules would round), for row counts that are and are not multiples of the period."""
    from vtpack_amd import ops
    g = torch.Generator().manual_seed(rows + C)
    x = (torch.randn(rows, C, generator=g) * 2 + 1).to(dtype).to(dev)
    w = (1 + 0.2 * torch.randn(C, generator=g)).to(dtype).to(dev)
    b = (0.1 * torch.randn(C, generator=g)).to(dtype).to(dev)
    pos = torch.randn(1, period, C, generator=g).to(dtype).to(dev)
    want = ops.layernorm(x, w, b, 1e-6)
    want = want + pos[0][torch.arange(rows, device=dev) % period]
    got = ops.layernorm(x, w, b, 1e-6, add=pos)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,N,C,count", [(256, 257, 384, 1), (5, 66, 192, 2), (3, 17, 768, 17), (9, 10, 64, 3)])
def test_layernorm_of_the_front_rows(dev, dtype, B, N, C, count):
    """The final norm on the class-token rows only, read in place: the same bits as LayerNorm of a copy of the slice."""
    from vtpack_amd import ops
    x = _t(randn(131, B, N, C) * 1.5 + 0.3, dev, dtype)
    w, b = _t(randn(132, C) * 0.2 + 1, dev, dtype), _t(randn(133, C) * 0.1, dev, dtype)
    got = ops.layernorm_front_rows(x, count, w, b, 1e-6)
    assert got.shape == (B, count, C)
    assert torch.equal(got, ops.layernorm(x[:, :count, :].contiguous(), w, b, 1e-6))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 192, 192), (904, 576, 192), (257, 384, 384), (1000, 1536, 384),
                                     (300, 384, 1536), (129, 1000, 192), (64, 72, 40)])
@pytest.mark.parametrize("epi", ["plain", "bias", "bias_gelu", "bias_res"])
def test_linear(dev, dtype, M, N, K, epi):
    from vtpack_amd import ops
    a, w = randn(41, M, K), randn(42, N, K) * 0.02   # the isolated-GEMM config: A ~ N(0,1), W ~ N(0,0.02)
    bias, res = randn(43, N) * 0.1, randn(44, M, N)
    if dtype == torch.bfloat16:
        a, w, bias, res = bf16_round(a), bf16_round(w), bf16_round(bias), bf16_round(res)
    want = torch.from_numpy(a).double() @ torch.from_numpy(w).double().T
    if epi != "plain":
        want = want + torch.from_numpy(bias).double()
    if epi == "bias_gelu":
        want = torch.nn.functional.gelu(want)
    if epi == "bias_res":
        want = want + torch.from_numpy(res).double()
    got = ops.linear(_t(a, dev, dtype), _t(w, dev, dtype), None if epi == "plain" else _t(bias, dev, dtype),
                     _t(res, dev, dtype) if epi == "bias_res" else None, act="gelu" if epi == "bias_gelu" else "none")
    assert_close(got.float(), want, dtype, f"linear {epi}")


def test_linear_device_rows(dev):
    from vtpack_amd import ops
    M, N, K, live = 700, 384, 192, 333
    a, w = randn(51, M, K), randn(52, N, K) * 0.05
    rows_dev = torch.tensor([live], dtype=torch.int64, device=dev)
    out = torch.full((M, N), 7.0, device=dev)
    ops.linear(_t(a, dev), _t(w, dev), rows_dev=rows_dev, out=out)
    want = torch.from_numpy(a[:live]).double() @ torch.from_numpy(w).double().T
    assert rel_err(out[:live], want) <= 1e-5
    assert bool((out[live:] == 7.0).all())


# The packed Linear of the C = 384 models in bf16 (K = 384, N a multiple of 384, >= 2048 rows) runs on the
# weight-stationary kernel: ragged last tiles, fewer tiles than workgroups, several column groups, every epilogue,
# live row count on the device.
@pytest.mark.parametrize("M,N", [(2048, 384), (2049, 768), (4127, 384), (9000, 1152), (33000, 1536), (70000, 768)])
@pytest.mark.parametrize("epi", ["plain", "bias", "bias_gelu", "bias_res", "gelu_res", "bias_gelu_res"])
def test_linear_weight_stationary(dev, M, N, epi):
    from vtpack_amd import ops
    if M > 40000 and epi not in ("bias", "bias_res"):
        pytest.skip("largest shape: the two epilogues of the model are enough")
    K = 384
    g = torch.Generator().manual_seed(M + N)
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    bias = (torch.randn(N, generator=g) * 0.5).bfloat16()
    res = torch.randn(M, N, generator=g).bfloat16()
    want = a.double() @ w.double().T
    if "bias" in epi:
        want = want + bias.double()
    if "gelu" in epi:
        want = torch.nn.functional.gelu(want)
    if "res" in epi:
        want = want + res.double()
    got = ops.linear(a.to(dev), w.to(dev), bias.to(dev) if "bias" in epi else None,
                     res.to(dev) if "res" in epi else None, act="gelu" if "gelu" in epi else "none")
    # one bf16 rounding of a value of magnitude up to ~8: half an ulp is 2^-6; the bar of the other bf16 tests
    # (2e-2) is kept on everything below 4
    err = (got.double().cpu() - want).abs()
    small = want.abs() < 4
    assert float(err[small].max()) <= BF16_ABS, f"weight-stationary linear {epi}: {float(err[small].max()):.3e}"
    assert float((err / want.abs().clamp_min(4)).max()) <= 2 ** -7, f"weight-stationary linear {epi} (relative)"


@pytest.mark.parametrize("N", [384, 1152, 1536])
def test_linear_on_skewed_segments(dev, N):
    """The isolated grouped GEMM of the benchmark (bf16, K = 384, 256 samples whose query counts follow a seeded
    skewed gate mix with a heavy tail, clipped to [16, 256]; A ~ N(0, 1), W ~ N(0, 0.02)): the packed rows of all
    segments against one shared weight, checked against fp64 on every row, with the live row count on the device."""
    from vtpack_amd import ops
    r = np.random.RandomState(0)
    p_fine = np.clip(r.beta(0.6, 2.0, size=256), 0, 1)
    lengths = np.clip(np.array([1 + int(r.choice([16, 4, 1], size=16, p=[pf, (1 - pf) * 0.4, (1 - pf) * 0.6]).sum())
                                for pf in p_fine]), 16, 256)
    L, K = int(lengths.sum()), 384
    assert L == 21911                                    # the benchmark's segments
    g = torch.Generator().manual_seed(0)
    a = torch.randn((L, K), generator=g).bfloat16().to(dev)
    w = (torch.randn((N, K), generator=g) * 0.02).bfloat16().to(dev)
    bias = (torch.randn(N, generator=g) * 0.02).bfloat16().to(dev)
    cap = torch.zeros((L + 4096, K), dtype=torch.bfloat16, device=dev)
    cap[:L] = a
    out = ops.linear(cap, w, bias, rows_dev=torch.tensor([L], dtype=torch.int64, device=dev))
    want = a.double() @ w.double().T + bias.double()
    assert abs_err(out[:L], want) <= BF16_ABS
    # segment boundaries mean nothing to a Linear with shared weights: any one segment alone gives the same rows
    off = np.concatenate([[0], np.cumsum(lengths)])
    big = int(lengths.argmax())
    alone = ops.linear(a[off[big]:off[big + 1]].contiguous(), w, bias)
    assert abs_err(alone, want[off[big]:off[big + 1]]) <= BF16_ABS


def test_linear_weight_stationary_device_rows(dev):
    from vtpack_amd import ops
    M, N, K, live = 6000, 768, 384, 4999
    g = torch.Generator().manual_seed(7)
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    res = torch.randn(M, N, generator=g).bfloat16()
    rows_dev = torch.tensor([live], dtype=torch.int64, device=dev)
    out = torch.full((M, N), 7.0, device=dev, dtype=torch.bfloat16)
    ops.linear(a.to(dev), w.to(dev), residual=res.to(dev), rows_dev=rows_dev, out=out)
    want = a[:live].double() @ w.double().T + res[:live].double()
    assert abs_err(out[:live], want) <= 4 * BF16_ABS        # values up to ~10: one bf16 rounding
    assert bool((out[live:] == 7.0).all())
    # a live count of zero touches nothing
    out.fill_(7.0)
    ops.linear(a.to(dev), w.to(dev), rows_dev=torch.zeros(1, dtype=torch.int64, device=dev), out=out)
    assert bool((out == 7.0).all())


def test_linear_weight_stationary_matches_streaming_kernel(dev):
    """Both bf16 kernels accumulate the K dimension in the same order in fp32 and differ only in how the bias
    reaches the sum (an extra K step of the MFMA against a vector addition), so their bf16 results agree except for
    an occasional last bit; fewer than 2048 rows send the same rows to the streaming kernel."""
    from vtpack_amd import ops
    M, N, K = 5003, 768, 384
    g = torch.Generator().manual_seed(11)
    a = torch.randn(M, K, generator=g).bfloat16().to(dev)
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(dev)
    bias = torch.randn(N, generator=g).bfloat16().to(dev)
    for act in ("none", "gelu"):
        got = ops.linear(a, w, bias, act=act)[:2000].float()
        few = ops.linear(a[:2000], w, bias, act=act).float()          # < 2048 rows: streaming kernel
        diff = (got - few).abs()
        assert float((diff / few.abs().clamp_min(2.0 ** -10)).max()) <= 2.0 ** -7      # at most one bf16 ulp
        assert float((diff > 0).float().mean()) < 0.01
    # without a bias the two are the same sum, bit for bit
    assert torch.equal(ops.linear(a, w)[:2000], ops.linear(a[:2000], w))


# The K-split weight-stationary kernel: bf16, K = 1536, N a multiple of 96, 2048 rows or more, no activation.
@pytest.mark.parametrize("M,N", [(2048, 384), (2053, 96), (4127, 384), (9001, 768), (33000, 384), (3000, 192)])
@pytest.mark.parametrize("epi", ["plain", "bias", "res", "bias_res"])
def test_linear_k_split(dev, M, N, epi):
    from vtpack_amd import ops
    K = 1536
    g = torch.Generator().manual_seed(3 * M + N)
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.03).bfloat16()
    bias = (torch.randn(N, generator=g) * 0.5).bfloat16()
    res = torch.randn(M, N, generator=g).bfloat16()
    want = a.double() @ w.double().T
    if "bias" in epi:
        want = want + bias.double()
    if "res" in epi:
        want = want + res.double()
    got = ops.linear(a.to(dev), w.to(dev), bias.to(dev) if "bias" in epi else None,
                     res.to(dev) if "res" in epi else None)
    err = (got.double().cpu() - want).abs()
    small = want.abs() < 4
    assert float(err[small].max()) <= BF16_ABS, f"k-split linear {epi}: {float(err[small].max()):.3e}"
    assert float((err / want.abs().clamp_min(4)).max()) <= 2 ** -7, f"k-split linear {epi} (relative)"


@pytest.mark.parametrize("live", [0, 1, 7, 15, 16, 17, 33, 1000, 4999])
def test_linear_k_split_device_rows(dev, live):
    """The live row count comes from device memory: any count, down to a lone short tile, and nothing past it is
    written."""
    from vtpack_amd import ops
    M, N, K = 6000, 384, 1536
    g = torch.Generator().manual_seed(17)
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.03).bfloat16()
    bias = torch.randn(N, generator=g).bfloat16()
    res = torch.randn(M, N, generator=g).bfloat16()
    rows_dev = torch.tensor([live], dtype=torch.int64, device=dev)
    out = torch.full((M, N), 7.0, device=dev, dtype=torch.bfloat16)
    ops.linear(a.to(dev), w.to(dev), bias.to(dev), residual=res.to(dev), rows_dev=rows_dev, out=out)
    if live:
        want = a[:live].double() @ w.double().T + bias.double() + res[:live].double()
        assert abs_err(out[:live], want) <= 4 * BF16_ABS        # values up to ~10: one bf16 rounding
    assert bool((out[live:] == 7.0).all())


def test_linear_k_split_strided_and_repeatable(dev):
    """Operands as column slices of wider buffers (row strides larger than the widths), and the same bytes on every
    call: the four partial sums of a tile are added in a fixed order."""
    from vtpack_amd import ops
    M, N, K = 5003, 384, 1536
    g = torch.Generator().manual_seed(23)
    abuf = torch.randn(M, K + 64, generator=g).bfloat16().to(dev)
    rbuf = torch.randn(M, N + 32, generator=g).bfloat16().to(dev)
    obuf = torch.full((M, N + 8), 7.0, dtype=torch.bfloat16, device=dev)
    w = (torch.randn(N, K, generator=g) * 0.03).bfloat16().to(dev)
    bias = torch.randn(N, generator=g).bfloat16().to(dev)
    a, res, out = abuf[:, 32:32 + K], rbuf[:, 16:16 + N], obuf[:, 4:4 + N]
    ops.linear(a, w, bias, residual=res, out=out)
    want = a.double() @ w.double().T + bias.double() + res.double()
    assert abs_err(out, want) <= 4 * BF16_ABS
    assert bool((obuf[:, :4] == 7.0).all()) and bool((obuf[:, 4 + N:] == 7.0).all())
    first = out.clone()
    for _ in range(3):
        ops.linear(a, w, bias, residual=res, out=out)
        assert torch.equal(out, first)
    # fewer than 2048 rows go to the streaming kernel: the same sum in another order, so a last bit may differ
    few = torch.empty((2000, N), dtype=torch.bfloat16, device=dev)
    ops.linear(a[:2000], w, bias, residual=res[:2000], out=few)
    diff = (first[:2000].float() - few.float()).abs()
    assert float((diff / few.float().abs().clamp_min(2.0 ** -6)).max()) <= 2.0 ** -6


@pytest.mark.parametrize("M,N,K,epi", [(4127, 384, 384, "bias"), (9000, 1152, 384, "bias_gelu"), (2049, 768, 384, "bias_res"),
                                       (33000, 1536, 384, "plain"), (4127, 384, 1536, "bias_res"), (2053, 96, 1536, "bias"),
                                       (9001, 768, 1536, "plain")])
def test_linear_with_packed_weights(dev, M, N, K, epi):
    """The weight-stationary kernels fill their registers from W through LDS or, given a copy of W in register
    order, straight from that: the same registers either way, so the same bytes come out."""
    from vtpack_amd import ops
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(dev)
    w = (torch.randn(N, K, generator=g) * 0.04).bfloat16().to(dev)
    bias = torch.randn(N, generator=g).bfloat16().to(dev) if "bias" in epi else None
    res = torch.randn(M, N, generator=g).bfloat16().to(dev) if "res" in epi else None
    act = "gelu" if "gelu" in epi else "none"
    assert ops.PACK_WEIGHTS
    packed = ops.packed_weight(w)
    assert packed is not None and packed.numel() == N * K * 2
    assert ops.packed_weight(w) is packed                        # made once per tensor and version
    got = ops.linear(a, w, bias, res, act=act)
    ops.PACK_WEIGHTS = False
    try:
        plain = ops.linear(a, w, bias, res, act=act)
    finally:
        ops.PACK_WEIGHTS = True
    assert torch.equal(got, plain)
    # a changed weight is packed again
    w.mul_(2)
    assert ops.packed_weight(w) is not packed
    again = ops.linear(a, w, bias, res, act=act)
    ops.PACK_WEIGHTS = False
    try:
        assert torch.equal(again, ops.linear(a, w, bias, res, act=act))
    finally:
        ops.PACK_WEIGHTS = True


def test_linear_packed_weights_only_where_a_kernel_uses_them(dev):
    from vtpack_amd import ops, _lib
    for shape, dtype in (((1000, 192), torch.bfloat16), ((384, 384), torch.float32), ((100, 1536), torch.bfloat16),
                         ((3456, 384), torch.bfloat16)):
        w = torch.zeros(shape, dtype=dtype, device=dev)
        assert ops.packed_weight(w) is None
    lib = _lib.load()
    buf = torch.zeros(1000 * 192, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(1000, 192, dtype=torch.bfloat16, device=dev)
    assert lib.vtdge_linear_prepack(w.data_ptr(), 1000, 192, _lib.BF16, buf.data_ptr(), 0) == _lib.ERR_UNSUPPORTED


# ------------------------------------------------------------------ attention / sparse gemm
def _lengths(seed, B, lo, hi):
    return rng(seed).randint(lo, hi + 1, size=B).astype(np.int64)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,h,d,n,lo,hi", [(8, 3, 64, 257, 17, 257), (2, 6, 64, 1025, 65, 400), (3, 2, 32, 50, 1, 70),
                                             (4, 1, 64, 128, 128, 128), (2, 2, 64, 129, 1, 3)])
def test_sparse_attention(dev, dtype, B, h, d, n, lo, hi):
    from vtpack_amd import _C
    lengths = _lengths(61 + n, B, lo, hi)
    L = int(lengths.sum())
    q, k, v = randn(62, h, L, d), randn(63, h, B, n, d), randn(64, h, B, n, d)
    if dtype == torch.bfloat16:
        q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
    scale = d ** -0.5
    want = orc.attention(q, k, v, lengths, scale)
    got = _C.batched_sparse_attention_forward(_t(q, dev, dtype), _t(k, dev, dtype), _t(v, dev, dtype),
                                              torch.from_numpy(lengths), scale)
    assert got.shape == (h, L, d)
    assert_close(got.float(), want, dtype, "sparse attention")


@pytest.mark.parametrize("n", [257, 1025])
@pytest.mark.parametrize("shape", ["ramp", "late spike", "early spike", "steps"])
def test_sparse_attention_scores_far_above_the_first_block(dev, n, shape):
    """The softmax's reference is taken from the first 32 keys and raised on the way: scores that climb steadily
    (the reference is raised many times), a single key hundreds above all others near the end (more than fp32 can
    hold as a probability relative to the old reference) or in the first block, and plateaus that jump by 60 between
    stages of 128 keys.  Both bf16 kernels (keys resident: 257, streamed: 1025) against the oracle's max-subtracted
    softmax."""
    from vtpack_amd import _C
    B, h, d = 3, 2, 64
    lengths = np.array([130, 33, 70], dtype=np.int64)
    L = int(lengths.sum())
    q, k, v = 0.05 * randn(720, h, L, d), 0.05 * randn(721, h, B, n, d), randn(722, h, B, n, d)
    j = np.arange(n, dtype=np.float32)
    level = {"ramp": 0.25 * j, "late spike": np.where(j == n - 7, 300.0, 0.0), "early spike": np.where(j == 5, 300.0, 0.0),
             "steps": 60.0 * np.floor(j / 128)}[shape]
    q[..., 0] = 8.0                               # times scale = 1/8: a key's score is its level plus noise
    k[..., 0] = level
    q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
    scale = d ** -0.5
    want = orc.attention(q, k, v, lengths, scale)
    assert np.isfinite(want).all()
    got = _C.batched_sparse_attention_forward(_t(q, dev, torch.bfloat16), _t(k, dev, torch.bfloat16),
                                              _t(v, dev, torch.bfloat16), torch.from_numpy(lengths), scale)
    assert bool(torch.isfinite(got).all())
    assert_close(got.float(), want, torch.bfloat16, f"sparse attention, {shape} over {n} keys")


@pytest.mark.parametrize("n", [20, 32, 64, 96, 128, 160, 192, 196, 256, 257, 288])
def test_sparse_attention_resident_keys_many_items(dev, n):
    """bf16, head_dim 64, up to 288 keys: the kernel that keeps an item's keys and values in LDS, with more
    (sample, head) items than compute units, so that every workgroup walks several items (double buffer, the next
    item's keys / values and first query tile fetched under the current item's arithmetic, the item table in LDS).
    One case per number of 32-key blocks (1 .. 9), with and without a partial last block; query counts mix empty
    samples, single queries, counts around the 32-query tile and the 128-query half, and samples of more than 256
    queries (a ninth tile, whose queries are loaded inside the loop)."""
    from vtpack_amd import _C
    B, h, d = 200, 3, 64
    r = rng(700 + n)
    lengths = r.choice([0, 1, 2, 31, 32, 33, 64, 100, 127, 128, 129, 200, 256, 257, 300], size=B,
                       p=[.1, .1, .08, .08, .08, .08, .08, .08, .06, .06, .06, .05, .03, .03, .03]).astype(np.int64)
    lengths[:4] = [300, 0, 257, 1]
    L = int(lengths.sum())
    q, k, v = bf16_round(randn(701, h, L, d)), bf16_round(randn(702, h, B, n, d)), bf16_round(randn(703, h, B, n, d))
    scale = d ** -0.5
    want = orc.attention(q, k, v, lengths, scale)
    got = _C.batched_sparse_attention_forward(_t(q, dev, torch.bfloat16), _t(k, dev, torch.bfloat16),
                                              _t(v, dev, torch.bfloat16), torch.from_numpy(lengths), scale)
    assert got.shape == (h, L, d)
    assert_close(got.float(), want, torch.bfloat16, f"sparse attention, {B * h} items of {n} keys")


def test_sparse_attention_more_items_than_the_item_table_holds(dev):
    """More than 512 items per workgroup (here 132 000 items of 8 keys): the first row and query count of an item
    are then read from `offsets` inside the loop instead of from the table in LDS."""
    from vtpack_amd import _C
    B, h, d, n = 22000, 6, 64, 8
    r = rng(710)
    lengths = r.choice([0, 1, 2, 3, 40], size=B, p=[.3, .4, .2, .09, .01]).astype(np.int64)
    L = int(lengths.sum())
    fast = np.random.default_rng(711)             # 135 M values: the legacy generator would take 12 s over them
    q, k, v = (bf16_round(fast.standard_normal(shape, dtype=np.float32)) for shape in ((h, L, d), (h, B, n, d), (h, B, n, d)))
    scale = d ** -0.5
    want = orc.attention(q, k, v, lengths, scale)
    got = _C.batched_sparse_attention_forward(_t(q, dev, torch.bfloat16), _t(k, dev, torch.bfloat16),
                                              _t(v, dev, torch.bfloat16), torch.from_numpy(lengths), scale)
    assert_close(got.float(), want, torch.bfloat16, "sparse attention, 132 000 items")


@pytest.mark.parametrize("dtype", DTYPES)
def test_sparse_attention_strided_kv(dev, dtype):
    """q straight from the q Linear ([L, h*d]) and k, v as views of the kv Linear output ([B, n, 2, h, d])."""
    from vtpack_amd import ops
    B, h, d, n = 4, 3, 64, 257
    C = h * d
    lengths = _lengths(71, B, 17, 257)
    L = int(lengths.sum())
    q, kv = randn(72, L, C), randn(73, B, n, 2 * C)
    if dtype == torch.bfloat16:
        q, kv = bf16_round(q), bf16_round(kv)
    qh = q.reshape(L, h, d).transpose(1, 0, 2)
    kvh = kv.reshape(B, n, 2, h, d).transpose(2, 3, 0, 1, 4)
    want = orc.attention(qh, kvh[0], kvh[1], lengths, d ** -0.5).transpose(1, 0, 2).reshape(L, C)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(lengths)])).to(dev)
    kvt = _t(kv, dev, dtype)
    got = ops.sparse_attention(_t(q, dev, dtype), kvt[:, :, :C], kvt[:, :, C:], off, d ** -0.5, h, int(lengths.max()))
    assert_close(got.float(), want, dtype, "strided sparse attention")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
def test_batched_sparse_gemm(dev, dtype, ta, tb):
    from vtpack_amd import _C
    B, h, d, n = 5, 3, 64, 70
    la = _lengths(81, B, 3, 90)
    if not ta and tb:        # Q K^T: a [h,La,d], b [h,B*n,d]
        lb = np.full(B, n, dtype=np.int64)
        a, b = randn(82, h, int(la.sum()), d), randn(83, h, int(lb.sum()), d)
    elif not ta and not tb:  # P V: a [h,La,n], b [h,B*n,d]
        lb = np.full(B, n, dtype=np.int64)
        a, b = randn(82, h, int(la.sum()), n), randn(83, h, int(lb.sum()), d)
    elif ta and not tb:      # A^T B: a [h,La,ka], b [h,La,kb]
        lb = la.copy()
        a, b = randn(82, h, int(la.sum()), 48), randn(83, h, int(lb.sum()), d)
    else:                    # A^T B^T: a [h,La,ka] -> [ka,la]; b [h,Lb,kb] with kb == la, so equal lengths
        la = np.full(B, 40, dtype=np.int64)
        lb = np.full(B, 24, dtype=np.int64)
        a, b = randn(82, h, int(la.sum()), 48), randn(83, h, int(lb.sum()), 40)
    if dtype == torch.bfloat16:
        a, b = bf16_round(a), bf16_round(b)
    want = orc.sparse_gemm(a, b, la, lb, ta, tb)
    for fn in (_C.batched_sparse_gemm_forward, _C.batched_sparse_gemm_v2_forward):
        got = fn(_t(a, dev, dtype), _t(b, dev, dtype), torch.from_numpy(la), torch.from_numpy(lb), ta, tb)
        assert tuple(got.shape) == want.shape
        if dtype == torch.float32:
            assert rel_err(got, want) <= 1e-5
        else:
            # bf16 output of sums of ~64 products of N(0,1) values: one bf16 rounding of |x| <~ 40
            assert rel_err(got.float(), want) <= 2 ** -8


@pytest.mark.parametrize("dtype", DTYPES)
def test_batched_sparse_gemm_tile_edges_and_empty_samples(dev, dtype):
    """Q K^T and P V with sample lengths around the 64-row tile (0, 1, 63, 64, 65, 129), a key count and a K extent
    that are multiples of nothing (n = 71: odd rows, a K tail in every stage), against the CPU restatement."""
    from vtpack_amd import _C
    h, d, n = 2, 40, 71
    la = np.array([0, 1, 63, 64, 65, 129, 0, 7], dtype=np.int64)
    lb = np.full(len(la), n, dtype=np.int64)
    q, k = randn(91, h, int(la.sum()), d), randn(92, h, int(lb.sum()), d)
    p, v = randn(93, h, int(la.sum()), n), randn(94, h, int(lb.sum()), d)
    if dtype == torch.bfloat16:
        q, k, p, v = bf16_round(q), bf16_round(k), bf16_round(p), bf16_round(v)
    tol = 1e-5 if dtype == torch.float32 else 2 ** -8
    got = _C.batched_sparse_gemm_forward(_t(q, dev, dtype), _t(k, dev, dtype), torch.from_numpy(la),
                                         torch.from_numpy(lb), False, True)
    assert rel_err(got.float(), orc.sparse_gemm(q, k, la, lb, False, True)) <= tol
    got = _C.batched_sparse_gemm_forward(_t(p, dev, dtype), _t(v, dev, dtype), torch.from_numpy(la),
                                         torch.from_numpy(lb), False, False)
    assert rel_err(got.float(), orc.sparse_gemm(p, v, la, lb, False, False)) <= tol
    # P^T dO (the transposed-a form of a backward pass): rows of the result are the n keys of every sample
    do = randn(95, h, int(la.sum()), d)
    if dtype == torch.bfloat16:
        do = bf16_round(do)
    got = _C.batched_sparse_gemm_forward(_t(p, dev, dtype), _t(do, dev, dtype), torch.from_numpy(la),
                                         torch.from_numpy(la), True, False)
    want = orc.sparse_gemm(p, do, la, la, True, False)
    assert tuple(got.shape) == want.shape and rel_err(got.float(), want) <= tol


def test_batched_sparse_gemm_many_samples(dev):
    """More (sample, head) pairs than a grid dimension holds (70 000): one launch, every product right."""
    from vtpack_amd import _C
    B, h, d = 35000, 2, 8
    la = (np.arange(B) % 3).astype(np.int64)                   # 0, 1 or 2 rows a sample
    lb = np.full(B, 2, dtype=np.int64)
    a, b = randn(96, h, int(la.sum()), d), randn(97, h, int(lb.sum()), d)
    got = _C.batched_sparse_gemm_forward(_t(a, dev), _t(b, dev), torch.from_numpy(la), torch.from_numpy(lb), False,
                                         True)
    assert rel_err(got, orc.sparse_gemm(a, b, la, lb, False, True)) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,Hr,Wr,C,extra", [(5, 4, 4, 384, 1), (3, 8, 8, 192, 1), (4, 3, 5, 64, 0), (2, 4, 4, 768, 2),
                                               (2, 14, 14, 64, 0), (3, 2, 2, 128, 1)])
def test_scatter_back_with_the_next_router(dev, dtype, B, Hr, Wr, C, extra):
    """The scatter-back by region that also routes the next block: the tokens, the next gate logits and the next
    gate indices equal those of the two separate operators bit for bit (which the oracle pins), for every split
    mix, width (one and several regions per wave, several vectors per lane) and count of extra tokens."""
    from vtpack_amd import ops
    H, W = 4 * Hr, 4 * Wr
    g = torch.Generator().manual_seed(B * 100 + C + extra)
    idx = torch.from_numpy(random_indices(B + C, B, Hr, Wr)).to(dev)
    splits = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    patches, offsets, lengths = ops.index_to_patch(idx, splits, 4, extra)
    L = int(offsets[-1])
    q = torch.randn(L, C, generator=g).to(dtype).to(dev)
    comp = torch.randn(L, C, generator=g).to(dtype).to(dev)
    x = torch.randn(B, extra + H * W, C, generator=g).to(dtype).to(dev)
    wgt = (torch.randn(3, C, generator=g) / C ** 0.5).to(dtype).to(dev)
    bias = (torch.randn(3, generator=g) * 0.1).to(dtype).to(dev)
    for sub in (comp, None):
        want = ops.decompress(q, patches[:L], x, W, extra, add_ref=True, sub=sub)
        want_gate, want_idx = ops.router(want, wgt, bias, H, W, 4)
        got, gate, nidx = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=sub, next_weight=wgt,
                                                next_bias=bias)
        assert torch.equal(got, want)
        assert torch.equal(nidx, want_idx) and torch.equal(gate, want_gate)
    # the query counts of the next block's regions, a byte each, for compress_regions
    got, gate, nidx, counts = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=None, next_weight=wgt,
                                                    next_bias=bias, next_splits=splits)
    assert torch.equal(nidx, want_idx) and counts.dtype == torch.uint8
    assert torch.equal(counts[:nidx.numel()].long(), (splits[nidx.reshape(-1)] ** 2))
    # a region's place handed over by compress_regions instead of added up from the gate indices
    cur = ops.region_counts_buffer(B, (H // 4) * (W // 4), dev)
    cur[:idx.numel()] = (splits[idx.reshape(-1)] ** 2).to(torch.uint8)
    per = (splits[idx.reshape(B, -1)] ** 2)
    rrows = (offsets[:B, None] + extra + per.cumsum(1) - per).reshape(-1).to(torch.int32)
    if ops.fits_compress_regions(x, H, W, 4, SPLITS):           # and that is what compress_regions leaves
        assert torch.equal(ops.compress_regions(x, idx, splits, H, W, 4, counts=cur, want_region_rows=True)[5], rrows)
    placed = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=comp, next_weight=wgt, next_bias=bias,
                                   region_rows=rrows, cur_counts=cur)
    want = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=comp, next_weight=wgt, next_bias=bias)
    assert all(torch.equal(a, b) for a, b in zip(placed, want))
    # without a next router it is the plain scatter-back
    alone, g0, i0 = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=comp)
    assert g0 is None and i0 is None
    assert torch.equal(alone, ops.decompress(q, patches[:L], x, W, extra, add_ref=True, sub=comp))


# ------------------------------------------------------------------ patch embedding
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,S,C,extra", [(3, 64, 192, 1), (2, 256, 384, 1), (2, 96, 768, 2), (5, 32, 64, 0)])
def test_patch_embed(dev, dtype, B, S, C, extra):
    """The convolution read straight from the images, bias and position embedding added in its epilogue, against
    nn.functional.conv2d in fp64; in fp32 also bit for bit against the unfolded Linear followed by the addition."""
    from vtpack_amd import ops
    P, Cin = 16, 3
    G = S // P
    g = torch.Generator().manual_seed(S + C)
    img = torch.rand(B, Cin, S, S, generator=g).to(dtype).to(dev)
    w = (torch.randn(C, Cin, P, P, generator=g) * 0.05).to(dtype).to(dev)
    b = (torch.randn(C, generator=g) * 0.1).to(dtype).to(dev)
    pos = (torch.randn(1, extra + G * G, C, generator=g) * 0.5).to(dtype).to(dev)
    assert ops.fits_patch_embed(img, w, b, pos, P)
    out = torch.full((B, extra + G * G, C), 7.0, dtype=dtype, device=dev)
    ops.patch_embed(img, w, b, pos, P, extra, out=out)
    assert bool((out[:, :extra] == 7.0).all())                       # the rows in front are not touched
    want = torch.nn.functional.conv2d(img.double(), w.double(), b.double(), stride=P).flatten(2).transpose(1, 2)
    want = want + pos.double()[:, extra:]
    err = float((out[:, extra:].double() - want).abs().max())
    assert err <= (1e-5 if dtype == torch.float32 else 2 ** -8) * float(want.abs().max())
    if dtype == torch.float32:
        patches = img.reshape(B, Cin, G, P, G, P).permute(0, 2, 4, 1, 3, 5).reshape(B * G * G, Cin * P * P)
        old = ops.linear(patches, w.reshape(C, -1), b).view(B, G * G, C) + pos[:, extra:]
        assert torch.equal(out[:, extra:], old)


def test_patch_embed_refusals(dev):
    from vtpack_amd import ops
    img = torch.zeros(2, 3, 64, 64, device=dev)
    w = torch.zeros(64, 3, 4, 4, device=dev)
    assert not ops.fits_patch_embed(img.bfloat16(), w.bfloat16(), torch.zeros(64, device=dev).bfloat16(),
                                    torch.zeros(1, 257, 64, device=dev).bfloat16(), 4)      # 8-byte patch rows
    with pytest.raises(ValueError):
        ops.patch_embed(img, torch.zeros(64, 3, 16, 16, device=dev), torch.zeros(64, device=dev),
                        torch.zeros(1, 99, 64, device=dev), 16, 1)                           # wrong table height
    with pytest.raises(TypeError):
        ops.patch_embed(img, torch.zeros(64, 3, 16, 16, device=dev).bfloat16(), torch.zeros(64, device=dev),
                        torch.zeros(1, 17, 64, device=dev), 16, 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,H,W,C,k,N", [(3, 8, 8, 64, 2, 128), (2, 16, 24, 128, 4, 128), (2, 16, 16, 64, 8, 64),
                                         (5, 14, 14, 320, 2, 512), (70, 28, 28, 128, 2, 320)])
def test_patch_linear(dev, dtype, B, H, W, C, k, N):
    """The strided convolution over a channels-last token grid read in place (vtdge_patch_linear) against
    F.conv2d in fp64 on the same (rounded) operands, and bit for bit against the Linear over a gathered copy of the
    blocks that it replaces (pvt_dge.py:62, :81-83, :164, :175)."""
    from vtpack_amd import engine, ops
    g = torch.Generator().manual_seed(H * W + C + k)
    x = torch.randn((B, H * W, C), generator=g).to(dtype)
    w4 = (torch.randn((N, C, k, k), generator=g) / (k * C ** 0.5)).to(dtype)
    b = torch.randn((N,), generator=g).to(dtype)
    wk = w4.permute(0, 2, 3, 1).reshape(N, -1).contiguous()
    xd, wd, bd = x.to(dev), wk.to(dev), b.to(dev)
    assert ops.fits_patch_linear(xd, H, W, k, wd, bd)
    got = ops.patch_linear(xd, H, W, k, wd, bd)
    want = F.conv2d(x.double().view(B, H, W, C).permute(0, 3, 1, 2), w4.double(), b.double(), stride=k)
    want = want.permute(0, 2, 3, 1).reshape(-1, N)
    assert_close(got, want, dtype, "patch_linear")
    old = ops.linear(engine.tokens_to_patches(xd, H, W, k), wd, bd)
    assert torch.equal(got, old)


def test_patch_linear_refusals(dev):
    from vtpack_amd import ops
    x = torch.zeros((2, 64, 48), device=dev, dtype=torch.bfloat16)      # 96-byte token rows: no whole 128-byte pieces
    w = torch.zeros((64, 4 * 48), device=dev, dtype=torch.bfloat16)
    b = torch.zeros((64,), device=dev, dtype=torch.bfloat16)
    assert not ops.fits_patch_linear(x, 8, 8, 2, w, b)
    with pytest.raises(ValueError):
        ops.patch_linear(x, 8, 8, 2, w, b)
    x = torch.zeros((2, 64, 64), device=dev, dtype=torch.bfloat16)
    w = torch.zeros((64, 9 * 64), device=dev, dtype=torch.bfloat16)
    assert not ops.fits_patch_linear(x, 8, 8, 3, w, b)                   # the grid is not a multiple of the block
    assert not ops.fits_patch_linear(x, 8, 8, 2, w, None)
