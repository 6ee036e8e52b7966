"""Edges of the weight-stationary Linear (bf16, K = 384, N a multiple of 384) and host-side operand checks.

The kernel is chosen from the HOST row capacity (2048 rows or more) while the live row count comes from device
memory, so any batch with B*N >= 2048 reaches it with as few live rows as the router leaves: a lone short tile
(fewer than 32 rows), exactly one tile, a last tile moved back to end at the last row, workgroups without any tile.
Inputs are scaled so that every expected value stays below 4 in magnitude: the bar is the plain 2e-2 max-abs.
"""
import pytest
import torch

from util import BF16_ABS, abs_err

pytestmark = pytest.mark.gpu

K = 384
EPILOGUES = ["plain", "bias", "bias_gelu", "bias_res", "res"]


def _operands(M, N, seed, dev):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    bias = (torch.randn(N, generator=g) * 0.3).bfloat16()
    res = (torch.randn(M, N, generator=g) * 0.5).bfloat16()
    return a, w, bias, res


def _want(a, w, bias, res, epi):
    want = a.double() @ w.double().T
    if "bias" in epi:
        want = want + bias.double()
    if "gelu" in epi:
        want = torch.nn.functional.gelu(want)
    if "res" in epi:
        want = want + res.double()
    return want


@pytest.mark.parametrize("live", [0, 1, 7, 31, 32, 33, 63, 65, 2047, 2500])
@pytest.mark.parametrize("epi", EPILOGUES)
@pytest.mark.parametrize("packed", [True, False])
def test_weight_stationary_live_rows(dev, live, epi, packed):
    from vtpack_amd import ops
    M, N = 2600, 768
    a, w, bias, res = _operands(M, N, 31 * live + len(epi), dev)
    rows_dev = torch.tensor([live], dtype=torch.int64, device=dev)
    out = torch.full((M, N), 7.0, device=dev, dtype=torch.bfloat16)
    ops.PACK_WEIGHTS = packed
    try:
        ops.linear(a.to(dev), w.to(dev), bias.to(dev) if "bias" in epi else None,
                   res.to(dev) if "res" in epi else None, act="gelu" if "gelu" in epi else "none",
                   rows_dev=rows_dev, out=out)
    finally:
        ops.PACK_WEIGHTS = True
    if live:
        want = _want(a[:live], w, bias, res[:live], epi)
        assert float(want.abs().max()) < 4.0
        assert abs_err(out[:live], want) <= BF16_ABS
    assert bool((out[live:] == 7.0).all())                      # nothing past the live rows is written


@pytest.mark.parametrize("live", [5, 40, 2049])
@pytest.mark.parametrize("epi", ["bias", "bias_gelu", "bias_res"])
def test_weight_stationary_strided_and_repeatable(dev, live, epi):
    """Operands as column slices of wider buffers (row strides larger than the widths); the columns beside the
    output slice stay untouched and every call returns the same bytes."""
    from vtpack_amd import ops
    M, N = 2304, 384
    a, w, bias, res = _operands(M, N, 77 + live, dev)
    abuf = torch.zeros(M, K + 64, dtype=torch.bfloat16)
    abuf[:, 32:32 + K] = a
    rbuf = torch.zeros(M, N + 32, dtype=torch.bfloat16)
    rbuf[:, 16:16 + N] = res
    abuf, rbuf = abuf.to(dev), rbuf.to(dev)
    obuf = torch.full((M, N + 16), 7.0, dtype=torch.bfloat16, device=dev)
    av, rv, ov = abuf[:, 32:32 + K], rbuf[:, 16:16 + N], obuf[:, 8:8 + N]
    rows_dev = torch.tensor([live], dtype=torch.int64, device=dev)
    args = dict(bias=bias.to(dev), residual=rv if "res" in epi else None, act="gelu" if "gelu" in epi else "none",
                rows_dev=rows_dev, out=ov)
    ops.linear(av, w.to(dev), **args)
    want = _want(a[:live], w, bias, res[:live], epi)
    assert abs_err(ov[:live], want) <= BF16_ABS
    assert bool((obuf[:, :8] == 7.0).all()) and bool((obuf[:, 8 + N:] == 7.0).all()) and bool((ov[live:] == 7.0).all())
    first = obuf.clone()
    for _ in range(3):
        ops.linear(av, w.to(dev), **args)
        assert torch.equal(obuf, first)


def test_weight_stationary_live_rows_match_host_rows(dev):
    """The same rows through the device-side count and as a plain host-side row count give the same bytes."""
    from vtpack_amd import ops
    M, N = 4096, 384
    a, w, bias, res = _operands(M, N, 5, dev)
    a, w, bias, res = a.to(dev), w.to(dev), bias.to(dev), res.to(dev)
    full = ops.linear(a, w, bias, residual=res)
    for live in (33, 1000, 4095):
        out = torch.zeros_like(full)
        ops.linear(a, w, bias, residual=res, rows_dev=torch.tensor([live], dtype=torch.int64, device=dev), out=out)
        assert torch.equal(out[:live], full[:live])


# ----------------------------------------------------------------------------- host-side operand checks
def test_operand_checks_raise_before_any_launch(dev):
    """Mismatched dtypes, devices or shapes raise on the host (TypeError / ValueError), as nn.Linear and
    nn.LayerNorm would, instead of letting a kernel read a buffer with the wrong element size."""
    from vtpack_amd import ops
    bf, f32 = torch.bfloat16, torch.float32
    a = torch.zeros(64, 384, dtype=bf, device=dev)
    w = torch.zeros(384, 384, dtype=bf, device=dev)
    b = torch.zeros(384, dtype=bf, device=dev)
    with pytest.raises(TypeError):
        ops.linear(a.float(), w, b)                                  # fp32 activations into a bf16 model
    with pytest.raises(TypeError):
        ops.linear(a, w, b.float())
    with pytest.raises(TypeError):
        ops.linear(a, w, b, residual=torch.zeros(64, 384, dtype=f32, device=dev))
    with pytest.raises(ValueError):
        ops.linear(a, torch.zeros(384, 192, dtype=bf, device=dev), b)    # weight of the wrong width
    with pytest.raises(ValueError):
        ops.linear(a, w, torch.zeros(100, dtype=bf, device=dev))
    with pytest.raises(ValueError):
        ops.linear(a, w, b, residual=torch.zeros(64, 192, dtype=bf, device=dev))
    with pytest.raises(RuntimeError):
        ops.linear(a.cpu(), w, b)                                    # no CPU fallback
    with pytest.raises(TypeError):
        ops.layernorm(a, b.float(), b)
    with pytest.raises(ValueError):
        ops.layernorm(a, b[:100], b)
    x = torch.zeros(2, 17, 384, dtype=bf, device=dev)
    idx = torch.zeros(2, 1, 1, dtype=torch.int64, device=dev)
    splits = torch.tensor([4, 2, 1], dtype=torch.int64, device=dev)
    patches, offsets, lengths = ops.index_to_patch(idx, splits, 4, 1)
    with pytest.raises(TypeError):
        ops.compress(x, patches, 4, 1, ln_weight=b.float(), ln_bias=b.float())
    with pytest.raises(ValueError):
        ops.compress(x, patches, 4, 1, ln_weight=b[:64], ln_bias=b[:64])
    q = torch.zeros(34, 384, dtype=bf, device=dev)
    with pytest.raises(TypeError):
        ops.decompress(q, patches, x.float(), 4, 1)
    with pytest.raises(TypeError):
        ops.decompress_layernorm(q, patches, x, 4, 1, b.float(), b.float())
    with pytest.raises(TypeError):
        ops.sparse_attention(q, x.float(), x.float(), offsets, 0.125, 6, 17)
    with pytest.raises(ValueError):
        ops.sparse_attention(q, x[:, :, :192], x[:, :, :192], offsets, 0.125, 6, 17)
    with pytest.raises(ValueError):
        ops.router(x, torch.zeros(3, 192, dtype=bf, device=dev), torch.zeros(3, dtype=bf, device=dev), 4, 4, 4)
    with pytest.raises(TypeError):
        ops.index_to_patch(idx.int(), splits, 4, 1)


def test_model_refuses_input_of_another_dtype(dev):
    from vtpack_amd.models.dge.deit_dge import VisionTransformer
    m = VisionTransformer(img_size=64, patch_size=16, embed_dim=192, depth=1, num_heads=3, split_sizes=[4, 2, 1])
    m = m.eval().to(dev).to(torch.bfloat16)
    with pytest.raises(TypeError):
        m(torch.zeros(2, 3, 64, 64, device=dev))                     # fp32 images, bf16 weights


def test_packed_weight_follows_every_edit_torch_counts_and_can_be_invalidated(dev):
    """The packed copy is refreshed by in-place torch ops, load_state_dict and dtype / device moves; a write
    through `.data` changes neither the version counter nor the address, so it needs `invalidate_packed`."""
    from vtpack_amd import ops
    lin = torch.nn.Linear(384, 384, bias=False).to(dev).to(torch.bfloat16)
    a = torch.randn(2304, 384, device=dev).bfloat16()

    def run():
        return ops.linear(a, lin.weight)

    def plain():
        ops.PACK_WEIGHTS = False
        try:
            return ops.linear(a, lin.weight)
        finally:
            ops.PACK_WEIGHTS = True

    base = run()
    assert torch.equal(base, plain())
    with torch.no_grad():
        lin.weight.mul_(0.5)                                         # counted by torch
    assert torch.equal(run(), plain())
    lin.load_state_dict({"weight": torch.randn(384, 384).bfloat16() * 0.05})
    assert torch.equal(run(), plain())
    lin.weight.data.mul_(2.0)                                        # NOT counted: the packed copy is stale ...
    ops.invalidate_packed(lin)                                       # ... until it is dropped
    got = run()
    assert torch.equal(got, plain())
    lin.weight.data.mul_(0.5)
    ops.invalidate_packed()                                          # every packed copy at once
    assert torch.equal(run(), plain())
