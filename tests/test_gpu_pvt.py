"""PVT+DGE caller (vtpack/models/dge/pvt_dge.py): blocks with spatially reduced keys/values, non-square token
grids without extra tokens, and the four-stage model, against the torch-CPU restatement on one state dict."""
import pytest
import torch

from oracle import torch_ref
from util import FP32_REL, abs_err, assert_close, randn, rel_err

pytestmark = pytest.mark.gpu


def _block(dim, heads, sr, dev, dtype, seed=0, fused=True, mlp_ratio=4, scale2d=3.0):
    from vtpack_amd.models.dge.pvt_dge import Block
    torch.manual_seed(seed)
    blk = Block(dim, heads, mlp_ratio=mlp_ratio, qkv_bias=True, norm_layer=lambda d: torch.nn.LayerNorm(d, eps=1e-6),
                sr_ratio=sr, split_sizes=[4, 2, 1], fused=fused)
    with torch.no_grad():      # non-trivial norms and biases so that mistakes in them are visible
        for p in blk.parameters():
            if p.is_floating_point() and p.dim() == 1:
                p.add_(0.1 * torch.randn_like(p))
            elif p.is_floating_point() and p.dim() == 2:
                p.mul_(scale2d)
    return blk.eval().to(dev).to(dtype)


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("dim,heads,sr,H,W,extra", [
    (128, 2, 4, 8, 16, 0),       # stage-2 style: reduction 4, non-square grid, KV length 8
    (64, 1, 2, 12, 8, 0),        # stage-1 style: one head, reduction 2, KV length 24
    (128, 2, 1, 8, 4, 1),        # last-stage style: class token, no reduction, non-square
])
def test_pvt_block_fp32(dev, fused, dim, heads, sr, H, W, extra):
    blk = _block(dim, heads, sr, dev, torch.float32, fused=fused)
    B = 3
    x = torch.from_numpy(randn(11, B, extra + H * W, dim))
    gate = torch.from_numpy(randn(12, B, H // 4, W // 4, 3))
    tr = {}
    want = torch_ref.block_forward(torch_ref.float_state_dict(blk), "", x, heads, gate=gate, trace=tr, size=(H, W),
                                   sr_ratio=sr)
    with torch.no_grad():
        got = blk(x.to(dev), H, W, gate=gate.to(dev))
    st = blk.dge.states
    L = int(tr["lengths"].sum())
    assert torch.equal(st["patches"][:L].cpu(), tr["patches"])
    lengths = st["batches"] if st["batches"] is not None else st["batches_device"].cpu()
    assert torch.equal(lengths, tr["lengths"])
    assert torch.equal(st["comp"][:L].cpu(), tr["comp"])
    assert rel_err(got, want) <= FP32_REL, rel_err(got, want)


def test_pvt_block_bf16(dev):
    """Stage-3 shape (C = 320, 5 heads, reduction 2) in bf16 against the fp32 CPU path on the same rounded weights."""
    dim, heads, sr, H, W = 320, 5, 2, 16, 16
    blk = _block(dim, heads, sr, dev, torch.bfloat16, seed=2, scale2d=1.0)
    x = torch.from_numpy(randn(13, 4, H * W, dim)).to(torch.bfloat16)
    gate = torch.from_numpy(randn(14, 4, 4, 4, 3)).to(torch.bfloat16)
    tr = {}
    want = torch_ref.block_forward(torch_ref.float_state_dict(blk), "", x.float(), heads, gate=gate.float(), trace=tr,
                                   size=(H, W), sr_ratio=sr)
    with torch.no_grad():
        got = blk(x.to(dev), H, W, gate=gate.to(dev))
    L = int(tr["lengths"].sum())
    assert torch.equal(blk.dge.states["patches"][:L].cpu(), tr["patches"])
    # the block adds a delta to its bf16 input: half a bf16 ulp of |x| <= 4 plus the delta's own 2e-2
    assert abs_err(got.float(), want) <= 2e-2 + 2 ** -7


def _pvt(dev, dtype, depths, seed=0, fused=True, img=128):
    from vtpack_amd.models.dge.pvt_dge import PyramidVisionTransformer
    from vtpack_amd.synthetic import set_synthetic_router
    torch.manual_seed(seed)
    m = PyramidVisionTransformer(img_size=img, patch_size=4, embed_dims=[64, 128, 320, 512], num_heads=[1, 2, 5, 8],
                                 mlp_ratios=[8, 8, 4, 4], qkv_bias=True,
                                 norm_layer=lambda d: torch.nn.LayerNorm(d, eps=1e-6), depths=depths,
                                 sr_ratios=[8, 4, 2, 1], split_sizes=[[4, 2, 1]] * 4, num_classes=100, fused=fused)
    set_synthetic_router(m, seed)
    return m.eval().to(dev).to(dtype)


def _dges(model):
    from vtpack_amd.layers import DynamicGrainedEncoder
    return [m for m in model.modules() if isinstance(m, DynamicGrainedEncoder)]


@pytest.mark.parametrize("fused", [True, False])
def test_pvt_model_fp32(dev, fused):
    """pvt_dge_s124 geometry at 128 px (token grids 32, 16, 8, 4 + class token), one block per stage, fp32."""
    from vtpack_amd.synthetic import synthetic_images
    depths = [1, 1, 1, 1]
    m = _pvt(dev, torch.float32, depths, fused=fused)
    img = synthetic_images(2, 128, seed=5)
    with torch.no_grad():
        got = m(img.to(dev))
    traces = []
    want = torch_ref.pvt_dge_forward(torch_ref.float_state_dict(m), img, [1, 2, 5, 8], depths, [8, 4, 2, 1],
                                     traces=traces)
    mixed = 0
    for dge, tr in zip(_dges(m), traces):
        assert torch.equal(dge.states["gate"].argmax(-1).cpu(), tr["indices"])
        L = int(tr["lengths"].sum())
        assert torch.equal(dge.states["patches"][:L].cpu(), tr["patches"])
        mixed += len(torch.unique(tr["indices"])) > 1
    assert mixed >= 3                                    # the synthetic router mixes granularities
    assert rel_err(got, want) <= FP32_REL, rel_err(got, want)


def test_pvt_model_bf16(dev):
    """Same geometry, two blocks per stage, bf16: logits within 2e-2 of the fp32 CPU path run on the same rounded
    weights with the GPU's gate choices forced; the free choices agree except at numerical near-ties."""
    from vtpack_amd.synthetic import synthetic_images
    depths = [2, 2, 2, 2]
    m = _pvt(dev, torch.bfloat16, depths, seed=1)
    img = synthetic_images(2, 128, seed=6, dtype=torch.bfloat16)
    with torch.no_grad():
        got = m(img.to(dev))
    forced = [d.states["gate"].float().argmax(-1).cpu() for d in _dges(m)]
    traces = []
    want = torch_ref.pvt_dge_forward(torch_ref.float_state_dict(m), img.float(), [1, 2, 5, 8], depths, [8, 4, 2, 1],
                                     forced_indices=forced, traces=traces)
    same = sum(int((f == tr["gate"].argmax(-1)).sum()) for f, tr in zip(forced, traces))
    total = sum(f.numel() for f in forced)
    print(f"bf16 gate agreement {same}/{total}")
    assert same / total >= 0.95
    assert_close(got.float(), want, torch.bfloat16, "PVT+DGE bf16 logits")


def test_pvt_feature_maps(dev):
    """Without a classifier the model returns the four stage outputs as NCHW maps (pvt_dge.py:318-325)."""
    from vtpack_amd.models.dge.pvt_dge import PyramidVisionTransformer
    from vtpack_amd.synthetic import synthetic_images
    torch.manual_seed(0)
    kw = dict(img_size=128, patch_size=4, embed_dims=[64, 128, 320, 512], num_heads=[1, 2, 5, 8],
              mlp_ratios=[8, 8, 4, 4], qkv_bias=True, depths=[1, 1, 1, 1], sr_ratios=[8, 4, 2, 1],
              split_sizes=[[4, 2, 1]] * 4, num_classes=0)
    m = PyramidVisionTransformer(**kw).eval().to(dev)
    img = synthetic_images(2, 128, seed=7).to(dev)
    with torch.no_grad():
        fused = m(img)
        layer = m.set_fused(False)(img)
    assert sorted(fused) == ["res2", "res3", "res4", "res5"]
    for name, c, s in (("res2", 64, 32), ("res3", 128, 16), ("res4", 320, 8), ("res5", 512, 4)):
        assert tuple(fused[name].shape) == (2, c, s, s)
        assert rel_err(fused[name], layer[name].cpu()) <= FP32_REL


@pytest.mark.parametrize("B,S,with_pos", [(2, 64, True), (3, 256, True), (1, 128, False)])
def test_first_stage_patch_embedding_in_one_pass(dev, B, S, with_pos):
    """Conv2d(3, 64, 4, 4) + bias, LayerNorm and `+ pos_embed` as one kernel (bf16): against torch in fp64 on the same
    bf16 operands, and against the three-launch composition it replaces (gathered patches -> Linear -> LayerNorm with
    the addend), from which it may differ by a rounding step where an fp32 sum falls next to a tie."""
    from vtpack_amd import ops
    g = torch.Generator().manual_seed(S + B)
    img = torch.randn(B, 3, S, S, generator=g).bfloat16().to(dev)
    conv_w = (torch.randn(64, 3, 4, 4, generator=g) * 0.2).bfloat16().to(dev)
    conv_b = (torch.randn(64, generator=g) * 0.1).bfloat16().to(dev)
    ln_w = (1 + 0.2 * torch.randn(64, generator=g)).bfloat16().to(dev)
    ln_b = (0.1 * torch.randn(64, generator=g)).bfloat16().to(dev)
    G = S // 4
    pos = (torch.randn(1, G * G, 64, generator=g) * 0.5).bfloat16().to(dev) if with_pos else None
    assert ops.fits_patch_embed_norm(img, conv_w, 4)
    got = ops.patch_embed_norm(img, conv_w, conv_b, ln_w, ln_b, 1e-6, pos, 4)
    assert got.shape == (B, G * G, 64)
    # fp64 statement of the modules, rounded to bf16 where they would round
    y = torch.nn.functional.conv2d(img.double(), conv_w.double(), conv_b.double(), stride=4)
    y = y.flatten(2).transpose(1, 2).bfloat16().double()
    y = torch.nn.functional.layer_norm(y, (64,), ln_w.double(), ln_b.double(), 1e-6).bfloat16().double()
    want = (y + pos.double()).bfloat16() if with_pos else y.bfloat16()
    err = (got.double() - want.double()).abs()
    assert float((err / want.double().abs().clamp_min(1.0)).max()) <= 2.0 ** -6          # at most two bf16 steps
    assert float((err > 0).double().mean()) < 0.03
    # the composition it replaces
    pat = img.reshape(B, 3, G, 4, G, 4).permute(0, 2, 4, 1, 3, 5).reshape(B * G * G, 48)
    tok = ops.linear(pat, conv_w.reshape(64, 48), conv_b)
    ref = ops.layernorm(tok, ln_w, ln_b, 1e-6, add=pos) if with_pos else ops.layernorm(tok, ln_w, ln_b, 1e-6)
    d = (got.float() - ref.view(B, G * G, 64).float()).abs()
    assert float((d / ref.view(B, G * G, 64).float().abs().clamp_min(1.0)).max()) <= 2.0 ** -6
    assert float((d > 0).float().mean()) < 0.03


def test_first_stage_patch_embedding_refuses_other_shapes(dev):
    from vtpack_amd import ops
    img = torch.zeros(1, 3, 96, 96, dtype=torch.bfloat16, device=dev)            # side not a multiple of 64
    w = torch.zeros(64, 3, 4, 4, dtype=torch.bfloat16, device=dev)
    assert not ops.fits_patch_embed_norm(img, w, 4)
    assert not ops.fits_patch_embed_norm(img.float(), w.float(), 4)
    assert not ops.fits_patch_embed_norm(torch.zeros(1, 3, 64, 64, dtype=torch.bfloat16, device=dev), w[:32], 4)
