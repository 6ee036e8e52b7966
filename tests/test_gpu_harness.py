"""The evaluation loop and the budget loss on the HIP path (vtpack/engine/engine.py:20-32, :58-63, :102-147)."""
import pytest
import torch

from oracle import torch_ref

pytestmark = pytest.mark.gpu


def _complexity_from_lengths(lengths_per_block, N, C, heads, num_features, num_classes, image_rows):
    """The reference's MAC model written out from the per-sample query counts (deit_dge.py:32-36, :61-68,
    :117-121, :234-249; dge.py:140-143): -> (static, dynamic) averaged over the batch."""
    def block(ni, nq):
        attn = nq * C * C + 2 * ni * C * C + 2 * nq * ni * C + 3 * nq * ni * heads + nq * C * C
        mlp = nq * C * 4 * C + nq * 4 * C + nq * 4 * C * C
        router = ni / 16 * C + ni / 16 * C * 3
        return ni * C * 2 + attn + mlp + router
    base = image_rows * num_features * 3 + num_features * num_classes
    ni = torch.full_like(lengths_per_block[0], N, dtype=torch.float64)
    static = sum(block(ni, ni) for _ in lengths_per_block) + base
    dynamic = sum(block(ni, l.double()) for l in lengths_per_block) + base
    return float(static.mean()), float(dynamic.mean())


def test_evaluate_reports_the_reference_meters(dev):
    from vtpack_amd import harness
    from vtpack_amd.models.dge.deit_dge import VisionTransformer
    from vtpack_amd.synthetic import set_synthetic_router
    torch.manual_seed(0)
    m = VisionTransformer(img_size=128, patch_size=16, embed_dim=192, depth=3, num_heads=3, mlp_ratio=4,
                          num_classes=10, split_sizes=[4, 2, 1])
    set_synthetic_router(m, 1)
    m = m.to(dev)
    batches = list(harness.synthetic_loader(2, 4, 128, num_classes=10, seed=3))
    stats = harness.evaluate(batches, m, dev, dge_enable=True, dge_budget=0.5, dge_lr_scale=2.0)
    assert set(stats) == {"loss", "loss_cls", "loss_dge", "dge_ratio", "comp_static", "comp_dynamic", "acc1", "acc5"}
    assert not m.training
    # the same numbers from the CPU restatement's query counts and the MAC model written out by hand
    sd = torch_ref.float_state_dict(m)
    st, dy, ce, hit = [], [], [], 0
    for img, tgt in batches:
        traces = []
        logits = torch_ref.deit_dge_forward(sd, img, 3, 3, traces=traces)
        s, d = _complexity_from_lengths([tr["lengths"] for tr in traces], 65, 192, 3, 192, 10, 3 * 128)
        st.append(s)
        dy.append(d)
        ce.append(float(torch.nn.functional.cross_entropy(logits, tgt)))
        hit += int((logits.argmax(1) == tgt).sum())
    ratios = [d / s for s, d in zip(st, dy)]
    assert stats["comp_static"] == pytest.approx(sum(st) / 2, rel=1e-9)
    assert stats["comp_dynamic"] == pytest.approx(sum(dy) / 2, rel=1e-9)
    assert stats["dge_ratio"] == pytest.approx(sum(ratios) / 2, rel=1e-9)
    assert stats["loss_dge"] == pytest.approx(sum(2.0 * (r - 0.5) ** 2 for r in ratios) / 2, rel=1e-6)
    assert stats["loss_cls"] == pytest.approx(sum(ce) / 2, rel=1e-4)
    assert stats["loss"] == pytest.approx(stats["loss_cls"] + stats["loss_dge"], rel=1e-6)
    assert stats["acc1"] == pytest.approx(100.0 * hit / 8)
    assert 0.2 < stats["dge_ratio"] < 0.9


def test_budget_loss_reaches_the_routers_in_training(dev):
    """In training mode the gate is a straight-through Gumbel sample, so (ratio - budget)^2 has a gradient with
    respect to every router's weights (vtpack/engine/engine.py:58-63 with vtpack/layers/dge.py:40-59, :66-67)."""
    from vtpack_amd import harness
    from vtpack_amd.models.dge.deit_dge import VisionTransformer
    from vtpack_amd.synthetic import set_synthetic_router, synthetic_images
    torch.manual_seed(0)
    m = VisionTransformer(img_size=64, patch_size=8, embed_dim=64, depth=2, num_heads=1, mlp_ratio=2,
                          num_classes=5, split_sizes=[4, 2, 1])
    set_synthetic_router(m, 2)
    m = m.to(dev).train()
    img = synthetic_images(3, 64, seed=1).to(dev)
    out = m(img)
    loss_dge, ratio, comp = harness.budget_loss(m, img, dge_budget=0.3, dge_lr_scale=1.0)
    assert 0.0 < float(ratio) <= 1.0 and float(loss_dge) > 0
    (out.square().mean() + loss_dge).backward()
    for blk in m.blocks:
        g = blk.dge.router.gate.weight.grad
        assert g is not None and bool(torch.isfinite(g).all()) and float(g.abs().max()) > 0
    # the loss alone moves the routers too
    m.zero_grad()
    m(img)
    harness.budget_loss(m, img, dge_budget=0.3)[0].backward()
    assert all(float(blk.dge.router.gate.weight.grad.abs().max()) > 0 for blk in m.blocks)
