"""Host-side logic of the package: API surface, state-dict names, error behaviour, complexity counter."""
import math

import pytest
import torch


def test_layer_api_surface():
    import vtpack_amd.layers as L
    for name in ["DynamicGrainedEncoder", "grained_sample_compress", "grained_sample_decompress",
                 "grained_sample_index_to_patch", "batched_sparse_gemm", "batched_sparse_attention"]:
        assert hasattr(L, name)          # vtpack/layers/__init__.py:1-10
    from vtpack_amd import _C
    for name in ["grained_sample_compress", "grained_sample_decompress", "grained_sample_index_to_patch",
                 "grained_sample_index_to_patch_dense", "batched_sparse_gemm_forward",
                 "batched_sparse_gemm_v2_forward", "batched_sparse_attention_forward"]:
        assert callable(getattr(_C, name))   # vtpack/layers/csrc/vision.cpp:11-21


def test_install_as_vtpack_registers_operator_module():
    import sys
    import vtpack_amd
    saved = {k: sys.modules.get(k) for k in ("vtpack", "vtpack._C")}
    try:
        c = vtpack_amd.install_as_vtpack()
        from vtpack import _C
        assert _C is c and callable(_C.grained_sample_compress)
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def test_state_dict_keys_follow_the_reference():
    from vtpack_amd.models.dge import deit_dge_s124_tiny_patch16_256
    m = deit_dge_s124_tiny_patch16_256()
    keys = set(m.state_dict().keys())
    want = {"cls_token", "pos_embed", "patch_embed.proj.weight", "patch_embed.proj.bias", "norm.weight",
            "norm.bias", "head.weight", "head.bias"}
    for i in range(12):
        for k in ["norm1.weight", "norm1.bias", "attn.q.weight", "attn.q.bias", "attn.kv.weight", "attn.kv.bias",
                  "attn.proj.weight", "attn.proj.bias", "norm2.weight", "norm2.bias", "mlp.fc1.weight",
                  "mlp.fc1.bias", "mlp.fc2.weight", "mlp.fc2.bias", "dge.splits", "dge.router.gate.weight",
                  "dge.router.gate.bias"]:
            want.add(f"blocks.{i}.{k}")
    assert keys == want
    assert m.blocks[0].dge.splits.dtype == torch.int64 and m.blocks[0].dge.splits.tolist() == [4, 2, 1]
    assert m.bfloat16().blocks[0].dge.splits.dtype == torch.int64      # integer data survives dtype casts
    assert m.pos_embed.shape == (1, 257, 192) and m.blocks[0].norm1.eps == 1e-6


def test_router_initialisation():
    # vtpack/layers/dge.py:129-138: bias = +-1/2 ln 38 in favour of the finest split
    from vtpack_amd.layers import DynamicGrainedEncoder
    d = DynamicGrainedEncoder(64, [4, 2, 1])
    b = 0.5 * math.log(38.0)
    assert torch.allclose(d.router.gate.bias, torch.tensor([b, -b, -b]), atol=1e-6)
    assert 0.005 < float(d.router.gate.weight.std()) < 0.015 and d.region_size == 4
    assert torch.allclose(DynamicGrainedEncoder(64, [1]).router.gate.bias, torch.zeros(1))


def test_operators_refuse_cpu_tensors_and_training():
    from vtpack_amd import _C
    from vtpack_amd.layers import DynamicGrainedEncoder
    x = torch.zeros(1, 17, 8)
    patches = torch.zeros(2, 4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="GPU only"):
        _C.grained_sample_compress(x, patches, 4, 4, 1)
    with pytest.raises(RuntimeError, match="GPU only"):
        _C.batched_sparse_attention_forward(torch.zeros(1, 2, 64), torch.zeros(1, 1, 3, 64), torch.zeros(1, 1, 3, 64),
                                            torch.tensor([2]), 1.0)
    with pytest.raises(ValueError):
        DynamicGrainedEncoder(8, [4, 3])           # 3 does not divide the region size 4
    d = DynamicGrainedEncoder(8, [4, 2, 1], sparse_train=True).train()
    with pytest.raises(RuntimeError, match="GPU only"):
        d.compress(x, 4, 4)                        # sparse training uses the kernels: no CPU path either
    with pytest.raises(TypeError):
        _C.grained_sample_index_to_patch(torch.zeros(1, 1, 1, dtype=torch.int32), torch.tensor([4, 2, 1]), 4, 1)


def _fake_states(model, gate_index):
    B, N, C = 2, 257, model.embed_dim
    for blk in model.blocks:
        gate = torch.zeros(B, 4, 4, 3)
        gate[..., gate_index] = 1.0
        blk.dge.states.update({"input": torch.zeros(B, N, C), "gate": gate, "num_extra_tokens": 1})


@pytest.mark.parametrize("factory,macs", [("deit_dge_s124_small_patch16_256", 6.1e9),
                                          ("deit_dge_s124_tiny_patch16_256", 1.7e9)])
def test_complexity_counter_reproduces_published_macs(factory, macs):
    """Static MACs of DeiT-S / DeiT-Ti at 256 px: 6.1 G / 1.7 G (README.md:59,61 of the reference)."""
    from vtpack_amd.models import dge as zoo
    m = getattr(zoo, factory)().eval()
    img = torch.zeros(2, 3, 256, 256)
    _fake_states(m, 0)                       # all-fine gate: every token is its own query
    c = m.complexity(img)
    assert abs(float(c["static"]) - macs) / macs < 0.03
    assert float(c["dynamic"]) == pytest.approx(float(c["static"]))
    _fake_states(m, 2)                       # all-coarse gate: 17 queries per image
    c2 = m.complexity(img)
    assert float(c2["static"]) == pytest.approx(float(c["static"]))
    assert 0.1 < float(c2["dynamic"]) / float(c2["static"]) < 0.4


def test_dense_training_branch_equals_the_sparse_statement_on_cpu():
    """Training without sparse_train is plain torch (vtpack/layers/dge.py:68-72, :91-95): with its hard one-hot
    gate it must give what the sparse operators give for the sampled granularity, and pass gradients to the
    input and to the router."""
    from oracle import torch_ref
    from vtpack_amd.layers import DynamicGrainedEncoder
    torch.manual_seed(3)
    B, H, W, C, extra = 2, 8, 12, 16, 1
    d = DynamicGrainedEncoder(C, [4, 2, 1]).train()
    with torch.no_grad():
        d.router.gate.bias.zero_()
        d.router.gate.weight.normal_(0, 1.0)
    x = torch.randn(B, extra + H * W, C, requires_grad=True)
    comp = d.compress(x, H, W)
    assert comp.shape[0] == B * (extra + H * W + H * W // 4 + H * W // 16) and d.states["patches"] is None
    gate = d.states["gate"]
    assert torch.equal(gate.sum(-1), torch.ones_like(gate.sum(-1))) and set(gate.unique().tolist()) <= {0.0, 1.0}
    out = d.decompress(torch.tanh(comp) * 2)
    idx = gate.argmax(-1)
    assert len(idx.unique()) > 1
    patches, _ = torch_ref.index_to_patch(idx, d.splits, 4, extra)
    xd = x.detach()
    c_ref = torch_ref.compress(xd, patches, H, W, extra)
    want = torch_ref.decompress(torch.tanh(c_ref) * 2 - c_ref, patches, xd, H, W, extra, True)
    assert float((out - want).abs().max()) <= 1e-5
    out.square().sum().backward()
    assert x.grad is not None and float(x.grad.abs().max()) > 0
    assert float(d.router.gate.weight.grad.abs().max()) > 0


def test_checkpoint_round_trip(tmp_path):
    """A checkpoint written the way the reference's training loop writes it ({"model": state_dict, ...}) loads
    through a loader that executes nothing from the file, into the same keys and values (main.py:372-379)."""
    from vtpack_amd import harness
    from vtpack_amd.models.dge import deit_dge_s124_tiny_patch16_256
    torch.manual_seed(0)
    a = deit_dge_s124_tiny_patch16_256(num_classes=10)
    with torch.no_grad():
        for p in a.parameters():
            if p.is_floating_point():
                p.add_(0.01 * torch.randn_like(p))
    path = tmp_path / "checkpoint.pth"
    torch.save({"model": a.state_dict(), "epoch": 7, "args": {"dge_budget": 0.5}}, path)
    torch.manual_seed(1)
    b = deit_dge_s124_tiny_patch16_256(num_classes=10)
    rest = harness.load_checkpoint(b, path)
    assert rest == {"epoch": 7, "args": {"dge_budget": 0.5}}
    sa, sb = a.state_dict(), b.state_dict()
    assert list(sa) == list(sb) and all(torch.equal(sa[k], sb[k]) for k in sa)
    assert sb["blocks.0.dge.splits"].dtype == torch.int64
    # a bare state dict and a DistributedDataParallel-style wrapper are accepted as well
    torch.save(a.state_dict(), path)

    class Wrapped(torch.nn.Module):
        def __init__(self, m):
            super().__init__()
            self.module = m

    torch.manual_seed(2)
    c = Wrapped(deit_dge_s124_tiny_patch16_256(num_classes=10))
    assert harness.load_checkpoint(c, path) == {}
    assert all(torch.equal(sa[k], v) for k, v in c.module.state_dict().items())
    # a checkpoint of another architecture is refused, not half-loaded
    with pytest.raises(RuntimeError):
        harness.load_checkpoint(deit_dge_s124_tiny_patch16_256(num_classes=10, distilled=True), path)


def test_evaluate_meters_on_a_plain_model():
    """The evaluation loop's meters (vtpack/engine/engine.py:102-147): per-batch means of the loss, accuracies
    weighted by the batch size, against a direct computation."""
    from vtpack_amd import harness
    torch.manual_seed(0)
    net = torch.nn.Sequential(torch.nn.Flatten(), torch.nn.Linear(3 * 8 * 8, 7))
    batches = [(torch.randn(5, 3, 8, 8), torch.randint(0, 7, (5,))), (torch.randn(3, 3, 8, 8), torch.randint(0, 7, (3,)))]
    stats = harness.evaluate(batches, net, "cpu")
    assert set(stats) == {"loss", "acc1", "acc5"}
    with torch.no_grad():
        outs = [net(x) for x, _ in batches]
    losses = [float(torch.nn.functional.cross_entropy(o, t)) for o, (_, t) in zip(outs, batches)]
    assert stats["loss"] == pytest.approx(sum(losses) / 2)
    hits1 = sum(int((o.argmax(1) == t).sum()) for o, (_, t) in zip(outs, batches))
    hits5 = sum(int((o.topk(5, 1).indices == t[:, None]).any(1).sum()) for o, (_, t) in zip(outs, batches))
    assert stats["acc1"] == pytest.approx(100.0 * hits1 / 8) and stats["acc5"] == pytest.approx(100.0 * hits5 / 8)


def test_budget_loss_from_planted_gates():
    """loss_dge = scale * (dynamic / static - budget)^2 (vtpack/engine/engine.py:58-63) on the counter's output."""
    from vtpack_amd import harness
    from vtpack_amd.models.dge import deit_dge_s124_tiny_patch16_256
    m = deit_dge_s124_tiny_patch16_256().eval()
    img = torch.zeros(2, 3, 256, 256)
    _fake_states(m, 2)
    loss, ratio, comp = harness.budget_loss(m, img, dge_budget=0.5, dge_lr_scale=3.0)
    assert float(ratio) == pytest.approx(float(comp["dynamic"]) / float(comp["static"]))
    assert float(loss) == pytest.approx(3.0 * (float(ratio) - 0.5) ** 2)
    _fake_states(m, 0)
    loss, ratio, _ = harness.budget_loss(m, img, dge_budget=1.0)
    assert float(ratio) == pytest.approx(1.0) and float(loss) == pytest.approx(0.0, abs=1e-12)
    # the per-encoder ratio of engine.py:20-32 on the same states
    assert float(harness.get_complexity(m)) == pytest.approx(1.0)


def test_states_resolve_deferred_values_on_every_read_and_on_every_way_out():
    """`states` hands out what the reference's plain dict would hold, however it is read, and a deferred value is
    worked out again on every read (a graph replay rewrites the tensors behind it without running Python)."""
    from vtpack_amd.layers.dge import Deferred, States
    box = {"n": 3}
    st = States({"plain": 7, "batches": Deferred(lambda: box["n"]), "comp": Deferred(lambda: list(range(box["n"])))})
    assert st["batches"] == 3 and st.get("comp") == [0, 1, 2] and st.get("missing", 5) == 5
    box["n"] = 2                                   # what a replay does: new counts, no Python
    assert st["batches"] == 2 and st["comp"] == [0, 1]
    assert isinstance(dict.__getitem__(st, "batches"), Deferred)       # nothing was stored back
    for view in (dict(st), {**st}, st.copy(), st.snapshot(), dict(st.items()), dict(zip(st.keys(), st.values()))):
        assert type(view) is dict and view == {"plain": 7, "batches": 2, "comp": [0, 1]}
    snap = st.copy()
    box["n"] = 4
    assert snap["batches"] == 2 and st["batches"] == 4                 # a snapshot does not follow
    assert st.setdefault("batches", 0) == 4 and st.setdefault("new", 9) == 9
    assert st.pop("comp") == [0, 1, 2, 3] and "comp" not in st and st.pop("comp", None) is None
    with pytest.raises(KeyError):
        st.pop("comp")
    seen = {}
    while st:
        k, v = st.popitem()
        seen[k] = v
    assert seen == {"plain": 7, "batches": 4, "new": 9}


def test_fused_forward_refuses_a_distillation_token_without_a_class_token():
    """The reference never builds that token order (deit_dge.py:270-275); layer mode raises in embed_tokens and the
    fused forward must not run with the distillation token in the class token's place."""
    from vtpack_amd import engine
    from vtpack_amd.models.dge.deit_dge import VisionTransformer
    m = VisionTransformer(img_size=32, patch_size=16, embed_dim=16, depth=1, num_heads=1, distilled=True,
                          split_sizes=[2, 1]).eval()
    m.cls_token = None
    img = torch.zeros(1, 3, 32, 32)
    with pytest.raises(ValueError, match="class token"):
        engine.model_forward(m, img)
    with pytest.raises(ValueError, match="class token"):
        m.embed_tokens(img)
