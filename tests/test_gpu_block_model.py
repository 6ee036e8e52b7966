"""Block- and model-level parity of the HIP path against the torch-CPU restatement, same state dict."""
import numpy as np
import pytest
import torch

from oracle import torch_ref
from util import FP32_REL, LaunchNames, abs_err, assert_close, forced_reference, randn, rel_err

pytestmark = pytest.mark.gpu


def _block(dim, heads, dev, dtype, seed=0, fused=True):
    from vtpack_amd.models.dge.deit_dge import Block
    torch.manual_seed(seed)
    blk = Block(dim, heads, mlp_ratio=4, qkv_bias=True, norm_layer=lambda d: torch.nn.LayerNorm(d, eps=1e-6),
                split_sizes=[4, 2, 1], fused=fused)
    with torch.no_grad():      # non-trivial norms and biases so that mistakes in them are visible
        for p in blk.parameters():
            if p.is_floating_point() and p.dim() == 1:
                p.add_(0.1 * torch.randn_like(p))
            elif p.is_floating_point():
                p.mul_(3.0)
    return blk.eval().to(dev).to(dtype)


@pytest.mark.parametrize("fused", [True, False])
def test_single_block_fp32_injected_gate(dev, fused):
    """Config 1: one DGE block, DeiT-Ti width, fp32, batch 8, gate logits injected."""
    blk = _block(192, 3, dev, torch.float32, fused=fused)
    x = torch.from_numpy(randn(1, 8, 257, 192))
    gate = torch.from_numpy(randn(2, 8, 4, 4, 3))
    tr = {}
    sd = torch_ref.float_state_dict(blk)
    want = torch_ref.block_forward(sd, "", x, 3, gate=gate, trace=tr)
    with torch.no_grad():
        got = blk(x.to(dev), gate=gate.to(dev))
    st = blk.dge.states
    L = int(tr["lengths"].sum())
    # integers: bit exact
    assert torch.equal(st["patches"][:L].cpu(), tr["patches"])
    lengths = st["batches"] if st["batches"] is not None else st["batches_device"].cpu()
    assert torch.equal(lengths, tr["lengths"])
    # floating point
    assert torch.equal(st["comp"][:L].cpu(), tr["comp"])          # window means: same order, bit exact
    if fused:
        assert rel_err(st["queries"][:L], tr["q2"]) <= FP32_REL
    assert rel_err(got, want) <= FP32_REL, rel_err(got, want)


def test_single_block_router_path(dev):
    """Same block with the router deciding: gate logits and choices agree with the CPU path."""
    blk = _block(192, 3, dev, torch.float32, seed=3)
    with torch.no_grad():
        blk.dge.router.gate.bias.zero_()
        blk.dge.router.gate.weight.copy_(torch.from_numpy(randn(5, 3, 192)) * 0.1)
    x = torch.from_numpy(randn(4, 8, 257, 192))
    tr = {}
    want = torch_ref.block_forward(torch_ref.float_state_dict(blk), "", x, 3, trace=tr)
    with torch.no_grad():
        got = blk(x.to(dev))
    assert rel_err(blk.dge.states["gate"], tr["gate"]) <= FP32_REL
    assert torch.equal(blk.dge.states["gate"].argmax(-1).cpu(), tr["indices"])
    assert rel_err(got, want) <= FP32_REL


def test_block_bf16(dev):
    blk = _block(384, 6, dev, torch.bfloat16, seed=1)
    with torch.no_grad():      # keep activations O(1): this is the 2e-2 max-abs regime
        for p in blk.parameters():
            if p.is_floating_point() and p.dim() == 2:
                p.mul_(1.0 / 3.0)
    x = torch.from_numpy(randn(7, 4, 257, 384)).to(torch.bfloat16)
    gate = torch.from_numpy(randn(8, 4, 4, 4, 3)).to(torch.bfloat16)
    tr = {}
    want = torch_ref.block_forward(torch_ref.float_state_dict(blk), "", x.float(), 6, gate=gate.float(), trace=tr)
    with torch.no_grad():
        got = blk(x.to(dev), gate=gate.to(dev))
    L = int(tr["lengths"].sum())
    assert torch.equal(blk.dge.states["patches"][:L].cpu(), tr["patches"])
    # the block adds a delta to its bf16 input: the error bound is half a bf16 ulp of |x| <= 4 plus the delta's own
    assert abs_err(got.float(), want) <= 2e-2 + 2 ** -7


def _model(name, dev, dtype, seed=0, **kw):
    from vtpack_amd.models import dge as zoo
    from vtpack_amd.synthetic import set_synthetic_router
    torch.manual_seed(seed)
    m = getattr(zoo, name)(**kw)
    set_synthetic_router(m, seed)
    return m.eval().to(dev).to(dtype)


def _gate_report(model, traces):
    """Compare the GPU's per-layer gate choices with the oracle's own argmax on its activations."""
    same = total = 0
    worst_margin = 0.0
    for blk, tr in zip(model.blocks, traces):
        gpu_idx = blk.dge.states["gate"].float().argmax(-1).cpu()
        ref_gate = tr["gate_free"]
        ref_idx = ref_gate.argmax(-1)
        diff = gpu_idx != ref_idx
        same += int((~diff).sum())
        total += diff.numel()
        if diff.any():
            top2 = ref_gate.topk(2, dim=-1).values
            worst_margin = max(worst_margin, float((top2[..., 0] - top2[..., 1])[diff].max()))
    return same, total, worst_margin


_forced_reference = forced_reference


def _assert_bf16_gates_differ_only_at_near_ties(model, traces, floor):
    """bf16 routing against the fp32 CPU path: the choices agree on at least `floor` of the regions, and wherever
    they differ the CPU path's own top-2 margin is within what bf16 rounding of the activations and of the logits
    can move a logit (a few bf16 steps at the logits' magnitude), i.e. a true near-tie."""
    same, total, worst = _gate_report(model, traces)
    scale = max(float(tr["gate_free"].abs().max()) for tr in traces)
    print(f"bf16 gate agreement {same}/{total}, largest margin among disagreements {worst:.4f}, "
          f"largest |logit| {scale:.2f}")
    assert same / total >= floor
    assert worst <= 4 * 2.0 ** -8 * max(scale, 1.0), (worst, scale)


@pytest.mark.parametrize("fused", [True, False])
def test_deit_tiny_fp32_model(dev, fused):
    """Config 2 at a CPU-friendly batch: 12-layer DeiT-Ti+DGE, fp32, mixed gate from the router."""
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_tiny_patch16_256", dev, torch.float32, fused=fused)
    img = synthetic_images(4, 256, seed=1)
    with torch.no_grad():
        got = m(img.to(dev))
    traces = []
    want = torch_ref.deit_dge_forward(torch_ref.float_state_dict(m), img, 3, 12, traces=traces)
    # gate choices and query counts of every layer, bit exact against the free-running CPU path
    ratios = []
    for blk, tr in zip(m.blocks, traces):
        assert torch.equal(blk.dge.states["gate"].argmax(-1).cpu(), tr["indices"])
        L = int(tr["lengths"].sum())
        assert torch.equal(blk.dge.states["patches"][:L].cpu(), tr["patches"])
        ratios.append(L / (4 * 257))
    assert 0.2 < np.mean(ratios) < 0.8, ratios          # the synthetic router really mixes granularities
    assert rel_err(got, want) <= FP32_REL, rel_err(got, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_with_and_without_fused_patch_embedding(dev, dtype):
    """The patch embedding read straight from the images (position embedding in its epilogue) against the unfolded
    copy + Linear + addition: the same logits bit for bit in fp32, the same routing and logits within two bf16
    steps in bf16 (one rounding of the tokens instead of two)."""
    from vtpack_amd import engine
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_tiny_patch16_256", dev, dtype)
    img = synthetic_images(4, 256, seed=2).to(dev).to(dtype)
    assert engine.FUSE_PATCH_EMBED
    with torch.no_grad():
        got = m(img)
        tok = m.blocks[0].dge.states["input"].clone()
        engine.FUSE_PATCH_EMBED = False
        try:
            ref = m(img)
            tok_ref = m.blocks[0].dge.states["input"]
        finally:
            engine.FUSE_PATCH_EMBED = True
    if dtype == torch.float32:
        assert torch.equal(tok, tok_ref) and torch.equal(got, ref)
    else:
        # the tokens differ by the one rounding saved; a routing decision on a near tie may follow them, so the
        # logits get the model-level bf16 bound
        assert abs_err(tok.float(), tok_ref.float()) <= 2.0 ** -7 * float(tok_ref.float().abs().max())
        assert abs_err(got.float(), ref.float()) <= 2e-2 * max(1.0, float(ref.float().abs().max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_with_fused_next_layernorm(dev, dtype):
    """The scatter-back that also writes the next block's first LayerNorm is an option of the fused path: with it
    the model gives the same gate choices and, the two LayerNorm kernels being one arithmetic, the same logits."""
    from vtpack_amd import engine
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_tiny_patch16_256", dev, dtype)
    img = synthetic_images(3, 256, seed=5, dtype=dtype).to(dev)
    with torch.no_grad():
        base = m(img)
        idx = [blk.dge.states["gate"].argmax(-1).clone() for blk in m.blocks]
        engine.FUSE_NEXT_NORM = True
        try:
            got = m(img)
        finally:
            engine.FUSE_NEXT_NORM = False
    for blk, want in zip(m.blocks, idx):
        assert torch.equal(blk.dge.states["gate"].argmax(-1), want)
    assert_close(got.float(), base.float().cpu(), dtype, "logits with the fused LayerNorm")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_router_with_layernorm_is_the_same_model(dev, dtype):
    """The router that also writes the first LayerNorm (an option of the fused path) and the two separate kernels
    are the same arithmetic: identical logits and gate choices."""
    from vtpack_amd import engine
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_tiny_patch16_256", dev, dtype)
    img = synthetic_images(3, 256, seed=6, dtype=dtype).to(dev)
    with torch.no_grad():
        apart = m(img)
        idx = [blk.dge.states["gate"].argmax(-1).clone() for blk in m.blocks]
        engine.FUSE_ROUTER_NORM = True
        try:
            fused = m(img)
        finally:
            engine.FUSE_ROUTER_NORM = False
    for blk, want in zip(m.blocks, idx):
        assert torch.equal(blk.dge.states["gate"].argmax(-1), want)
    assert torch.equal(fused, apart)


def test_deit_small_bf16_model(dev):
    """Config 3 at a CPU-friendly batch: DeiT-S+DGE bf16 logits within 2e-2 of the fp32 CPU path fed the same
    (bf16-rounded) weights and the same gate choices; the gate choices themselves agree with the CPU path's own
    argmax except at numerical near-ties."""
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_small_patch16_256", dev, torch.bfloat16)
    img = synthetic_images(4, 256, seed=2, dtype=torch.bfloat16)
    with torch.no_grad():
        got = m(img.to(dev))
    want, traces = _forced_reference(m, img.float(), 6, 12)
    _assert_bf16_gates_differ_only_at_near_ties(m, traces, 0.97)
    assert_close(got.float(), want, torch.bfloat16, "DeiT-S+DGE bf16 logits")


def test_deit_small_bf16_model_on_the_weight_stationary_kernels(dev):
    """The same comparison at batch 8: 2056 token rows, the smallest batch at which the 256 px model takes the path
    the headline measurement runs - both LayerNorms folded into weight-stationary Linears, proj writing the
    statistics records, the scatter-back routing the next block and writing the records of its tokens, attention with
    resident keys and values - instead of the streaming Linear and standalone LayerNorms of smaller batches."""
    from vtpack_amd import _lib
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_small_patch16_256", dev, torch.bfloat16, seed=4)
    img = synthetic_images(8, 256, seed=5, dtype=torch.bfloat16)
    _lib.timer = names = LaunchNames()
    try:
        with torch.no_grad():
            got = m(img.to(dev))
    finally:
        _lib.timer = None
    assert names.names.count("vtdge_linear_layernorm") == 12 and names.names.count("vtdge_linear_layernorm_pair") == 12
    assert names.names.count("vtdge_linear_stats") == 12
    # the first block packs its own queries; every scatter-back but the last also packs the next block's
    assert names.names.count("vtdge_decompress_router_compress") == 11 and names.names.count("vtdge_decompress") == 1
    assert names.names.count("vtdge_decompress_router") == 0 and names.names.count("vtdge_layernorm_rows") == 1
    assert names.names.count("vtdge_compress_regions") == 1 and names.names.count("vtdge_index_to_patch") == 0
    want, traces = forced_reference(m, img.float(), 6, 12)
    for blk, tr in zip(m.blocks, traces):
        assert torch.equal(blk.dge.states["patches"].cpu(), tr["patches"])
        assert torch.equal(blk.dge.states["batches"], tr["lengths"])
    _assert_bf16_gates_differ_only_at_near_ties(m, traces, 0.97)
    assert_close(got.float(), want, torch.bfloat16, "DeiT-S+DGE bf16 logits, batch 8")


def test_scatter_back_that_packs_the_next_block_is_the_same_model(dev):
    """With and without the scatter-back packing the next block's queries (and with the region kernels off
    altogether) the model is the same arithmetic on the same rows: logits, gate choices, descriptors and query
    counts of every block are identical."""
    from vtpack_amd import engine
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_small_patch16_256", dev, torch.bfloat16, seed=7)
    img = synthetic_images(8, 256, seed=8, dtype=torch.bfloat16).to(dev)

    def run():
        with torch.no_grad():
            out = m(img)
        return out, [(b.dge.states["gate"].clone(), b.dge.states["patches"].clone(), b.dge.states["batches"].clone(),
                      b.dge.states["comp"].clone()) for b in m.blocks]

    chained, st_chained = run()
    engine.PACK_NEXT = False
    try:
        apart, st_apart = run()
    finally:
        engine.PACK_NEXT = True
    assert torch.equal(chained, apart)
    for a, b in zip(st_chained, st_apart):
        for u, v in zip(a, b):
            assert torch.equal(u, v)


@pytest.mark.parametrize("factory,heads", [("deit_dge_s124_base_patch16_256", 12), ("deit_dge_s124_tiny_patch16_256", 3)])
def test_deit_other_widths_bf16_model(dev, factory, heads):
    """The other widths the reference ships (DeiT-Base: 768 channels, 12 heads; DeiT-Ti: 192 channels, 3 heads;
    vtpack/models/dge/deit_dge.py:302-329) in bf16: the streaming Linear and the row-wise sampling kernels instead of
    the weight-stationary ones, same bar as DeiT-S."""
    from vtpack_amd.synthetic import synthetic_images
    m = _model(factory, dev, torch.bfloat16, seed=6)
    img = synthetic_images(2, 256, seed=8, dtype=torch.bfloat16)
    with torch.no_grad():
        got = m(img.to(dev))
    want, traces = forced_reference(m, img.float(), heads, 12)
    for blk, tr in zip(m.blocks, traces):
        assert torch.equal(blk.dge.states["patches"].cpu(), tr["patches"])
        assert torch.equal(blk.dge.states["batches"], tr["lengths"])
    _assert_bf16_gates_differ_only_at_near_ties(m, traces, 0.95)
    assert_close(got.float(), want, torch.bfloat16, f"{factory} bf16 logits")


def test_high_res_geometry(dev):
    """Config 5 geometry (512 px: 1024 tokens + cls, 64 regions, KV length 1025) on a 2-layer fp32 model."""
    from vtpack_amd.models.dge.deit_dge import VisionTransformer
    from vtpack_amd.synthetic import set_synthetic_router, synthetic_images
    torch.manual_seed(0)
    m = VisionTransformer(img_size=512, patch_size=16, embed_dim=192, depth=2, num_heads=3, mlp_ratio=4,
                          qkv_bias=True, split_sizes=[4, 2, 1])
    set_synthetic_router(m, 4)
    m = m.eval().to(dev)
    img = synthetic_images(2, 512, seed=3)
    with torch.no_grad():
        got = m(img.to(dev))
    traces = []
    want = torch_ref.deit_dge_forward(torch_ref.float_state_dict(m), img, 3, 2, traces=traces)
    for blk, tr in zip(m.blocks, traces):
        assert torch.equal(blk.dge.states["gate"].argmax(-1).cpu(), tr["indices"])
    assert rel_err(got, want) <= FP32_REL


def test_deit_small_bf16_512px_model(dev):
    """Config 5 at a CPU-friendly batch: the 12-layer DeiT-S+DGE in bf16 at 512 px (1024 tokens + cls, 64 regions
    per sample, keys / values of length 1025: the streaming attention kernel and the weight-stationary Linears on
    N = 1025 token rows per sample), logits within 2e-2 of the fp32 CPU path fed the same bf16 weights and the same
    gate choices; integer outputs of every layer bit exact given those choices."""
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_small_patch16_256", dev, torch.bfloat16, seed=2, img_size=512)
    img = synthetic_images(2, 512, seed=7, dtype=torch.bfloat16)
    with torch.no_grad():
        got = m(img.to(dev))
    want, traces = _forced_reference(m, img.float(), 6, 12)
    for blk, tr in zip(m.blocks, traces):
        L = int(tr["lengths"].sum())
        assert torch.equal(blk.dge.states["patches"].cpu(), tr["patches"]) and L == tr["patches"].shape[0]
        assert torch.equal(blk.dge.states["batches"], tr["lengths"])
    _assert_bf16_gates_differ_only_at_near_ties(m, traces, 0.95)
    assert_close(got.float(), want, torch.bfloat16, "DeiT-S+DGE bf16 512 px logits")


@pytest.mark.parametrize("variant,fused", [("distilled", True), ("distilled", False), ("representation", True),
                                           ("no_cls", True)])
def test_deit_variants_fp32(dev, variant, fused):
    """The other shapes of the reference's VisionTransformer (vtpack/models/dge/deit_dge.py:171-214, :267-299): a
    distillation token (two extra tokens, the mean of two heads), a pre-logits layer, no class token."""
    from vtpack_amd.models.dge.deit_dge import VisionTransformer
    from vtpack_amd.synthetic import set_synthetic_router, synthetic_images
    kw = {"distilled": {"distilled": True}, "representation": {"representation_size": 96},
          "no_cls": {"cls_token": False}}[variant]
    torch.manual_seed(4)
    m = VisionTransformer(img_size=128, patch_size=16, embed_dim=192, depth=3, num_heads=3, mlp_ratio=4,
                          qkv_bias=True, num_classes=100, split_sizes=[4, 2, 1], fused=fused, **kw)
    set_synthetic_router(m, 5)
    with torch.no_grad():
        for name, p in m.named_parameters():
            if p.dim() == 1 and p.is_floating_point() and "router" not in name:
                p.add_(0.1 * torch.randn_like(p))
    m = m.eval().to(dev)
    img = synthetic_images(3, 128, seed=8)
    with torch.no_grad():
        got = m(img.to(dev))
    traces = []
    want = torch_ref.deit_dge_forward(torch_ref.float_state_dict(m), img, 3, 3, traces=traces)
    extra = {"distilled": 2, "representation": 1, "no_cls": 0}[variant]
    for blk, tr in zip(m.blocks, traces):
        assert blk.dge.states["num_extra_tokens"] == extra
        assert torch.equal(blk.dge.states["gate"].argmax(-1).cpu(), tr["indices"])
        assert torch.equal(blk.dge.states["patches"].cpu(), tr["patches"])
        assert torch.equal(blk.dge.states["batches"], tr["lengths"])
    assert got.shape == want.shape == (3, 100)
    assert rel_err(got, want) <= FP32_REL, rel_err(got, want)


def test_states_of_fused_and_layer_mode_agree(dev):
    """`states` as the reference's code reads it (vtpack/layers/dge.py:81-84): the fused path hands out the same
    keys as the layer path - CPU query counts, tensors cut to the live rows - worked out on first read."""
    blk = _block(192, 3, dev, torch.float32, seed=9)
    x = torch.from_numpy(randn(11, 4, 257, 192)).to(dev)
    gate = torch.from_numpy(randn(12, 4, 4, 4, 3)).to(dev)
    with torch.no_grad():
        blk.fused = True
        out_f = blk(x, gate=gate)
        st_f = {k: blk.dge.states[k] for k in ("comp", "patches", "batches", "size", "num_extra_tokens")}
        blk.fused = False
        out_l = blk(x, gate=gate)
        st_l = blk.dge.states
    assert st_f["batches"].device.type == "cpu" and torch.equal(st_f["batches"], st_l["batches"])
    L = int(st_l["batches"].sum())
    assert st_f["patches"].shape == (L, 4) and st_f["comp"].shape == (L, 192)
    keep = [0, 1, 3]                                           # column 2 of extra-token rows is undefined
    assert torch.equal(st_f["patches"][:, keep], st_l["patches"][:, keep])
    assert torch.equal(st_f["comp"], st_l["comp"])
    assert st_f["size"] == st_l["size"] and st_f["num_extra_tokens"] == st_l["num_extra_tokens"] == 1
    assert rel_err(out_f, out_l) <= FP32_REL


def test_forward_captured_in_a_graph_follows_its_input(dev):
    """The whole forward holds no synchronisation and no host-side length (every packed kernel reads the live row
    count from device memory), so it can be captured once in a HIP graph and replayed on new images written into
    the captured input buffer: the router then takes other decisions and the row counts change inside the graph.
    Every replay must give, bit for bit, what the eager forward gives for the same images - with eager work and
    synchronisations of the program between the replays, and the two streams of a block inside the capture."""
    from vtpack_amd.synthetic import synthetic_images
    m = _model("deit_dge_s124_small_patch16_256", dev, torch.bfloat16)
    static_in = synthetic_images(8, 256, seed=11, dtype=torch.bfloat16).to(dev)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):           # warm-up off the default stream, as capture requires
            m(static_in)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            static_out = m(static_in)
        counts = []
        for seed in (11, 12, 13, 11):
            img = synthetic_images(8, 256, seed=seed, dtype=torch.bfloat16).to(dev)
            eager = m(img)
            counts.append(int(m.blocks[3].dge.states["batches_device"].sum()))
            torch.cuda.synchronize()
            static_in.copy_(img)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, eager), f"replay on the images of seed {seed} differs from the eager forward"
    assert len(set(counts[:3])) > 1, "the inputs were meant to change the number of queries"
