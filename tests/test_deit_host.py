"""Pins for the DeiT-level CPU restatement (oracle/torch_ref.py: deit_dge_forward, block_forward with extra
tokens).  No GPU needed.

Two independent statements hold it in place:
  * with every region routed to the finest split a DGE block IS a standard pre-norm transformer block, so the whole
    model must equal a dense ViT assembled from torch library modules on the same state dict (patch embedding
    unfold order, class / distillation tokens, positional embedding, final LayerNorm on the right rows, heads);
  * with a mixed gate, every token's output is the output of the one query whose window covers it: computed here
    token by token from the window definition (vtpack/layers/dge.py:61-112, vtpack/models/dge/deit_dge.py:123-130)
    in float64, without the patch list, the packed order or the gather / scatter functions of the restatement.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import torch_ref


def _tiny_vit(**kw):
    from vtpack_amd.models.dge.deit_dge import VisionTransformer
    torch.manual_seed(kw.pop("seed", 0))
    args = dict(img_size=64, patch_size=8, embed_dim=48, depth=3, num_heads=3, mlp_ratio=2, qkv_bias=True,
                num_classes=10, split_sizes=[4, 2, 1])
    args.update(kw)
    m = VisionTransformer(**args).eval()
    with torch.no_grad():      # every parameter away from its init value, so that a skipped one is visible
        for name, p in m.named_parameters():
            if p.is_floating_point():
                p.add_(torch.randn_like(p) * (0.1 if p.dim() > 1 else 0.3))
    return m


def _dense_block(blk, x):
    B, N, C = x.shape
    h = blk.attn.num_heads
    d = C // h
    xl = blk.norm1(x)
    q = blk.attn.q(xl).reshape(B, N, h, d).transpose(1, 2)
    kv = blk.attn.kv(xl).reshape(B, N, 2, h, d)
    att = F.scaled_dot_product_attention(q, kv[:, :, 0].transpose(1, 2), kv[:, :, 1].transpose(1, 2))
    y = x + blk.attn.proj(att.transpose(1, 2).reshape(B, N, C))
    return y + blk.mlp(blk.norm2(y))


@pytest.mark.parametrize("variant", ["cls", "distilled", "representation", "no_cls", "no_head"])
def test_deit_restatement_all_fine_matches_dense_vit(variant):
    kw = {"cls": {}, "distilled": {"distilled": True}, "representation": {"representation_size": 24},
          "no_cls": {"cls_token": False}, "no_head": {"num_classes": 0}}[variant]
    m = _tiny_vit(**kw)
    with torch.no_grad():
        for name, p in m.named_parameters():
            if name.endswith("router.gate.bias"):
                p.copy_(torch.tensor([60.0, -60.0, -60.0]))           # the finest split always wins
    sd = torch_ref.float_state_dict(m)
    img = torch.randn(3, 3, 64, 64)
    traces = []
    got = torch_ref.deit_dge_forward(sd, img, 3, 3, patch=8, traces=traces)
    extra = {"cls": 1, "distilled": 2, "representation": 1, "no_cls": 0, "no_head": 1}[variant]
    for tr in traces:
        assert tr["lengths"].tolist() == [extra + 64] * 3

    with torch.no_grad():
        conv = torch.nn.Conv2d(3, 48, 8, stride=8)
        conv.load_state_dict({"weight": sd["patch_embed.proj.weight"], "bias": sd["patch_embed.proj.bias"]})
        x = conv(img).flatten(2).transpose(1, 2)
        if variant == "distilled":
            x = torch.cat((m.cls_token.expand(3, -1, -1), m.dist_token.expand(3, -1, -1), x), dim=1)
        elif variant != "no_cls":
            x = torch.cat((m.cls_token.expand(3, -1, -1), x), dim=1)
        x = x + m.pos_embed
        for blk in m.blocks:
            x = _dense_block(blk, x)
        x = m.norm(x)
        if variant == "distilled":
            want = (m.head(x[:, 0]) + m.head_dist(x[:, 1])) / 2
        elif variant == "no_cls":
            want = m.head(x.mean(dim=1))
        elif variant == "representation":
            want = m.head(torch.tanh(m.pre_logits.fc(x[:, 0])))
        else:
            want = m.head(x[:, 0])
    assert got.shape == want.shape
    assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max())
    # the counterpart's own module composition (training-free layer path is GPU only) agrees on the variant's shape
    assert got.shape[-1] == (48 if variant == "no_head" else 10)


def _brute_force_block(sd, x, idx, heads, splits, extra, H, W, eps=1e-6):
    """Output of one DGE block, token by token, float64.  For token t of sample b: find its window from the gate
    index of its region, average the window, run that single query through attention over all tokens of the sample
    and the MLP, add (query output - query input) to x[b, t]."""
    p = lambda k: sd[k].double()  # noqa: E731
    B, N, C = x.shape
    d = C // heads
    R = max(splits)
    x = x.double()
    ln = lambda t, n: F.layer_norm(t, (C,), p(n + ".weight"), p(n + ".bias"), eps)  # noqa: E731
    out = torch.empty_like(x)
    counts = []
    for b in range(B):
        xl = ln(x[b], "norm1")
        kv = F.linear(xl, p("attn.kv.weight"), p("attn.kv.bias"))
        k, v = kv[:, :C], kv[:, C:]                                           # channel = head*d + j
        seen = set()
        for t in range(N):
            if t < extra:
                win = [t]
                seen.add(("e", t))
            else:
                y, xx = divmod(t - extra, W)
                step = R // splits[int(idx[b, y // R, xx // R])]
                y0, x0 = y // step * step, xx // step * step
                win = [(y0 + dy) * W + x0 + dx + extra for dy in range(step) for dx in range(step)]
                seen.add((y0, x0, step))
            comp = x[b, win].mean(dim=0)
            q = F.linear(ln(comp, "norm1"), p("attn.q.weight"), p("attn.q.bias"))
            o = torch.empty(C, dtype=torch.float64)
            for a in range(heads):
                sl = slice(a * d, (a + 1) * d)
                s = (k[:, sl] @ q[sl]) * d ** -0.5
                w = torch.exp(s - s.max())
                o[sl] = (w / w.sum()) @ v[:, sl]
            q1 = comp + F.linear(o, p("attn.proj.weight"), p("attn.proj.bias"))
            hdn = F.linear(ln(q1, "norm2"), p("mlp.fc1.weight"), p("mlp.fc1.bias"))
            hdn = 0.5 * hdn * (1.0 + torch.erf(hdn / 2 ** 0.5))
            q2 = q1 + F.linear(hdn, p("mlp.fc2.weight"), p("mlp.fc2.bias"))
            out[b, t] = x[b, t] + (q2 - comp)
        counts.append(len(seen))
    return out, counts


@pytest.mark.parametrize("extra,H,W", [(1, 8, 8), (2, 8, 8), (0, 4, 12)])
def test_block_restatement_mixed_gate_against_per_token_brute_force(extra, H, W):
    from vtpack_amd.models.dge.deit_dge import Block
    torch.manual_seed(3 + extra)
    C, heads, B = 24, 3, 2
    splits = [4, 2, 1]
    blk = Block(C, heads, mlp_ratio=2, qkv_bias=True, norm_layer=lambda n: torch.nn.LayerNorm(n, eps=1e-6),
                split_sizes=splits).eval()
    with torch.no_grad():
        for prm in blk.parameters():
            if prm.is_floating_point():
                prm.copy_(torch.randn_like(prm) * (0.3 if prm.dim() > 1 else 0.5))
    sd = torch_ref.float_state_dict(blk)
    x = torch.randn(B, extra + H * W, C)
    nreg = B * (H // 4) * (W // 4)
    idx = torch.from_numpy(np.random.RandomState(extra).permutation(np.arange(nreg) % 3).astype(np.int64))
    idx = idx.reshape(B, H // 4, W // 4)
    assert len(set(idx.reshape(-1).tolist())) == 3                           # a truly mixed gate
    tr = {}
    got = torch_ref.block_forward(sd, "", x, heads, indices=idx, size=(H, W), trace=tr)
    want, counts = _brute_force_block(sd, x, idx, heads, splits, extra, H, W)
    assert tr["lengths"].tolist() == counts                                  # distinct windows = queries per sample
    assert float((got.double() - want).abs().max()) <= 2e-5 * float(want.abs().max())
    # the same with the gate given as logits: argmax with the lowest index on ties (torch.argmax semantics)
    gate = F.one_hot(idx, 3).float()
    again = torch_ref.block_forward(sd, "", x, heads, gate=gate, size=(H, W))
    assert torch.equal(again, got)


def test_router_logits_restatement_against_loop():
    """router_gate (vtpack/layers/dge.py:145-150) against an explicit mean over each region's tokens."""
    torch.manual_seed(0)
    B, H, W, C, extra = 2, 8, 12, 16, 1
    x = torch.randn(B, extra + H * W, C)
    w, bias = torch.randn(3, C), torch.randn(3)
    got = torch_ref.router_gate(x, H, W, w, bias, 4)
    for b in range(B):
        for ry in range(H // 4):
            for rx in range(W // 4):
                toks = [extra + (ry * 4 + dy) * W + rx * 4 + dx for dy in range(4) for dx in range(4)]
                want = x[b, toks].double().mean(0) @ w.double().T + bias.double()
                assert float((got[b, ry, rx].double() - want).abs().max()) < 1e-5
