"""PyTorch-CPU restatement of the DGE query path at block and model level.  TEST INFRASTRUCTURE ONLY.

The reference has no CPU implementation of its native operators (its extension is CUDA only), so
"the reference's PyTorch CPU path" is this file: the reference's Python control flow
(vtpack/layers/dge.py, vtpack/models/dge/deit_dge.py) with every `_C` call replaced by the plain
torch statement of the same arithmetic.  It works directly on a state dict with the reference's
key names, so the same weights drive it and the HIP path.

What pins it: the operator-level functions are checked against oracle/dge_oracle.c (itself pinned
by closed forms, see its header) in tests/test_oracle_pins.py; the dense pieces are torch library
routines (F.layer_norm, F.linear, F.gelu, F.conv2d, softmax).  The compositions are pinned too:
deit_dge_forward with an all-fine router equals a dense ViT built from F.conv2d, nn.LayerNorm and
F.scaled_dot_product_attention on the same state dict (also distilled / pre-logits / no class token),
and block_forward with an extra token and a mixed gate equals a brute-force loop in which every
token takes the output of the query that covers it (tests/test_deit_host.py); pvt_dge_forward has the
same pins in tests/test_pvt_host.py.
"""
import math

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------- operators
def router_gate(x, H, W, weight, bias, region_size):
    """vtpack/layers/dge.py:145-150 on x [B, extra+H*W, C] -> gate logits [B, Hr, Wr, S]."""
    B, N, C = x.shape
    extra = N - H * W
    g = x[:, extra:, :].reshape(B, H, W, C).permute(0, 3, 1, 2)
    g = F.avg_pool2d(g, region_size, region_size).permute(0, 2, 3, 1)
    return F.linear(g, weight, bias)


def index_to_patch(indices, splits, region_size, extra):
    """Vectorised form of grained_sample.cu:302-345 + :146-196 -> (patches [L,4], lengths [B]) int64.

    Like the reference's host code, every sample owns 1 + Hr*Wr slots (slot 0 = the extra tokens)
    whose counts are prefix-summed; each slot then emits its rows."""
    B, Hr, Wr = indices.shape
    nslot = 1 + Hr * Wr
    ps = splits[indices].reshape(B, -1)                                         # [B, Hr*Wr]
    counts = torch.cat([torch.full((B, 1), extra, dtype=torch.int64), ps * ps], dim=1)
    lengths = counts.sum(1)
    flat = counts.reshape(-1)
    ends = flat.cumsum(0)
    slot = torch.repeat_interleave(torch.arange(B * nslot), flat)             # owning slot of every row
    j = torch.arange(int(ends[-1])) - (ends - flat)[slot]                       # index inside the slot
    b, s_in = slot // nslot, slot % nslot
    is_extra = s_in == 0
    r = (s_in - 1).clamp(min=0)
    p = torch.cat([torch.ones((B, 1), dtype=torch.int64), ps], dim=1).reshape(-1)[slot]
    step = region_size // p
    y0 = (r // Wr) * region_size + (j // p) * step
    x0 = (r % Wr) * region_size + (j % p) * step
    patches = torch.stack([b, torch.where(is_extra, -j - 1, y0), torch.where(is_extra, torch.zeros_like(j), x0),
                           torch.where(is_extra, torch.ones_like(j), step)], dim=1)
    return patches.to(torch.int64), lengths


def compress(x, patches, H, W, extra):
    """avg_pool2d-style statement of grained_sample.cu:31-69 (the reference's own dense form,
    vtpack/layers/grained_sample.py:130-139, sampled at the chosen patches)."""
    B, N, C = x.shape
    out = x.new_empty((patches.shape[0], C))
    b, y0, x0, sz = patches.unbind(1)
    is_extra = y0 < 0
    if is_extra.any():
        out[is_extra] = x[b[is_extra], -y0[is_extra] - 1]
    grid = x[:, extra:, :].reshape(B, H, W, C).permute(0, 3, 1, 2)
    for s in torch.unique(sz[~is_extra]).tolist():
        sel = (~is_extra) & (sz == s)
        pooled = F.avg_pool2d(grid, s, s) if s > 1 else grid          # [B,C,H/s,W/s]
        out[sel] = pooled[b[sel], :, y0[sel] // s, x0[sel] // s]
    return out


def token_to_row(patches, B, N, W, extra):
    """Inverse index of the patch list: for every token the packed row that covers it."""
    m = torch.full((B, N), -1, dtype=torch.int64)
    b, y0, x0, sz = patches.unbind(1)
    rows = torch.arange(patches.shape[0])
    is_extra = y0 < 0
    m[b[is_extra], -y0[is_extra] - 1] = rows[is_extra]
    for s in torch.unique(sz[~is_extra]).tolist():
        sel = (~is_extra) & (sz == s)
        for dy in range(s):
            for dx in range(s):
                m[b[sel], (y0[sel] + dy) * W + x0[sel] + dx + extra] = rows[sel]
    return m


def decompress(inp, patches, reference, H, W, extra, is_add_ref=True):
    """Index form of grained_sample.cu:71-144: out[b,t] = inp[row covering t] (+ reference[b,t])."""
    B, N, C = reference.shape
    m = token_to_row(patches, B, N, W, extra)
    if (m < 0).any():
        raise ValueError("patch list does not cover every token")
    out = inp[m.reshape(-1)].reshape(B, N, C)
    return out + reference if is_add_ref else out


def attention(q, k, v, lengths, scale):
    """Per-sample loop of batched_sparse_gemm.cu:267-301.  q [h,L,d]; k,v [h,B,n,d] -> [h,L,d]."""
    outs, off = [], 0
    for i, m in enumerate(lengths.tolist()):
        s = torch.matmul(q[:, off:off + m], k[:, i].transpose(-1, -2)) * scale
        outs.append(torch.matmul(torch.softmax(s, dim=-1), v[:, i]))
        off += m
    return torch.cat(outs, 1)


def sparse_gemm(a, b, a_lengths, b_lengths, ta, tb):
    """batched_sparse_gemm.cu:150-195: per-sample bmm over heads, cat on dim 1."""
    outs, sa, sb = [], 0, 0
    for la, lb in zip(a_lengths.tolist(), b_lengths.tolist()):
        ai, bi = a[:, sa:sa + la], b[:, sb:sb + lb]
        ai = ai.transpose(-1, -2) if ta else ai
        bi = bi.transpose(-1, -2) if tb else bi
        outs.append(torch.bmm(ai, bi))
        sa, sb = sa + la, sb + lb
    return torch.cat(outs, 1)


# ----------------------------------------------------------------------------- block / model
def block_forward(sd, prefix, x, num_heads, gate=None, indices=None, eps=1e-6, trace=None, size=None, sr_ratio=1,
                  sr_eps=1e-5):
    """vtpack/models/dge/deit_dge.py:123-130 and vtpack/models/dge/pvt_dge.py:134-140 (eval) for the block whose
    keys start with `prefix`.

    gate: optional logits injected in place of the router output.
    indices: optional gate indices forced on the block (teacher forcing), overriding both.
    trace: optional dict that receives every intermediate.
    size: (H, W) of the token grid (default: square, as deit_dge.py:125 assumes).
    sr_ratio: spatial reduction of the key/value tokens (pvt_dge.py:83-87): Conv2d(C, C, sr, stride sr) on the
        normalised token grid, then LayerNorm(eps = sr_eps, nn.LayerNorm's default).
    """
    p = lambda name: sd[prefix + name]  # noqa: E731
    B, N, C = x.shape
    H, W = size if size is not None else (int(math.sqrt(N)),) * 2
    extra = N - H * W
    splits = p("dge.splits").to(torch.int64)
    R = int(splits.max())
    if gate is None:
        gate = router_gate(x, H, W, p("dge.router.gate.weight"), p("dge.router.gate.bias"), R)
    if indices is None:
        indices = gate.argmax(dim=-1)
    patches, lengths = index_to_patch(indices, splits, R, extra)
    comp = compress(x, patches, H, W, extra)

    ln = lambda t, n: F.layer_norm(t, (C,), p(n + ".weight"), p(n + ".bias"), eps)  # noqa: E731
    d = C // num_heads
    q = F.linear(ln(comp, "norm1"), p("attn.q.weight"), p("attn.q.bias")).reshape(-1, num_heads, d).permute(1, 0, 2)
    kv_src = ln(x, "norm1")
    if sr_ratio > 1:
        grid = kv_src.permute(0, 2, 1).reshape(B, C, H, W)
        grid = F.conv2d(grid, p("attn.sr.weight"), p("attn.sr.bias"), stride=sr_ratio)
        kv_src = F.layer_norm(grid.reshape(B, C, -1).permute(0, 2, 1), (C,), p("attn.norm.weight"),
                              p("attn.norm.bias"), sr_eps)
    kv = F.linear(kv_src, p("attn.kv.weight"), p("attn.kv.bias"))
    kv = kv.reshape(B, -1, 2, num_heads, d).permute(2, 3, 0, 1, 4)
    att = attention(q, kv[0], kv[1], lengths, d ** -0.5).transpose(0, 1).reshape(-1, C)
    q1 = comp + F.linear(att, p("attn.proj.weight"), p("attn.proj.bias"))
    hid = F.gelu(F.linear(ln(q1, "norm2"), p("mlp.fc1.weight"), p("mlp.fc1.bias")))
    q2 = q1 + F.linear(hid, p("mlp.fc2.weight"), p("mlp.fc2.bias"))
    out = decompress(q2 - comp, patches, x, H, W, extra, True)
    if trace is not None:
        trace.update(gate=gate, indices=indices, patches=patches, lengths=lengths, comp=comp, attn=att, q1=q1,
                     q2=q2, out=out)
    return out


def deit_dge_forward(sd, images, num_heads, depth, patch=16, eps=1e-6, forced_indices=None, traces=None):
    """vtpack/models/dge/deit_dge.py:267-299 at inference.  images [B,3,S,S] -> logits.

    The variant is read off the state dict, as the reference's constructor fixes it (deit_dge.py:179-214):
    `cls_token` absent -> no extra token and the head sees the token mean; `dist_token` present -> two extra tokens
    and the mean of `head` and `head_dist`; `pre_logits.fc.*` present -> Linear + tanh before the head."""
    x = F.conv2d(images, sd["patch_embed.proj.weight"], sd["patch_embed.proj.bias"], stride=patch)
    x = x.flatten(2).transpose(1, 2)
    B = x.shape[0]
    if "cls_token" in sd:
        front = [sd["cls_token"].expand(B, -1, -1)]
        if "dist_token" in sd:
            front.append(sd["dist_token"].expand(B, -1, -1))
        x = torch.cat(front + [x], dim=1)
    x = x + sd["pos_embed"]
    for i in range(depth):
        tr = {} if traces is not None else None
        x = block_forward(sd, f"blocks.{i}.", x, num_heads, eps=eps, trace=tr,
                          indices=None if forced_indices is None else forced_indices[i])
        if traces is not None:
            traces.append(tr)
    C = x.shape[-1]
    x = F.layer_norm(x, (C,), sd["norm.weight"], sd["norm.bias"], eps)
    head = lambda name, t: F.linear(t, sd[name + ".weight"], sd[name + ".bias"]) if name + ".weight" in sd else t  # noqa: E731
    if "cls_token" not in sd:
        return head("head", x.mean(dim=1))
    if "dist_token" in sd:
        return (head("head", x[:, 0]) + head("head_dist", x[:, 1])) / 2
    x = x[:, 0]
    if "pre_logits.fc.weight" in sd:
        x = torch.tanh(F.linear(x, sd["pre_logits.fc.weight"], sd["pre_logits.fc.bias"]))
    return head("head", x)


def pvt_dge_forward(sd, images, num_heads, depths, sr_ratios, patch=4, eps=1e-6, embed_eps=1e-5, forced_indices=None,
                    traces=None):
    """vtpack/models/dge/pvt_dge.py:290-339 with a classifier.  images [B,3,S,S] -> logits.

    The positional embeddings must match the token grids (no interpolation branch).  forced_indices / traces are
    flat lists over all blocks in execution order.
    """
    B = images.shape[0]
    x = images
    nblk = 0
    last = len(depths) - 1
    for i, depth in enumerate(depths):
        pre = f"patch_embed{i + 1}."
        x = F.conv2d(x, sd[pre + "proj.weight"], sd[pre + "proj.bias"], stride=patch if i == 0 else 2)
        H, W = x.shape[2], x.shape[3]
        C = x.shape[1]
        x = F.layer_norm(x.flatten(2).transpose(1, 2), (C,), sd[pre + "norm.weight"], sd[pre + "norm.bias"], embed_eps)
        if i == last:
            x = torch.cat((sd["cls_token"].expand(B, -1, -1), x), dim=1)
        x = x + sd[f"pos_embed{i + 1}"]
        for j in range(depth):
            tr = {} if traces is not None else None
            x = block_forward(sd, f"block{i + 1}.{j}.", x, num_heads[i], eps=eps, trace=tr, size=(H, W),
                              sr_ratio=sr_ratios[i],
                              indices=None if forced_indices is None else forced_indices[nblk])
            nblk += 1
            if traces is not None:
                traces.append(tr)
        if i != last:
            x = x.reshape(B, H, W, C).permute(0, 3, 1, 2)
    C = x.shape[-1]
    x = F.layer_norm(x, (C,), sd["norm.weight"], sd["norm.bias"], eps)[:, 0]
    return F.linear(x, sd["head.weight"], sd["head.bias"])


def float_state_dict(module_or_sd):
    sd = module_or_sd if isinstance(module_or_sd, dict) else module_or_sd.state_dict()
    return {k: (v.detach().cpu().float() if v.is_floating_point() else v.detach().cpu()) for k, v in sd.items()}
