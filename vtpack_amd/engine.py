"""Fused inference path of one DGE transformer block: every step on libvtdge kernels.

What `Block.forward` of the reference does with ~30 library launches and one device->host copy
(vtpack/models/dge/deit_dge.py:123-130) becomes 13 kernel launches on the caller's stream with the
packed query count kept in device memory: buffers are sized for the worst case (one query per
token) and every packed kernel reads the live row count itself.  Nothing here synchronises, so the
whole forward can be captured into a HIP graph.
"""
import torch

from . import ops


def block_forward(block, x, H, W, gate=None):
    """x [B, N, C] -> [B, N, C] for a `vtpack_amd.models.dge.deit_dge.Block` in eval mode.

    `gate` [B, Hr, Wr, S] overrides the router's logits (used by the parity tests).
    """
    dge, attn, mlp = block.dge, block.attn, block.mlp
    B, N, C = x.shape
    extra = N - H * W
    R = dge.region_size
    x = x.contiguous()

    if gate is None:
        gate, indices = ops.router(x, dge.router.gate.weight, dge.router.gate.bias, H, W, R)
    else:
        indices = gate.argmax(dim=-1)
    cap = B * N
    patches, offsets, lengths = ops.index_to_patch(indices, dge.splits, R, extra, capacity=cap)
    rows_dev = offsets[B:]

    n1, n2 = block.norm1, block.norm2
    comp, comp_ln = ops.compress(x, patches, W, extra, rows_dev=rows_dev, rows=cap, ln_weight=n1.weight,
                                 ln_bias=n1.bias, ln_eps=n1.eps)
    x_ln = ops.layernorm(x, n1.weight, n1.bias, n1.eps)

    q = ops.linear(comp_ln, attn.q.weight, attn.q.bias, rows_dev=rows_dev)
    kv = ops.linear(x_ln, attn.kv.weight, attn.kv.bias)                       # [B, N, 2C] = [B, N, 2, h, d]
    o = ops.sparse_attention(q, kv[:, :, :C], kv[:, :, C:], offsets, attn.scale, attn.num_heads, N)
    q1 = ops.linear(o, attn.proj.weight, attn.proj.bias, residual=comp, rows_dev=rows_dev)

    q1_ln = ops.layernorm(q1, n2.weight, n2.bias, n2.eps, rows_dev=rows_dev)
    hid = ops.linear(q1_ln, mlp.fc1.weight, mlp.fc1.bias, act="gelu", rows_dev=rows_dev)
    q2 = ops.linear(hid, mlp.fc2.weight, mlp.fc2.bias, residual=q1, rows_dev=rows_dev)

    out = ops.decompress(q2, patches, x, W, extra, add_ref=True, sub=comp, rows_dev=rows_dev, rows=cap)

    dge.states.update({"comp": comp, "input": x, "patches": patches, "batches": None, "batches_device": lengths,
                       "offsets_device": offsets, "gate": gate, "size": (H, W), "num_extra_tokens": extra,
                       "queries": q2})
    return out
