"""Fused inference path of one DGE transformer block: every step on libvtdge kernels.

What `Block.forward` of the reference does with ~30 library launches and one device->host copy
(vtpack/models/dge/deit_dge.py:123-130) becomes six kernel launches on the caller's stream where the weight-stationary
and region kernels apply (bf16, 384 channels: key/value + query projection, attention, output projection, fc1, fc2,
and a scatter-back that also routes and packs the next block), nine on two streams joined before attention
elsewhere, with the packed query count kept in device memory: buffers are sized for the worst case (one query per
token) and every packed kernel reads the live row count itself.  Nothing here synchronises, so the whole forward can
be captured into a HIP graph.
"""
import torch

from . import ops
from .layers.dge import Deferred

# Where the block runs on two streams, it has two independent chains before attention: the routing chain (router -> index->patch -> compress ->
# q projection: small, latency-bound launches) and the key/value chain (LayerNorm of all tokens -> kv projection:
# the largest GEMM).  They are issued on two HIP streams of equal (default) priority and joined before attention,
# in eager mode and inside a captured graph alike.
_side_streams = {}
OVERLAP = True          # module switch (benchmarks turn it off to time kernels one at a time)
# The scatter-back of a block can also write the next block's first LayerNorm (one kernel less, 50 MB less read per
# block).  Off by default: that LayerNorm runs on the second stream next to the routing chain and costs nothing on
# the critical path, while the fused scatter-back is on it and slower (measured -4 % end to end at the headline
# config); useful when `OVERLAP` is off.
FUSE_NEXT_NORM = False
# The router reads every spatial token anyway and can write the block's first LayerNorm of all tokens on the way
# (one pass over x less, one kernel less).  Off by default as well: one wave then loads, normalises and stores a
# whole region with nothing to overlap the three phases (30 us against 22 us for the two kernels side by side at the
# headline config), and both chains of the block wait for it.
FUSE_ROUTER_NORM = False
# The scatter-back of a block can route the next block on the tokens it has just written (by region instead of by
# packed row: `vtdge_decompress_router`): the next block's router kernel and its pass over x disappear, and with it
# the first kernel of the routing chain, the longer of the two chains.  On by default (same bits as the two kernels).
FUSE_NEXT_ROUTER = True
# The two LayerNorms of a block folded into the Linears that consume them (norm1 -> kv, norm2 -> fc1): the Linear
# takes the raw rows and a 32-byte statistics record per row, so no normalised copy of the tokens is written or read.
# Taken where the weight-stationary kernel applies (bf16, 384 channels, 2048 rows or more, no spatial reduction).
FOLD_NORMS = True
# The patch embedding read straight from the images, position embedding added in its epilogue (`vtdge_patch_embed`),
# instead of an unfolded copy of the images, a Linear, a copy into the token tensor and an addition.
FUSE_PATCH_EMBED = True
# Which of the two chains at the head of a block runs on the second stream.  The one that finishes last should sit
# on the caller's stream, where attention follows it without a wait across queues: the key/value Linear covers all
# B N tokens whatever the router decides, the routing chain only the queries, so in most layers the Linear is the
# longer of the two (measured: +0.5 % end to end against the Linear on the second stream).
ROUTING_ON_SIDE = True
# The q Linear issued behind the join, on the caller's stream, instead of at the end of the routing chain: the chain
# (index->patch, compress) then ends before the key/value Linear does, and the wait across queues that attention would
# otherwise make for the chain's last kernel is over by the time the caller's stream reaches it.
Q_AFTER_JOIN = True
# index->patch and compress as one kernel that works by region (`vtdge_compress_regions`): the routing chain loses
# its first, latency-bound kernel, and with FOLD_NORMS the q Linear takes norm1 folded in (statistics records of the
# packed rows instead of their normalised copy).  Taken where the kernel applies (regions of 4, rows of 264 to 512
# channels in bf16).
REGION_COMPRESS = True
# A kernel of the routing chain can only run beside the key/value Linear where that leaves it registers: the
# weight-stationary Linear fills every SIMD with two waves of 216 registers, so `compress` gets one wave per SIMD and
# finishes 10 - 20 us after the Linear instead of under it, and the fork and the join of the two streams cost 5 and
# 9.5 us of idle queue each.  Where both kernels apply (the 384-channel bf16 models) the block therefore runs on ONE
# stream, routing chain first (it reads the tokens the scatter-back has just written): measured +1 % end to end
# against two streams, and no second queue in the captured graph.
SERIAL_BESIDE_WEIGHT_STATIONARY = True
ROUTING_FIRST = True
Q_BEFORE_KV = True
# On one stream the key/value Linear and the q Linear (both with norm1 folded in) go out as ONE launch
# (`vtdge_linear_layernorm_pair`): alone the q Linear has three or four tiles per workgroup behind the fixed cost of
# fetching its weights.
PAIR_KV_Q = True
# The first block of a model has no scatter-back before it to route it and to leave the statistics of its tokens:
# one kernel does both (`vtdge_router_stats`) instead of a router and a statistics pass, and stores the class-token
# rows on the way.
ROUTER_STATS = True
# `vtdge_compress_regions` leaves every region's first packed row for the scatter-back of the same block, which then
# needs no sum over the gate indices before it can start on its rows.
REGION_ROWS = True
# The scatter-back also packs the next block's queries (`vtdge_decompress_router_compress`): the wave that has just
# written a region's tokens and routed it reads them back from L2 and writes the next block's packed rows, their
# records, descriptors and offsets, so that `vtdge_compress_regions` runs for a model's first block only.
PACK_NEXT = True


def _side_stream(device, slot=0):
    s = _side_streams.get((device, slot))
    if s is None:
        s = _side_streams[(device, slot)] = torch.cuda.Stream(device=device)
    return s


def prepare(model):
    """Drop every derived copy of the model's weights (packed Linear weights, channels-last convolution weights) and
    make the packed ones again now.  Derived copies are otherwise made on first use and refreshed whenever a weight's
    storage, dtype, device or version counter changes; call this after writing weights in a way torch does not count
    (`p.data.copy_(...)`, `p.data.mul_(...)`) and, optionally, before capturing a graph so that no packing kernel lands
    in the capture."""
    ops.invalidate_packed(model)
    if getattr(model, "_vtdge_front", None) is not None:
        object.__setattr__(model, "_vtdge_front", None)
    for mod in model.modules():
        if hasattr(mod, "_vtdge_khwc"):
            mod._vtdge_khwc = None
        if isinstance(mod, torch.nn.Linear) and mod.weight.is_cuda and mod.weight.dtype == torch.bfloat16:
            ops.packed_weight(mod.weight)
        # a block's LayerNorms folded into the Linears behind them (see FOLD_NORMS)
        if FOLD_NORMS and all(hasattr(mod, name) for name in ("norm1", "norm2", "attn", "mlp")):
            for norm, lin in ((mod.norm1, getattr(mod.attn, "kv", None)), (mod.norm1, getattr(mod.attn, "q", None)),
                              (mod.norm2, getattr(mod.mlp, "fc1", None))):
                w = getattr(lin, "weight", None)
                if (w is not None and w.is_cuda and w.dtype == torch.bfloat16 and w.shape[1] == 384
                        and w.shape[0] % 384 == 0 and w.shape[0] <= 3072):
                    ops.folded_weight(w, lin.bias, norm.weight, norm.bias)
    return model


def _khwc_weight(conv):
    """Conv2d weight [O, C, kh, kw] as a Linear weight over channels-last patches: [O, kh*kw*C] (see `prepare` for
    when the cached copy is refreshed)."""
    w = conv.weight
    key = (w.data_ptr(), w._version, w.dtype, w.device)
    cached = getattr(conv, "_vtdge_khwc", None)
    if cached is None or cached[0] != key:
        flat = w.detach().permute(0, 2, 3, 1).reshape(w.shape[0], -1).contiguous()
        conv._vtdge_khwc = cached = (key, flat)
    return cached[1]


def tokens_to_patches(x, H, W, k):
    """Channels-last tokens [B, H*W, C] -> non-overlapping k x k patches [B*(H/k)*(W/k), k*k*C] (one copy)."""
    B, _, C = x.shape
    return x.reshape(B, H // k, k, W // k, k, C).permute(0, 1, 3, 2, 4, 5).reshape(B * (H // k) * (W // k), k * k * C)


def _strided_conv(x, H, W, k, conv):
    """Conv2d(k, stride k) over the channels-last token grid x [B, H*W, C] -> [B*(H/k)*(W/k), O], as a Linear over
    the k x k blocks of tokens: read in place where the kernel takes the shape, else from a gathered copy."""
    w = _khwc_weight(conv)
    if FUSE_PATCH_EMBED and ops.fits_patch_linear(x, H, W, k, w, conv.bias):
        return ops.patch_linear(x, H, W, k, w, conv.bias)
    return ops.linear(tokens_to_patches(x, H, W, k), w, conv.bias)


def _key_value_source(attn, x_ln, H, W, extra):
    """Tokens the keys and values are projected from: LN1(x) itself, or, with spatial reduction
    (vtpack/models/dge/pvt_dge.py:83-87), LayerNorm(Conv2d(C, C, sr, stride sr)(LN1(x))) with the convolution run
    as a Linear over channels-last patches."""
    sr = getattr(attn, "sr_ratio", 1)
    if sr <= 1:
        return x_ln
    if extra:
        raise ValueError("spatial reduction needs a token grid without extra tokens")
    if H % sr or W % sr:
        raise ValueError(f"token grid {H}x{W} is not a multiple of the reduction ratio {sr}")
    B, _, C = x_ln.shape
    red = _strided_conv(x_ln, H, W, sr, attn.sr)
    return ops.layernorm(red, attn.norm.weight, attn.norm.bias, attn.norm.eps).view(B, -1, C)


def block_forward(block, x, H, W, gate=None, overlap=True, carry=None, next_block=None):
    """x [B, N, C] -> [B, N, C] for a DGE transformer block (`models.dge.deit_dge.Block` or
    `models.dge.pvt_dge.Block`) in eval mode.

    `gate` [B, Hr, Wr, S] overrides the router's logits (used by the parity tests).
    `overlap` issues the key/value chain and the routing chain on two streams, side by side.
    `next_block` is the block that runs next on this block's output (same token grid): the call then returns
    (out, carry), where `carry` holds what this block has already worked out for it - the next block's gate logits and
    indices from the scatter-back kernel (`FUSE_NEXT_ROUTER`), or its first LayerNorm (`FUSE_NEXT_NORM`) - to be
    passed to the next call as `carry`.
    """
    dge, attn, mlp = block.dge, block.attn, block.mlp
    B, N, C = x.shape
    extra = N - H * W
    R = dge.region_size
    x = x.contiguous()
    carry = carry or {}
    x_ln = carry.get("x_ln")
    routed = carry.get("routed") if gate is None else None

    n1, n2 = block.norm1, block.norm2
    fold1 = (FOLD_NORMS and x_ln is None and getattr(attn, "sr_ratio", 1) <= 1
             and ops.fits_linear_layernorm(x, attn.kv.weight))
    use_regions = REGION_COMPRESS and ops.fits_compress_regions(x, H, W, R, dge.router.split_sizes)
    overlap = overlap and OVERLAP and not (SERIAL_BESIDE_WEIGHT_STATIONARY and fold1 and use_regions)
    main = torch.cuda.current_stream(x.device)
    side = _side_stream(x.device, main.cuda_stream) if overlap else main
    swap = overlap and ROUTING_ON_SIDE

    front = carry.get("front")
    if (ROUTER_STATS and routed is None and gate is None and x_ln is None and fold1 and R == 4
            and not FUSE_ROUTER_NORM and ops.fits_scatter_stats(x)):
        # a model's first block: its router, the statistics records of all tokens for norm1 -> kv, the query counts
        # of its regions and, on the way, the class-token rows put in front of every sample, in one pass over x
        g0, i0, rec0, cnt0 = ops.router_stats(x, dge.router.gate.weight, dge.router.gate.bias, H, W, R, n1.eps,
                                              front_rows=front, splits=dge.splits if use_regions else None,
                                              clear=carry.get("clear"))
        routed = (g0, i0)
        carry = dict(carry, x_stats=rec0, counts=cnt0, clear=None)
    elif front is not None:
        x[:, :front.shape[0], :] = front
    if carry.get("clear") is not None:      # workspaces of the blocks' scatter-backs that no kernel has cleared yet
        carry["clear"].zero_()

    fuse_rn = (FUSE_ROUTER_NORM and gate is None and routed is None and x_ln is None
               and ops.fits_router_layernorm(x, R))
    if fuse_rn:
        gate, indices, x_ln = ops.router_layernorm(x, dge.router.gate.weight, dge.router.gate.bias, H, W, R,
                                                   n1.weight, n1.bias, n1.eps)

    def kv_chain():
        nonlocal x_ln
        if fold1:
            rec1 = carry.get("x_stats")
            if rec1 is None:
                rec1 = ops.layernorm_stats(x, n1.eps)
            return x, ops.linear_layernorm(x, rec1, attn.kv.weight, attn.kv.bias, n1.weight, n1.bias)
        if x_ln is None:
            x_ln = ops.layernorm(x, n1.weight, n1.bias, n1.eps)
        src = _key_value_source(attn, x_ln, H, W, extra)
        return src, ops.linear(src, attn.kv.weight, attn.kv.bias)             # [B, n, 2C] = [B, n, 2, h, d]

    cap = B * N
    placed = {}      # where compress_regions has put every region's rows, for the scatter-back of this block

    def routing_chain():
        """-> (gate, indices, patches, offsets, lengths, comp, LayerNorm(comp) or None, records of comp or None)"""
        g, idx = gate, None
        if routed is not None:
            g, idx = routed
        elif fuse_rn:
            idx = indices
        elif g is None:
            g, idx = ops.router(x, dge.router.gate.weight, dge.router.gate.bias, H, W, R)
        else:
            idx = g.argmax(dim=-1)
        packed = carry.get("packed") if routed is not None else None
        if packed is not None:
            # the previous block's scatter-back has packed this block's queries already
            if REGION_ROWS:
                placed["region_rows"], placed["cur_counts"] = packed["region_rows"], carry["counts"]
            return g, idx, packed["patches"], packed["offsets"], None, packed["comp"], None, packed["records"]
        if use_regions:
            # index->patch and compress in one kernel, by region; with the folded norm1 -> q it leaves the statistics
            # records of the packed rows instead of their normalised copy
            foldq = FOLD_NORMS and ops.fits_linear_layernorm(x, attn.q.weight)
            cnt = carry.get("counts") if routed is not None else None
            cmp_, rec, pat, off, lens, rrows = ops.compress_regions(
                x, idx, dge.splits, H, W, R, counts=cnt, stats_eps=n1.eps if foldq else None, capacity=cap,
                want_region_rows=True)
            if cnt is not None and REGION_ROWS:
                placed["region_rows"], placed["cur_counts"] = rrows, cnt
            ln = None if foldq else ops.layernorm(cmp_, n1.weight, n1.bias, n1.eps, rows_dev=off[B:])
            return g, idx, pat, off, lens, cmp_, ln, rec
        pat, off, lens = ops.index_to_patch(idx, dge.splits, R, extra, capacity=cap)
        cmp_, ln = ops.compress(x, pat, W, extra, rows_dev=off[B:], rows=cap, ln_weight=n1.weight, ln_bias=n1.bias,
                                ln_eps=n1.eps)
        return g, idx, pat, off, lens, cmp_, ln, None

    def q_linear():
        if comp_rec is not None:
            return ops.linear_layernorm(comp, comp_rec, attn.q.weight, attn.q.bias, n1.weight, n1.bias,
                                        rows_dev=rows_dev)
        return ops.linear(comp_ln, attn.q.weight, attn.q.bias, rows_dev=rows_dev)

    q = None
    if overlap:
        # the two chains side by side on two streams, joined before attention
        side.wait_stream(main)
        with torch.cuda.stream(main if swap else side):
            kv_src, kv = kv_chain()
        with torch.cuda.stream(side if swap else main):
            gate, indices, patches, offsets, lengths, comp, comp_ln, comp_rec = routing_chain()
            rows_dev = offsets[B:]
            if not Q_AFTER_JOIN:
                q = q_linear()
        main.wait_stream(side)
        crossing = ((gate, indices, patches, offsets, lengths, comp, comp_ln, comp_rec, q) if swap
                    else (x_ln, kv_src, kv))
        for t in crossing:
            if t is not None:
                t.record_stream(main)    # allocated on the side stream, consumed (and released) on the caller's
        if q is None:
            q = q_linear()
    else:
        # one stream: the routing chain, then the two Linears
        if not ROUTING_FIRST:
            kv_src, kv = kv_chain()
        gate, indices, patches, offsets, lengths, comp, comp_ln, comp_rec = routing_chain()
        rows_dev = offsets[B:]
        if PAIR_KV_Q and ROUTING_FIRST and fold1 and comp_rec is not None:
            # the key/value and the query projection as one launch, the grid shared out by their live rows
            rec1 = carry.get("x_stats")
            if rec1 is None:
                rec1 = ops.layernorm_stats(x, n1.eps)
            kv_src = x
            kv, q = ops.linear_layernorm_pair(x, rec1, attn.kv.weight, attn.kv.bias, comp, comp_rec, attn.q.weight,
                                              attn.q.bias, n1.weight, n1.bias, rows_dev1=rows_dev)
        else:
            if Q_BEFORE_KV:
                q = q_linear()
            if ROUTING_FIRST:
                kv_src, kv = kv_chain()
            if q is None:
                q = q_linear()
    o = ops.sparse_attention(q, kv[:, :, :C], kv[:, :, C:], offsets, attn.scale, attn.num_heads, N)
    fold2 = FOLD_NORMS and ops.fits_linear_layernorm(o, mlp.fc1.weight)
    if fold2 and ops.fits_linear_stats(o, attn.proj.weight):
        q1, rec2 = ops.linear(o, attn.proj.weight, attn.proj.bias, residual=comp, rows_dev=rows_dev, stats_eps=n2.eps)
    else:
        q1 = ops.linear(o, attn.proj.weight, attn.proj.bias, residual=comp, rows_dev=rows_dev)
        rec2 = ops.layernorm_stats(q1, n2.eps, rows_dev=rows_dev) if fold2 else None

    if fold2:
        hid = ops.linear_layernorm(q1, rec2, mlp.fc1.weight, mlp.fc1.bias, n2.weight, n2.bias, act="gelu",
                                   rows_dev=rows_dev)
    else:
        q1_ln = ops.layernorm(q1, n2.weight, n2.bias, n2.eps, rows_dev=rows_dev)
        hid = ops.linear(q1_ln, mlp.fc1.weight, mlp.fc1.bias, act="gelu", rows_dev=rows_dev)
    q2 = ops.linear(hid, mlp.fc2.weight, mlp.fc2.bias, residual=q1, rows_dev=rows_dev)

    handed = {}
    nxt = next_block.dge if next_block is not None else None
    if nxt is not None and FUSE_NEXT_NORM and ops.fits_decompress_layernorm(x):
        nn1 = next_block.norm1
        out, handed["x_ln"] = ops.decompress_layernorm(q2, patches, x, W, extra, nn1.weight, nn1.bias, nn1.eps,
                                                       sub=comp, rows_dev=rows_dev, rows=cap)
    elif nxt is not None and FUSE_NEXT_ROUTER and R == 4 and nxt.region_size == 4:
        nattn = next_block.attn
        want_stats = (FOLD_NORMS and getattr(nattn, "sr_ratio", 1) <= 1 and ops.fits_scatter_stats(x)
                      and ops.fits_linear_layernorm(x, nattn.kv.weight))
        want_counts = REGION_COMPRESS and ops.fits_compress_regions(x, H, W, 4, nxt.router.split_sizes)
        # the next block's queries too, where that block takes them with their records (norm1 folded into q) on one
        # stream, as this one does
        pack = (PACK_NEXT and want_stats and want_counts and fold1 and use_regions and not overlap
                and ops.fits_pack_next(x, H, W, 4, nxt.router.split_sizes)
                and ops.fits_linear_layernorm(x, nattn.q.weight))
        spaces = carry.get("workspaces")
        if pack:
            placed.update(pack_next=True, pack_eps=next_block.norm1.eps, capacity=cap,
                          workspace=spaces.pop() if spaces else None)
        res = ops.decompress_router(q2, indices, dge.splits, offsets, x, H, W, R, sub=comp,
                                    next_weight=nxt.router.gate.weight, next_bias=nxt.router.gate.bias,
                                    stats_eps=next_block.norm1.eps if want_stats else None,
                                    next_splits=nxt.splits if want_counts else None, **placed)
        out, ngate, nidx = res[:3]
        handed["routed"] = (ngate, nidx)
        if want_stats:
            handed["x_stats"] = res[3]
        if want_counts:
            handed["counts"] = res[4 if want_stats else 3]
        if pack:
            handed["packed"] = res[5]
        if spaces:
            handed["workspaces"] = spaces
    else:
        out = ops.decompress(q2, patches, x, W, extra, add_ref=True, sub=comp, rows_dev=rows_dev, rows=cap)

    # `states` as the reference's code reads it (vtpack/layers/dge.py:81-84): the host-side counts and the tensors cut
    # to the live rows are produced when they are read (one device->host copy per read, nothing cached: a graph replay
    # rewrites `lengths` without running this code); nothing is copied otherwise.
    came_packed = carry.get("packed") if lengths is None else None

    def live():
        if came_packed is not None and int(came_packed["workspace"][0]) != 0:
            raise RuntimeError("the scatter-back that packed this block's queries gave up waiting (see "
                               "vtdge_decompress_router_compress): rows are missing")
        return offsets[1:] - offsets[:-1] if lengths is None else lengths

    def batches():
        return live().cpu()

    def cut(t):
        return lambda: t[:int(live().sum())]

    dge.states.update({"comp": Deferred(cut(comp)), "input": x, "patches": Deferred(cut(patches)),
                       "batches": Deferred(batches),
                       "batches_device": Deferred(live) if lengths is None else lengths, "offsets_device": offsets,
                       "gate": gate, "size": (H, W), "num_extra_tokens": extra, "queries": Deferred(cut(q2))})
    if next_block is not None:
        return out, handed
    return out


def _run_blocks(blocks, x, H, W, front=None):
    """A chain of blocks on one token grid, each handing the next what it has already computed for it.  `front`
    [extra, C]: rows the first block stores as the extra tokens of every sample before anything reads them."""
    carry = {"front": front} if front is not None else {}
    R = blocks[0].dge.region_size if blocks else 0
    if (PACK_NEXT and len(blocks) > 1 and R == 4
            and ops.fits_pack_next(x, H, W, R, blocks[0].dge.router.split_sizes)):
        # one slice of workspace per scatter-back that packs the next block's queries, all cleared by the first
        # block's first kernel
        words = ops.pack_next_workspace_words(x.shape[0], H, W, R)
        spaces = torch.empty((len(blocks) - 1, words), dtype=torch.int64, device=x.device)
        carry["workspaces"], carry["clear"] = list(spaces.unbind(0)), spaces
    for i, blk in enumerate(blocks):
        if i + 1 < len(blocks):
            x, carry = block_forward(blk, x, H, W, carry=carry, next_block=blocks[i + 1])
        else:
            x = block_forward(blk, x, H, W, carry=carry)
    return x


def _front_rows(model, front):
    """[extra, C]: the class (and distillation) token plus its row of the position table - what the reference puts
    in front of every sample's patch tokens (deit_dge.py:270-277).  The same for every sample and every call: made
    once per set of parameter versions and kept on the model."""
    parts = front + [model.pos_embed]
    key = tuple((t.data_ptr(), t._version, t.dtype, t.device) for t in parts)
    cached = getattr(model, "_vtdge_front", None)
    if cached is None or cached[0] != key:
        with torch.no_grad():
            rows = (torch.cat([t.detach() for t in front], dim=1) + model.pos_embed.detach()[:, :len(front), :])[0]
        cached = (key, rows.contiguous())
        object.__setattr__(model, "_vtdge_front", cached)
    return cached[1]


def model_forward(model, images):
    """images [B, 3, S, S] -> logits for a `VisionTransformer` in eval mode, dense pieces included.

    The patch embedding (a stride-16 16x16 convolution, i.e. a Linear over the patches, read straight from the
    images, with the position embedding added on the way out), the final LayerNorm (only the class-token rows are
    needed) and the classifier run on the same libvtdge kernels; torch contributes only the few rows of the class
    tokens.  vtpack/models/dge/deit_dge.py:267-299.
    """
    pe = model.patch_embed
    B, Cin, S, _ = images.shape
    if tuple(images.shape[-2:]) != pe.img_size:
        raise ValueError(f"input {tuple(images.shape[-2:])} does not match the model's image size {pe.img_size}")
    P = pe.patch_size[0]
    G = S // P
    C = model.embed_dim
    front = [t for t in (model.cls_token, getattr(model, "dist_token", None)) if t is not None]
    if model.cls_token is None and front:
        raise ValueError("a distillation token needs a class token (deit_dge.py:270-275)")
    extra = len(front)
    if FUSE_PATCH_EMBED and ops.fits_patch_embed(images, pe.proj.weight, pe.proj.bias, model.pos_embed, P):
        # the convolution reads the images in place and adds the position embedding on its way out
        x = ops.patch_embed(images, pe.proj.weight, pe.proj.bias, model.pos_embed, P, extra)
        front_rows = _front_rows(model, front) if extra else None
    else:
        front_rows = None
        patches = images.reshape(B, Cin, G, P, G, P).permute(0, 2, 4, 1, 3, 5).reshape(B * G * G, Cin * P * P)
        x = torch.empty((B, extra + G * G, C), dtype=images.dtype, device=images.device)
        tok = ops.linear(patches, pe.proj.weight.reshape(C, Cin * P * P), pe.proj.bias)
        x[:, extra:, :] = tok.view(B, G * G, C)
        for e, t in enumerate(front):
            x[:, e:e + 1, :] = t
        x += model.pos_embed
    x = _run_blocks(list(model.blocks), x, G, G, front=front_rows)
    nrm = model.norm

    def head(lin, t):
        return ops.linear(t, lin.weight, lin.bias) if isinstance(lin, torch.nn.Linear) else t

    if extra == 0:      # no class token: the classifier sees the mean over all normalised tokens
        return head(model.head, ops.layernorm(x, nrm.weight, nrm.bias, nrm.eps).mean(dim=1))
    # only the rows of the extra tokens are needed after the last block
    feats = ops.layernorm_front_rows(x, extra, nrm.weight, nrm.bias, nrm.eps)
    if extra == 2:      # class + distillation token: the mean of the two classifiers (deit_dge.py:288-294)
        return (head(model.head, feats[:, 0]) + head(model.head_dist, feats[:, 1])) / 2
    cls = feats[:, 0]
    pre = getattr(model, "pre_logits", None)
    if isinstance(pre, torch.nn.Sequential):            # Linear + Tanh (deit_dge.py:198-204)
        cls = torch.tanh(ops.linear(cls, pre.fc.weight, pre.fc.bias))
    return head(model.head, cls)


def pvt_forward(model, images):
    """images [B, 3, S, S] -> logits (or the per-stage feature maps when the model has no classifier) for a
    `models.dge.pvt_dge.PyramidVisionTransformer` in eval mode.  vtpack/models/dge/pvt_dge.py:295-339.

    Tokens stay channels-last between stages: every stage's patch embedding (a stride-k k x k convolution) runs as
    a Linear over k x k patches gathered from the previous stage's token grid, followed by its LayerNorm.
    """
    B, Cin, Hi, Wi = images.shape
    x = None
    outputs = {}
    for i in range(model.num_stages):
        pe = getattr(model, f"patch_embed{i + 1}")
        pos = getattr(model, f"pos_embed{i + 1}")
        k = pe.patch_size[0]
        last = i == model.num_stages - 1
        tok = None
        if i == 0:
            H, W = Hi // k, Wi // k
            if (FUSE_PATCH_EMBED and not last and Hi == Wi and H * W == pe.num_patches
                    and ops.fits_patch_embed_norm(images, pe.proj.weight, k)):
                # convolution, the embedding's LayerNorm and the position embedding in one pass over the images
                x = ops.patch_embed_norm(images, pe.proj.weight, pe.proj.bias, pe.norm.weight, pe.norm.bias,
                                         pe.norm.eps, pos, k)
                C = x.shape[-1]
            else:
                pat = images[:, :, :H * k, :W * k].reshape(B, Cin, H, k, W, k).permute(0, 2, 4, 1, 3, 5)
                tok = ops.linear(pat.reshape(B * H * W, Cin * k * k),
                                 pe.proj.weight.reshape(pe.proj.weight.shape[0], -1), pe.proj.bias)
        else:
            if H % k or W % k:
                raise ValueError(f"token grid {H}x{W} is not a multiple of the stage's patch size {k}")
            tok = _strided_conv(x, H, W, k, pe.proj)
            H, W = H // k, W // k
        if tok is None:
            pass
        elif not last:
            # the patch embedding's norm and `+ pos_embed` in one pass
            C = tok.shape[-1]
            x = ops.layernorm(tok, pe.norm.weight, pe.norm.bias, pe.norm.eps,
                              add=model._get_pos_embed(pos, pe, H, W)).view(B, H * W, C)
        else:
            C = tok.shape[-1]
            tok = ops.layernorm(tok, pe.norm.weight, pe.norm.bias, pe.norm.eps).view(B, H * W, C)
        if last:
            x = torch.empty((B, 1 + H * W, C), dtype=tok.dtype, device=tok.device)
            x[:, 1:, :] = tok
            x[:, :1, :] = model.cls_token
            if H * W != pe.num_patches:
                pos = torch.cat((pos[:, :1], model._get_pos_embed(pos[:, 1:], pe, H, W)), dim=1)
            x += pos
        x = _run_blocks(list(getattr(model, f"block{i + 1}")), x, H, W)
        if not last:
            outputs[f"res{i + 2}"] = x.view(B, H, W, C)
        elif model.num_classes == 0:
            outputs[f"res{i + 2}"] = x[:, 1:].reshape(B, H, W, C)
    if model.num_classes == 0:
        return {name: t.permute(0, 3, 1, 2).contiguous() for name, t in outputs.items()}
    cls = ops.layernorm(x[:, 0, :], model.norm.weight, model.norm.bias, model.norm.eps)
    return ops.linear(cls, model.head.weight, model.head.bias)
