"""Thin tensor-level wrappers over the C ABI (include/vtdge.h).

Every function here only checks shapes, allocates outputs with torch and hands
raw device pointers plus the current HIP stream to libvtdge.  Row counts of
packed operands may stay on the device (`rows_dev`), so nothing in this module
synchronises with the GPU.
"""
import ctypes

import torch

from . import _lib
from ._lib import call, dtype_code, ptr, stream_ptr


def _need_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("vtdge operators run on the GPU only (got a CPU tensor); there is no CPU fallback")


def _contig(t):
    return t if t.is_contiguous() else t.contiguous()


def _check_like(x, **operands):
    """Every given operand must have x's dtype and device: the kernels read all of them through one dtype code, so a
    mismatch would make them read a buffer with the wrong element size (nn.Linear / nn.LayerNorm raise likewise)."""
    for name, t in operands.items():
        if t is None:
            continue
        if t.dtype != x.dtype:
            raise TypeError(f"{name} is {t.dtype} but the activation is {x.dtype}: cast the module or the input")
        if t.device != x.device:
            raise TypeError(f"{name} is on {t.device} but the activation is on {x.device}")


def _check_vector(name, t, n):
    if t is not None and tuple(t.shape) != (n,):
        raise ValueError(f"{name} has shape {tuple(t.shape)}, expected ({n},)")


def _check_router(weight, bias, C, S, extra, H, W, region_size):
    if tuple(weight.shape) != (S, C) or tuple(bias.shape) != (S,):
        raise ValueError(f"router weight {tuple(weight.shape)} / bias {tuple(bias.shape)} do not map {C} channels")
    if extra < 0 or H % region_size or W % region_size:
        raise ValueError(f"a {H}x{W} token grid with {extra} extra tokens does not tile into regions of "
                         f"{region_size}")


def router(x, weight, bias, H, W, region_size, want_gate=True):
    """AvgPool(R) -> Linear -> argmax on the spatial tokens of x [B, extra+H*W, C].

    Returns (gate [B,Hr,Wr,S] or None, indices int64 [B,Hr,Wr]).  vtpack/layers/dge.py:145-150, :75.
    """
    _need_gpu(x, weight, bias)
    x, weight, bias = _contig(x), _contig(weight), _contig(bias)
    B, N, C = x.shape
    S = weight.shape[0]
    extra = N - H * W
    _check_router(weight, bias, C, S, extra, H, W, region_size)
    Hr, Wr = H // region_size, W // region_size
    gate = torch.empty((B, Hr, Wr, S), dtype=x.dtype, device=x.device) if want_gate else None
    indices = torch.empty((B, Hr, Wr), dtype=torch.int64, device=x.device)
    weight, bias = weight.to(x.dtype), bias.to(x.dtype)
    call("vtdge_router", ptr(x), ptr(weight), ptr(bias), ptr(gate), ptr(indices), B, H, W, C,
         extra, region_size, S, dtype_code(x), stream_ptr(), tag=("router", C))
    return gate, indices


def fits_router_layernorm(x, region_size):
    """Whether the router can also write LayerNorm(x): region size 4 or 2, one 16-byte vector per lane and row."""
    return region_size in (2, 4) and x.shape[-1] * x.element_size() <= 64 * 16


def router_layernorm(x, weight, bias, H, W, region_size, ln_weight, ln_bias, ln_eps, want_gate=True):
    """`router` and LayerNorm of every token of x in one pass: (gate or None, indices, LayerNorm(x)).

    vtpack/layers/dge.py:145-150, :75 and norm1 of vtpack/models/dge/deit_dge.py:127."""
    _need_gpu(x, weight, bias, ln_weight, ln_bias)
    x, weight, bias = _contig(x), _contig(weight), _contig(bias)
    B, N, C = x.shape
    S = weight.shape[0]
    extra = N - H * W
    _check_router(weight, bias, C, S, extra, H, W, region_size)
    Hr, Wr = H // region_size, W // region_size
    gate = torch.empty((B, Hr, Wr, S), dtype=x.dtype, device=x.device) if want_gate else None
    indices = torch.empty((B, Hr, Wr), dtype=torch.int64, device=x.device)
    ln_out = torch.empty_like(x)
    weight, bias = weight.to(x.dtype), bias.to(x.dtype)
    call("vtdge_router_layernorm", ptr(x), ptr(weight), ptr(bias), ptr(gate), ptr(indices),
         ptr(_contig(ln_weight).to(x.dtype)), ptr(_contig(ln_bias).to(x.dtype)), float(ln_eps), ptr(ln_out), B, H, W,
         C, extra, region_size, S, dtype_code(x), stream_ptr(), tag=("router_layernorm", C, B * N))
    return gate, indices, ln_out


def index_to_patch(indices, splits, region_size, num_extra_tokens, capacity=None):
    """Device-only compaction: (patches [capacity,4], offsets [B+1], lengths [B]), all on the GPU."""
    _need_gpu(indices, splits)
    if indices.dtype != torch.int64 or splits.dtype != torch.int64 or indices.dim() != 3:
        raise TypeError("indices must be int64 [B, Hr, Wr] and splits int64")
    indices, splits = _contig(indices), _contig(splits)
    B, Hr, Wr = indices.shape
    if capacity is None:
        capacity = B * (num_extra_tokens + Hr * Wr * region_size * region_size)
    patches = torch.empty((capacity, 4), dtype=torch.int64, device=indices.device)
    offsets = torch.empty((B + 1,), dtype=torch.int64, device=indices.device)
    lengths = torch.empty((B,), dtype=torch.int64, device=indices.device)
    call("vtdge_index_to_patch", ptr(indices), ptr(splits), B, Hr, Wr, splits.numel(), region_size,
         num_extra_tokens, ptr(patches), capacity, ptr(offsets), ptr(lengths), stream_ptr(), tag=("index_to_patch",))
    return patches, offsets, lengths


def compress(x, patches, width, num_extra_tokens, rows_dev=None, rows=None, ln_weight=None, ln_bias=None,
             ln_eps=1e-6):
    """x [B,N,C] -> comp [rows,C] (and LayerNorm(comp) when ln_weight is given)."""
    _need_gpu(x, patches, ln_weight, ln_bias)
    x, patches = _contig(x), _contig(patches)
    B, N, C = x.shape
    _check_like(x, ln_weight=ln_weight, ln_bias=ln_bias)
    _check_vector("ln_weight", ln_weight, C)
    _check_vector("ln_bias", ln_bias, C)
    if (ln_weight is None) != (ln_bias is None):
        raise ValueError("the fused LayerNorm needs both its weight and its bias")
    ln_weight, ln_bias = (None, None) if ln_weight is None else (_contig(ln_weight), _contig(ln_bias))
    rows = patches.shape[0] if rows is None else rows
    out = torch.empty((rows, C), dtype=x.dtype, device=x.device)
    ln_out = torch.empty_like(out) if ln_weight is not None else None
    call("vtdge_compress", ptr(x), ptr(patches), ptr(rows_dev), rows, ptr(out), ptr(ln_out), ptr(ln_weight),
         ptr(ln_bias), float(ln_eps), B, N, C, width, num_extra_tokens, dtype_code(x), stream_ptr(),
         tag=("compress", ln_weight is not None, rows, C))
    return (out, ln_out) if ln_weight is not None else out


def decompress(inp, patches, reference, width, num_extra_tokens, add_ref=True, sub=None, rows_dev=None, rows=None,
               out=None):
    """Scatter (inp - sub) back over the tokens each patch covers, plus reference when add_ref."""
    _need_gpu(inp, patches, reference, sub)
    inp, patches, reference = _contig(inp), _contig(patches), _contig(reference)
    sub = None if sub is None else _contig(sub)
    B, N, C = reference.shape
    _check_like(inp, reference=reference, sub=sub, out=out)
    if inp.shape[-1] != C or (sub is not None and sub.shape != inp.shape):
        raise ValueError(f"packed rows {tuple(inp.shape)} / {None if sub is None else tuple(sub.shape)} do not match "
                         f"the reference's {C} channels")
    rows = patches.shape[0] if rows is None else rows
    if out is None:
        out = torch.empty((B, N, C), dtype=inp.dtype, device=inp.device)
    call("vtdge_decompress", ptr(inp), ptr(sub), ptr(patches), ptr(rows_dev), rows,
         ptr(reference) if add_ref else 0, ptr(out), B, N, C, width, num_extra_tokens, dtype_code(inp), stream_ptr(),
         tag=("decompress", sub is not None, bool(add_ref), C))
    return out


def decompress_layernorm(inp, patches, reference, width, num_extra_tokens, ln_weight, ln_bias, ln_eps=1e-6, sub=None,
                         rows_dev=None, rows=None):
    """Scatter (inp - sub) + reference back over the tokens, and the LayerNorm of the result: (out, LayerNorm(out))."""
    _need_gpu(inp, patches, reference, sub, ln_weight, ln_bias)
    inp, patches, reference = _contig(inp), _contig(patches), _contig(reference)
    sub = None if sub is None else _contig(sub)
    B, N, C = reference.shape
    _check_like(inp, reference=reference, sub=sub, ln_weight=ln_weight, ln_bias=ln_bias)
    _check_vector("ln_weight", ln_weight, C)
    _check_vector("ln_bias", ln_bias, C)
    if inp.shape[-1] != C or (sub is not None and sub.shape != inp.shape):
        raise ValueError("packed rows do not match the reference's channel count")
    ln_weight, ln_bias = _contig(ln_weight), _contig(ln_bias)
    rows = patches.shape[0] if rows is None else rows
    out = torch.empty((B, N, C), dtype=inp.dtype, device=inp.device)
    ln_out = torch.empty_like(out)
    call("vtdge_decompress_layernorm", ptr(inp), ptr(sub), ptr(patches), ptr(rows_dev), rows, ptr(reference), ptr(out),
         ptr(ln_out), ptr(ln_weight), ptr(ln_bias), float(ln_eps), B, N, C, width, num_extra_tokens, dtype_code(inp),
         stream_ptr(), tag=("decompress_ln", sub is not None, C))
    return out, ln_out


def region_counts_buffer(B, regions, device):
    """An uninitialised uint8 buffer for the per-region query counts `decompress_router` leaves for
    `compress_regions`, padded so that the reader's 16-byte loads stay inside it."""
    return torch.empty((-(-(B * regions) // 16) * 16,), dtype=torch.uint8, device=device)


def fits_compress_regions(x, H, W, region_size, split_sizes):
    """Whether `compress_regions` has a kernel: regions of 4 x 4 tokens split 1, 2 or 4 ways, a row of at most 64
    16-byte vectors (and more than 32: narrower rows are better served by the row-wise kernels, which give several
    rows to a wave), at most 65536 regions."""
    if x.dim() != 3 or x.dtype not in (torch.float32, torch.bfloat16) or region_size != 4:
        return False
    B, N, C = x.shape
    nvec = C * x.element_size() // 16
    return (x.is_cuda and H % 4 == 0 and W % 4 == 0 and N >= H * W and N - H * W <= 64
            and (C * x.element_size()) % 16 == 0 and 32 < nvec <= 64
            and set(int(s) for s in split_sizes) <= {1, 2, 4}
            and B * (H // 4) * (W // 4) <= 65536 and B * N < (1 << 24))


def compress_regions(x, indices, splits, H, W, region_size=4, counts=None, stats_eps=None, capacity=None,
                     want_patches=True, want_region_rows=False):
    """index_to_patch and compress in one kernel, by region: x [B, extra + H*W, C] and the gate indices [B, Hr, Wr]
    -> (comp [capacity, C], records or None, patches or None, offsets [B+1], lengths [B]).  `counts` is the uint8
    buffer a `decompress_router(..., next_splits=...)` has filled for these indices (optional: the kernel otherwise
    works the counts out from the indices); with `stats_eps` (bf16) the statistics records of the rows of comp are
    written for a `linear_layernorm` that takes comp next.  comp, patches, offsets and lengths equal those of
    `index_to_patch` + `compress` bit for bit.  With `want_region_rows` a sixth value: int32 [B * regions], the first
    packed row of every region (for the `decompress_router` of the same block).  vtpack/layers/dge.py:76-79."""
    _need_gpu(x, indices, splits, counts)
    x, indices, splits = _contig(x), _contig(indices), _contig(splits)
    if indices.dtype != torch.int64 or splits.dtype != torch.int64 or indices.dim() != 3:
        raise TypeError("indices must be int64 [B, Hr, Wr] and splits int64")
    B, N, C = x.shape
    extra = N - H * W
    if extra < 0 or H % region_size or W % region_size or tuple(indices.shape) != (B, H // region_size, W // region_size):
        raise ValueError(f"gate indices {tuple(indices.shape)} do not match a {H}x{W} grid of regions of {region_size}")
    regions = (H // region_size) * (W // region_size)
    if counts is not None and (counts.dtype != torch.uint8 or counts.numel() < -(-(B * regions) // 16) * 16):
        raise ValueError("counts must be a uint8 buffer from region_counts_buffer")
    if stats_eps is not None and x.dtype != torch.bfloat16:
        raise TypeError("compress_regions: records exist for bfloat16 rows only")
    if capacity is None:
        capacity = B * N
    if capacity < B * N:
        raise ValueError("compress_regions writes without bounds checks on comp: capacity must be at least B * N")
    comp = torch.empty((capacity, C), dtype=x.dtype, device=x.device)
    rec = torch.empty((capacity, 16), dtype=torch.bfloat16, device=x.device) if stats_eps is not None else None
    patches = torch.empty((capacity, 4), dtype=torch.int64, device=x.device) if want_patches else None
    offsets = torch.empty((B + 1,), dtype=torch.int64, device=x.device)
    lengths = torch.empty((B,), dtype=torch.int64, device=x.device)
    region_rows = torch.empty((B * regions,), dtype=torch.int32, device=x.device) if want_region_rows else None
    call("vtdge_compress_regions", ptr(x), ptr(indices), ptr(splits), ptr(counts), ptr(comp), ptr(rec),
         float(stats_eps if stats_eps is not None else 0.0), ptr(patches), capacity, ptr(offsets), ptr(lengths),
         ptr(region_rows), B, H, W, C, extra, region_size, splits.numel(), dtype_code(x), stream_ptr(),
         tag=("compress_regions", rec is not None, C, counts is not None))
    if want_region_rows:
        return comp, rec, patches, offsets, lengths, region_rows
    return comp, rec, patches, offsets, lengths


def pack_next_workspace_words(B, H, W, region_size=4):
    """64-bit words of workspace `decompress_router(..., pack_next=True)` needs."""
    return int(_lib.load().vtdge_decompress_router_compress_workspace(B, H, W, region_size)) // 8


def fits_pack_next(x, H, W, region_size, split_sizes):
    """True when `decompress_router(..., pack_next=True)` takes these tokens: what `compress_regions` and the
    statistics records need, and whole workgroups of four regions."""
    B = x.shape[0]
    return (fits_compress_regions(x, H, W, region_size, split_sizes) and fits_scatter_stats(x)
            and (B * (H // region_size) * (W // region_size)) % 4 == 0)


def decompress_router(inp, indices, splits, offsets, reference, H, W, region_size, sub=None, next_weight=None,
                      next_bias=None, want_gate=True, stats_eps=None, next_splits=None, region_rows=None,
                      cur_counts=None, pack_next=False, pack_eps=None, capacity=None, workspace=None):
    """Scatter (inp - sub) + reference back over the tokens by region, and route the NEXT block on the result:
    -> (out, next_gate or None, next_indices or None), and with `stats_eps` (a LayerNorm's eps; bf16 rows of 264 to
    512 channels) a fourth value: the statistics records of the rows of `out` for `linear_layernorm`; with `next_splits`
    (the next block's split sizes, int64 on the device) one more at the end: the uint8 query counts of the next block's
    regions for `compress_regions`.  `indices` [B, Hr, Wr] are this block's gate indices, `offsets` [B+1] the prefix of
    its query counts; `region_rows` with `cur_counts` (from this block's `compress_regions` and the count bytes it
    read) spare the kernel adding a region's place up from them.  The three outputs equal decompress(...) and router(out, next_weight,
    next_bias) bit for bit.  vtpack/layers/dge.py:87-112 and, for the next block, :145-150, :75.

    `pack_next` (see `fits_pack_next`; needs stats_eps and next_splits): the kernel also packs the next block's
    queries, as `compress_regions(out, next_indices, next_splits, counts=...)` would, and the result ends with a dict
    of comp [capacity, C], records (LayerNorm eps `pack_eps`), patches, offsets [B+1], region_rows and `workspace`,
    whose first word stays 0 unless the kernel failed.  `workspace` is a zeroed int64 tensor of
    `pack_next_workspace_words(...)` words that nothing else uses meanwhile; without it the call makes and clears
    one; "static" takes the array built into the library (`vtdge_decompress_router_compress_static`: no allocation
    inside the library call, one call at a time per GPU), and the dict's `workspace` is then None."""
    _need_gpu(inp, indices, splits, offsets, reference, sub, next_weight, next_bias)
    inp, reference = _contig(inp), _contig(reference)
    sub = None if sub is None else _contig(sub)
    indices, splits = _contig(indices), _contig(splits)
    B, N, C = reference.shape
    extra = N - H * W
    _check_like(inp, reference=reference, sub=sub, next_weight=next_weight, next_bias=next_bias)
    if inp.shape[-1] != C or (sub is not None and sub.shape != inp.shape):
        raise ValueError("packed rows do not match the reference's channel count")
    if indices.dtype != torch.int64 or splits.dtype != torch.int64 or offsets.dtype != torch.int64:
        raise TypeError("indices, splits and offsets must be int64")
    if extra < 0 or H % region_size or W % region_size or tuple(indices.shape) != (B, H // region_size, W // region_size):
        raise ValueError(f"gate indices {tuple(indices.shape)} do not match a {H}x{W} grid of regions of {region_size}")
    if offsets.numel() != B + 1:
        raise ValueError("offsets must have B + 1 entries")
    out = torch.empty((B, N, C), dtype=inp.dtype, device=inp.device)
    S = splits.numel()
    gate = nidx = None
    S2 = S
    if next_weight is not None:
        next_weight, next_bias = _contig(next_weight), _contig(next_bias)
        S2 = next_weight.shape[0]
        _check_router(next_weight, next_bias, C, S2, extra, H, W, region_size)
        Hr, Wr = H // region_size, W // region_size
        gate = torch.empty((B, Hr, Wr, S2), dtype=inp.dtype, device=inp.device) if want_gate else None
        nidx = torch.empty((B, Hr, Wr), dtype=torch.int64, device=inp.device)
    rec = None
    if stats_eps is not None:
        rec = torch.empty((B * N, 16), dtype=torch.bfloat16, device=inp.device)
    counts = None
    if next_splits is not None:
        if next_weight is None or next_splits.dtype != torch.int64 or next_splits.numel() != S2:
            raise ValueError("next_splits goes with the next router: int64, one entry per row of next_weight")
        _need_gpu(next_splits)
        next_splits = _contig(next_splits)
    if (region_rows is None) != (cur_counts is None):
        raise ValueError("region_rows (from compress_regions) and cur_counts (this block's count bytes) go together")
    if region_rows is not None:
        _need_gpu(region_rows, cur_counts)
        nr = B * (H // region_size) * (W // region_size)
        if region_rows.dtype != torch.int32 or region_rows.numel() != nr or cur_counts.dtype != torch.uint8 \
                or cur_counts.numel() < nr:
            raise ValueError("region_rows must be int32 with one entry per region, cur_counts the uint8 buffer beside it")
    if next_splits is not None:
        counts = region_counts_buffer(B, (H // region_size) * (W // region_size), inp.device)
    if pack_next:
        if rec is None or counts is None or pack_eps is None:
            raise ValueError("pack_next needs stats_eps, next_splits and pack_eps")
        regions = B * (H // region_size) * (W // region_size)
        if capacity is None:
            capacity = B * N
        if capacity < B * N:
            raise ValueError("the packed rows are written without bounds checks: capacity must be at least B * N")
        words = pack_next_workspace_words(B, H, W, region_size)
        built_in = isinstance(workspace, str) and workspace == "static"
        clear = workspace is None
        if built_in:
            workspace = None
        elif clear:
            workspace = torch.empty((words,), dtype=torch.int64, device=inp.device)
        elif workspace.dtype != torch.int64 or workspace.numel() < words or not workspace.is_contiguous():
            raise ValueError(f"workspace must be a contiguous int64 tensor of at least {words} words")
        ncomp = torch.empty((capacity, C), dtype=inp.dtype, device=inp.device)
        nrec = torch.empty((capacity, 16), dtype=torch.bfloat16, device=inp.device)
        npat = torch.empty((capacity, 4), dtype=torch.int64, device=inp.device)
        noff = torch.empty((B + 1,), dtype=torch.int64, device=inp.device)
        nrows = torch.empty((regions,), dtype=torch.int32, device=inp.device)
        head = (ptr(inp), ptr(sub), ptr(indices), ptr(splits), ptr(offsets), ptr(reference), ptr(out),
                ptr(next_weight), ptr(next_bias), ptr(gate), ptr(nidx), ptr(rec), float(stats_eps), ptr(next_splits),
                ptr(counts), ptr(region_rows), ptr(cur_counts), ptr(ncomp), ptr(nrec), float(pack_eps), ptr(npat),
                capacity, ptr(noff), ptr(nrows))
        tail = (B, H, W, C, extra, region_size, S, S2, dtype_code(inp), stream_ptr())
        if built_in:       # the status words inside the library: the call itself allocates nothing
            call("vtdge_decompress_router_compress_static", *head, *tail,
                 tag=("decompress_router_compress", sub is not None, C, True))
        else:
            _need_gpu(workspace)
            call("vtdge_decompress_router_compress", *head, ptr(workspace), workspace.numel() * 8, int(clear), *tail,
                 tag=("decompress_router_compress", sub is not None, C, True))
        packed = {"comp": ncomp, "records": nrec, "patches": npat, "offsets": noff, "region_rows": nrows,
                  "workspace": workspace}
        return (out, gate, nidx, rec, counts, packed)
    call("vtdge_decompress_router", ptr(inp), ptr(sub), ptr(indices), ptr(splits), ptr(offsets), ptr(reference),
         ptr(out), ptr(next_weight), ptr(next_bias), ptr(gate), ptr(nidx), ptr(rec),
         float(stats_eps if stats_eps is not None else 0.0), ptr(next_splits), ptr(counts), ptr(region_rows),
         ptr(cur_counts), B, H, W, C, extra, region_size, S, S2, dtype_code(inp), stream_ptr(),
         tag=("decompress_router", sub is not None, next_weight is not None, C, rec is not None))
    res = (out, gate, nidx) + ((rec,) if stats_eps is not None else ()) + ((counts,) if counts is not None else ())
    return res


def router_stats(x, weight, bias, H, W, region_size, stats_eps, front_rows=None, splits=None, want_gate=True,
                 clear=None):
    """`router` and `layernorm_stats` of every token in one pass over x [B, extra + H*W, C] (bf16, see
    `fits_scatter_stats`): -> (gate or None, indices, records [B*N, 16], counts or None).  `front_rows` [extra, C] are
    first written into the extra-token rows of every sample of x (in place); with `splits` (int64, device) the uint8
    query counts per region are left for `compress_regions`.  `clear`: a contiguous int64 tensor the launch zeroes on
    its way (the workspaces of the `decompress_router(..., pack_next=True)` calls that follow)."""
    _need_gpu(x, weight, bias, front_rows, splits)
    if not x.is_contiguous():
        raise ValueError("router_stats works on x in place: it must be contiguous")
    B, N, C = x.shape
    S = weight.shape[0]
    extra = N - H * W
    weight, bias = _contig(weight), _contig(bias)
    _check_like(x, weight=weight, bias=bias, front_rows=front_rows)
    _check_router(weight, bias, C, S, extra, H, W, region_size)
    if front_rows is not None:
        front_rows = _contig(front_rows.reshape(-1, C))
        if front_rows.shape[0] != extra:
            raise ValueError(f"front_rows holds {front_rows.shape[0]} rows, the tokens have {extra} in front")
    Hr, Wr = H // region_size, W // region_size
    gate = torch.empty((B, Hr, Wr, S), dtype=x.dtype, device=x.device) if want_gate else None
    indices = torch.empty((B, Hr, Wr), dtype=torch.int64, device=x.device)
    rec = torch.empty((B * N, 16), dtype=torch.bfloat16, device=x.device)
    counts = None
    if splits is not None:
        if splits.dtype != torch.int64 or splits.numel() != S:
            raise ValueError("splits must be int64 with one entry per row of the router's weight")
        splits = _contig(splits)
        counts = region_counts_buffer(B, Hr * Wr, x.device)
    if clear is not None:
        _need_gpu(clear)
        if clear.dtype != torch.int64 or not clear.is_contiguous():
            raise ValueError("clear must be a contiguous int64 tensor")
    call("vtdge_router_stats", ptr(x), ptr(front_rows), ptr(weight), ptr(bias), ptr(gate), ptr(indices), ptr(rec),
         float(stats_eps), ptr(splits), ptr(counts), ptr(clear), clear.numel() if clear is not None else 0,
         B, H, W, C, extra, region_size, S, dtype_code(x), stream_ptr(),
         tag=("router_stats", C))
    return gate, indices, rec, counts


def fits_scatter_stats(x):
    """Whether `decompress_router` can write statistics records for rows like those of x [B, N, C]."""
    return x.is_cuda and x.dtype == torch.bfloat16 and 264 <= x.shape[-1] <= 512 and x.shape[-1] % 8 == 0


def fits_decompress_layernorm(x):
    """Whether a row of x is at most 64 16-byte vectors (the fused scatter + LayerNorm holds a row in one wave)."""
    return x.shape[-1] * x.element_size() <= 64 * 16


def fits_patch_embed_norm(images, weight, P):
    """Whether `patch_embed_norm` has a kernel: bf16 images of 3 channels, 4 x 4 patches, 64 outputs, a side that is a
    multiple of 64."""
    return (images.is_cuda and images.dtype == torch.bfloat16 and images.dim() == 4 and images.shape[1] == 3 and P == 4
            and weight.shape[0] == 64 and images.shape[2] == images.shape[3] and images.shape[2] % 64 == 0
            and images.is_contiguous())


def patch_embed_norm(images, weight, bias, ln_weight, ln_bias, ln_eps, pos, P):
    """images [B, 3, S, S] -> tokens [B, (S/P)^2, N]: the stride-P convolution (weight [N, 3, P, P]) + bias, LayerNorm
    and `+ pos` [(S/P)^2, N] (optional) in one pass.  See `fits_patch_embed_norm`."""
    _need_gpu(images, weight, bias, ln_weight, ln_bias, pos)
    B, Cin, S, _ = images.shape
    N = weight.shape[0]
    G = S // P
    _check_like(images, weight=weight, bias=bias, ln_weight=ln_weight, ln_bias=ln_bias, pos=pos)
    w2 = _contig(weight.reshape(N, Cin * P * P))
    if pos is not None:
        pos = _contig(pos.reshape(-1, N))
        if pos.shape[0] != G * G:
            raise ValueError(f"pos holds {pos.shape[0]} rows, the grid has {G * G} patches")
    out = torch.empty((B, G * G, N), dtype=images.dtype, device=images.device)
    call("vtdge_patch_embed_norm", ptr(images), ptr(w2), ptr(_contig(bias)), ptr(_contig(ln_weight)),
         ptr(_contig(ln_bias)), float(ln_eps), ptr(pos), ptr(out), B, Cin, S, P, N, dtype_code(images), stream_ptr(),
         tag=("patch_embed_norm", B, S))
    return out


def layernorm(x, weight, bias, eps=1e-6, rows_dev=None, out=None, add=None):
    """LayerNorm over the last dimension.  `add` [P, C] (e.g. a position embedding): row r of the result also gets row
    r mod P of it, added after the LayerNorm's rounding to the storage type as `norm(x) + pos` would."""
    _need_gpu(x, weight, bias, add)
    x = _contig(x)
    C = x.shape[-1]
    _check_like(x, weight=weight, bias=bias, out=out)
    _check_vector("weight", weight, C)
    _check_vector("bias", bias, C)
    weight, bias = _contig(weight), _contig(bias)
    rows = x.numel() // C
    if out is None:
        out = torch.empty_like(x)
    elif out.shape != x.shape or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor of the input's shape")
    if add is not None:
        if rows_dev is not None:
            raise ValueError("layernorm: `add` goes with all rows (no live row count)")
        _check_like(x, add=add)
        add = _contig(add.reshape(-1, C))
        call("vtdge_layernorm_add", ptr(x), ptr(weight), ptr(bias), ptr(add), add.shape[0], ptr(out), rows, C,
             float(eps), dtype_code(x), stream_ptr(), tag=("layernorm", False, rows, C))
        return out
    call("vtdge_layernorm", ptr(x), ptr(weight), ptr(bias), ptr(out), ptr(rows_dev), rows, C, float(eps),
         dtype_code(x), stream_ptr(), tag=("layernorm", rows_dev is not None, rows, C))
    return out


def layernorm_front_rows(x, count, weight, bias, eps=1e-6):
    """LayerNorm of the first `count` rows of every sample of x [B, N, C] -> [B, count, C], read in place (no copy of
    the slice): the model's final norm on the class-token rows only."""
    _need_gpu(x, weight, bias)
    if x.dim() != 3 or not x.is_contiguous() or not 0 < count <= x.shape[1]:
        raise ValueError("layernorm_front_rows takes contiguous [B, N, C] tokens and 0 < count <= N")
    B, N, C = x.shape
    _check_like(x, weight=weight, bias=bias)
    _check_vector("weight", weight, C)
    _check_vector("bias", bias, C)
    out = torch.empty((B, count, C), dtype=x.dtype, device=x.device)
    call("vtdge_layernorm_rows", ptr(x), N * C, count, ptr(_contig(weight)), ptr(_contig(bias)), ptr(out), B * count, C,
         float(eps), dtype_code(x), stream_ptr(), tag=("layernorm", False, B * count, C))
    return out


PACK_WEIGHTS = True     # module switch (tests compare the two paths)
_pack_epoch = 0         # bumped by invalidate_packed(): every packed copy made before is stale


def invalidate_packed(obj=None):
    """Forget packed copies of Linear weights: all of them (no argument), one tensor's, or those of every parameter
    of a module.

    The copy is keyed on the weight's storage address, shape, dtype, device and version counter, which covers
    `load_state_dict`, `.to()` / `.bfloat16()`, optimiser steps and every in-place torch op on the parameter.  It does
    NOT see writes that bypass the version counter: `w.data.copy_(...)`, `w.data.mul_(...)`, a raw kernel writing
    into the storage.  After such a write call this function (or `engine.prepare(model)`) before the next forward;
    otherwise the weight-stationary kernels keep multiplying by the old weights."""
    global _pack_epoch
    if obj is None:
        _pack_epoch += 1
        return
    tensors = obj.parameters() if isinstance(obj, torch.nn.Module) else [obj]
    for t in tensors:
        if getattr(t, "_vtdge_packed", None) is not None:
            t._vtdge_packed = None
        if getattr(t, "_vtdge_folded", None) is not None:
            t._vtdge_folded = None


def packed_weight(weight):
    """The copy of a Linear weight [N, K] in the register order of the weight-stationary kernels, made once per
    weight tensor and version and kept on the tensor object; None when the kernels for this shape take W as it is.
    See `invalidate_packed` for the one kind of edit the key cannot detect."""
    key = (weight.data_ptr(), weight._version, tuple(weight.shape), weight.dtype, weight.device, _pack_epoch)
    cached = getattr(weight, "_vtdge_packed", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    N, K = weight.shape
    lib = _lib.load()        # not through call(): these two are no part of a timed step
    size = ctypes.c_int64(0)
    if lib.vtdge_linear_packed_size(N, K, dtype_code(weight), ctypes.addressof(size)) != 0:
        raise _lib.VtdgeError(lib.vtdge_last_error().decode("utf-8", "replace"))
    packed = None
    if size.value:
        packed = torch.empty((size.value,), dtype=torch.uint8, device=weight.device)
        if lib.vtdge_linear_prepack(ptr(weight), N, K, dtype_code(weight), ptr(packed), stream_ptr()) != 0:
            raise _lib.VtdgeError(lib.vtdge_last_error().decode("utf-8", "replace"))
    try:
        weight._vtdge_packed = (key, packed)
    except AttributeError:      # an object that takes no attributes: pack again next time
        pass
    return packed


def fits_linear_stats(a, weight):
    """Whether `linear(..., stats_eps=...)` has a kernel for these operands (bf16, 384 -> 384, 2048 rows or more)."""
    return fits_linear_layernorm(a, weight) and weight.shape[0] == 384


def linear(a, weight, bias=None, residual=None, act="none", rows_dev=None, out=None, stats_eps=None):
    """out = act(a @ weight.T + bias) + residual; a [..., K] (last dim contiguous), weight [N, K].
    With `stats_eps` (a LayerNorm's eps; see `fits_linear_stats`) -> (out, statistics records of the rows of out) for a
    `linear_layernorm` that takes `out` next."""
    _need_gpu(a, weight, bias, residual)
    _check_like(a, weight=weight, bias=bias, residual=residual, out=out)
    K = a.shape[-1]
    if weight.dim() != 2 or weight.shape[1] != K:
        raise ValueError(f"weight {tuple(weight.shape)} does not take inputs of width {K}")
    a2 = a.reshape(-1, K)
    if a2.stride(-1) != 1:
        a2 = a2.contiguous()
    weight = _contig(weight)
    N = weight.shape[0]
    _check_vector("bias", bias, N)
    bias = None if bias is None else _contig(bias)
    rows = a2.shape[0]
    if out is None:
        out = torch.empty(a.shape[:-1] + (N,), dtype=a.dtype, device=a.device)
    elif out.numel() != rows * N or out.shape[-1] != N:
        raise ValueError(f"out {tuple(out.shape)} does not hold {rows} rows of {N}")
    o2 = out.view(-1, N)
    r2 = None
    if residual is not None:
        if residual.numel() != rows * N or residual.shape[-1] != N:
            raise ValueError(f"residual {tuple(residual.shape)} does not hold {rows} rows of {N}")
        r2 = residual.reshape(-1, N)
        if r2.stride(-1) != 1:
            r2 = r2.contiguous()
    packed = packed_weight(weight) if PACK_WEIGHTS and a.dtype == torch.bfloat16 and rows >= 2048 else None
    if stats_eps is not None:
        if act != "none" or not fits_linear_stats(a2, weight):
            raise ValueError("linear: no kernel that writes statistics records for these operands (see fits_linear_stats)")
        rec = torch.empty((rows, 16), dtype=torch.bfloat16, device=a.device)
        call("vtdge_linear_stats", ptr(a2), a2.stride(0), ptr(weight), ptr(packed), ptr(bias), ptr(r2),
             r2.stride(0) if r2 is not None else 0, ptr(o2), o2.stride(0), ptr(rec), float(stats_eps), ptr(rows_dev),
             rows, N, K, dtype_code(a), stream_ptr(),
             tag=("linear_stats", bias is not None, residual is not None, rows, N, K, rows_dev is not None))
        return out, rec
    call("vtdge_linear_prepacked", ptr(a2), a2.stride(0) if rows > 1 else K, ptr(weight), ptr(packed), ptr(bias), ptr(r2),
         (r2.stride(0) if rows > 1 else N) if r2 is not None else 0, ptr(o2), o2.stride(0) if rows > 1 else N,
         ptr(rows_dev), rows, N, K, _lib.ACT_GELU if act == "gelu" else _lib.ACT_NONE, dtype_code(a), stream_ptr(),
         tag=("linear", act, bias is not None, residual is not None, rows, N, K, rows_dev is not None))
    return out


# ------------------------------------------------------------------ LayerNorm folded into the Linear behind it
def fits_linear_layernorm(a, weight):
    """Whether `linear_layernorm` has a kernel for these operands (bf16, rows of 384, 2048 rows or more, an output
    width that is a multiple of 384 up to 3072)."""
    K = a.shape[-1]
    rows = a.numel() // max(K, 1)
    return (a.is_cuda and a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and K == 384
            and weight.dim() == 2 and weight.shape[1] == K and weight.shape[0] % 384 == 0 and weight.shape[0] <= 3072
            and rows >= 2048 and a.stride(-1) == 1)


def layernorm_stats(x, eps=1e-6, rows_dev=None, out=None):
    """The statistics records [rows, 16] bf16 of the rows of x [..., C] (bf16): what `linear_layernorm` takes next to
    the raw rows instead of a normalised copy."""
    _need_gpu(x)
    if x.dtype != torch.bfloat16:
        raise TypeError("layernorm_stats: records exist for bfloat16 rows only")
    x = _contig(x)
    C = x.shape[-1]
    rows = x.numel() // C
    if out is None:
        out = torch.empty((rows, 16), dtype=torch.bfloat16, device=x.device)
    elif out.shape != (rows, 16) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise ValueError(f"records must be a contiguous bfloat16 tensor of shape ({rows}, 16)")
    call("vtdge_layernorm_stats", ptr(x), ptr(out), ptr(rows_dev), rows, C, float(eps), dtype_code(x), stream_ptr(),
         tag=("layernorm_stats", rows, C))
    return out


def folded_weight(weight, bias, ln_weight, ln_bias):
    """-> (W', column records, packed copy of W' or None) for `linear_layernorm`: the Linear's weight with the
    LayerNorm's scale folded in, and per output column the colsum of W' and bias + W @ ln_bias.  Made once per set of
    tensors and versions and kept on the weight tensor; `invalidate_packed` drops it like the packed copies."""
    parts = (weight, bias, ln_weight, ln_bias)
    key = tuple((t.data_ptr(), t._version, tuple(t.shape), t.dtype, t.device) if t is not None else None
                for t in parts) + (_pack_epoch,)
    cached = getattr(weight, "_vtdge_folded", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    N, K = weight.shape
    _check_like(weight, bias=bias, ln_weight=ln_weight, ln_bias=ln_bias)
    _check_vector("bias", bias, N)
    _check_vector("ln_weight", ln_weight, K)
    _check_vector("ln_bias", ln_bias, K)
    lib = _lib.load()        # not through call(): no part of a timed step
    wf = torch.empty_like(weight, memory_format=torch.contiguous_format)
    rec = torch.empty((N, 16), dtype=torch.bfloat16, device=weight.device)
    if lib.vtdge_layernorm_fold(ptr(_contig(weight.detach())), ptr(None if bias is None else _contig(bias.detach())),
                                ptr(_contig(ln_weight.detach())), ptr(_contig(ln_bias.detach())), N, K,
                                dtype_code(weight), ptr(wf), ptr(rec), stream_ptr()) != 0:
        raise _lib.VtdgeError(lib.vtdge_last_error().decode("utf-8", "replace"))
    value = (wf, rec, packed_weight(wf) if PACK_WEIGHTS else None)
    try:
        weight._vtdge_folded = (key, value)
    except AttributeError:
        pass
    return value


def fits_patch_embed(images, weight, bias, pos_embed, patch):
    """Whether `patch_embed` has a kernel: a patch row of 16, 32, 64 or 128 bytes (patch 16 in both types), square
    images whose edge is a multiple of the patch, bias and position table present."""
    if images.dim() != 4 or images.shape[2] != images.shape[3] or bias is None or pos_embed is None:
        return False
    esz = images.element_size()
    row = patch * esz
    S = images.shape[2]
    return (images.dtype in (torch.float32, torch.bfloat16) and patch > 0 and S % patch == 0 and row % 16 == 0
            and 128 % row == 0 and patch % (128 // row) == 0 and (S * esz) % 16 == 0
            and weight.shape[0] % (16 // esz) == 0)


def patch_embed(images, weight, bias, pos_embed, patch, extra, out=None):
    """tokens [B, extra + G*G, C]: rows extra.. of every sample = the stride-`patch` convolution of `images`
    [B, Cin, S, S] with `weight` [C, Cin, patch, patch] (or flattened) + bias + pos_embed[extra..]; rows before them
    are left as they are (uninitialised in a fresh tensor).  Replaces PatchEmbed's Conv2d and the addition of the
    position embedding (vtpack/models/dge/deit_dge.py:141-155, :277) without an unfolded copy of the images."""
    _need_gpu(images, weight, bias, pos_embed)
    _check_like(images, weight=weight, bias=bias, pos_embed=pos_embed, out=out)
    if not fits_patch_embed(images, weight, bias, pos_embed, patch):
        raise ValueError("patch_embed: no kernel for these operands (see fits_patch_embed)")
    B, Cin, S, _ = images.shape
    G = S // patch
    C = weight.shape[0]
    w2 = _contig(weight.reshape(C, -1))
    if w2.shape[1] != Cin * patch * patch:
        raise ValueError(f"weight {tuple(weight.shape)} does not take {Cin} x {patch} x {patch} patches")
    _check_vector("bias", bias, C)
    pos = _contig(pos_embed.reshape(-1, C))
    if pos.shape[0] != extra + G * G:
        raise ValueError(f"pos_embed holds {pos.shape[0]} rows, the tokens {extra + G * G}")
    images = _contig(images)
    if out is None:
        out = torch.empty((B, extra + G * G, C), dtype=images.dtype, device=images.device)
    elif tuple(out.shape) != (B, extra + G * G, C) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous tensor of shape {(B, extra + G * G, C)}")
    call("vtdge_patch_embed", ptr(images), ptr(w2), ptr(_contig(bias)), ptr(pos), ptr(out), B, Cin, S, patch, C, extra,
         dtype_code(images), stream_ptr(), tag=("patch_embed", B, S, patch, C))
    return out


def fits_patch_linear(x, H, W, k, weight, bias):
    """Whether `patch_linear` has a kernel: contiguous tokens whose channels fill whole 128-byte pieces, a grid that
    is a multiple of the block edge, a bias."""
    if x.dim() != 3 or bias is None or x.dtype not in (torch.float32, torch.bfloat16):
        return False
    esz = x.element_size()
    C = x.shape[-1]
    return (k > 0 and H > 0 and W > 0 and x.shape[1] == H * W and H % k == 0 and W % k == 0 and (C * esz) % 128 == 0
            and weight.dim() == 2 and weight.shape[1] == k * k * C and weight.shape[0] % (16 // esz) == 0)


def patch_linear(x, H, W, k, weight, bias, out=None):
    """[B * (H/k) * (W/k), N]: the stride-k k x k convolution over the channels-last token grid x [B, H*W, C], as a
    Linear over its k x k blocks of tokens read in place; `weight` [N, k*k*C] is the convolution's weight in
    (kh, kw, c) order.  Replaces the spatial-reduction Conv2d and the later stages' PatchEmbed Conv2d
    (vtpack/models/dge/pvt_dge.py:62, :81-83, :164, :175) without a gathered copy of the tokens."""
    _need_gpu(x, weight, bias)
    _check_like(x, weight=weight, bias=bias, out=out)
    if not fits_patch_linear(x, H, W, k, weight, bias):
        raise ValueError("patch_linear: no kernel for these operands (see fits_patch_linear)")
    B, _, C = x.shape
    N = weight.shape[0]
    _check_vector("bias", bias, N)
    x = _contig(x)
    rows = B * (H // k) * (W // k)
    if out is None:
        out = torch.empty((rows, N), dtype=x.dtype, device=x.device)
    elif tuple(out.shape) != (rows, N) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous tensor of shape {(rows, N)}")
    call("vtdge_patch_linear", ptr(x), ptr(_contig(weight)), ptr(_contig(bias)), ptr(out), B, H, W, C, k, N,
         dtype_code(x), stream_ptr(), tag=("patch_linear", B, H, W, C, k, N))
    return out


def linear_layernorm(a, records, weight, bias, ln_weight, ln_bias, act="none", rows_dev=None, out=None):
    """out = act(LayerNorm(a) @ weight.T + bias) from the raw rows a [..., 384] and their statistics records (from
    `layernorm_stats` or from the kernel that produced the rows): no normalised copy of `a` is written or read.
    The LayerNorm's eps is the one the records were made with."""
    _need_gpu(a, weight, bias, ln_weight, ln_bias, records)
    _check_like(a, weight=weight, bias=bias, ln_weight=ln_weight, ln_bias=ln_bias, out=out)
    if not fits_linear_layernorm(a, weight):
        raise ValueError("linear_layernorm: no kernel for these operands (see fits_linear_layernorm)")
    K = a.shape[-1]
    a2 = a.reshape(-1, K)
    rows = a2.shape[0]
    if records.shape != (rows, 16) or records.dtype != torch.bfloat16 or not records.is_contiguous():
        raise ValueError(f"records must be a contiguous bfloat16 tensor of shape ({rows}, 16)")
    N = weight.shape[0]
    wf, colrec, packed = folded_weight(weight, bias, ln_weight, ln_bias)
    if out is None:
        out = torch.empty(a.shape[:-1] + (N,), dtype=a.dtype, device=a.device)
    elif out.numel() != rows * N or out.shape[-1] != N:
        raise ValueError(f"out {tuple(out.shape)} does not hold {rows} rows of {N}")
    o2 = out.view(-1, N)
    call("vtdge_linear_layernorm", ptr(a2), a2.stride(0), ptr(records), ptr(wf), ptr(packed), ptr(colrec), ptr(o2),
         o2.stride(0), ptr(rows_dev), rows, N, K, _lib.ACT_GELU if act == "gelu" else _lib.ACT_NONE, dtype_code(a),
         stream_ptr(), tag=("linear_layernorm", act, rows, N, K, rows_dev is not None))
    return out


def linear_layernorm_pair(a0, records0, weight0, bias0, a1, records1, weight1, bias1, ln_weight, ln_bias,
                          rows_dev0=None, rows_dev1=None):
    """(linear_layernorm(a0, records0, weight0, bias0, ...), linear_layernorm(a1, records1, weight1, bias1, ...)) with
    the same LayerNorm weights, as one launch whose workgroups are shared out between the two by their live rows:
    norm1 -> kv on the tokens and norm1 -> q on the packed queries.  Same bits as the two calls."""
    _need_gpu(a0, a1, weight0, weight1, bias0, bias1, ln_weight, ln_bias, records0, records1)
    outs, args, shapes = [], [], ()
    for a, rec, w, b, rd in ((a0, records0, weight0, bias0, rows_dev0), (a1, records1, weight1, bias1, rows_dev1)):
        _check_like(a, weight=w, bias=b, ln_weight=ln_weight, ln_bias=ln_bias)
        if not fits_linear_layernorm(a, w):
            raise ValueError("linear_layernorm_pair: no kernel for these operands (see fits_linear_layernorm)")
        K = a.shape[-1]
        a2 = a.reshape(-1, K)
        rows = a2.shape[0]
        if rec.shape != (rows, 16) or rec.dtype != torch.bfloat16 or not rec.is_contiguous():
            raise ValueError(f"records must be a contiguous bfloat16 tensor of shape ({rows}, 16)")
        wf, colrec, packed = folded_weight(w, b, ln_weight, ln_bias)
        N = w.shape[0]
        out = torch.empty(a.shape[:-1] + (N,), dtype=a.dtype, device=a.device)
        outs.append(out)
        args += [ptr(a2), a2.stride(0), ptr(rec), ptr(wf), ptr(packed), ptr(colrec), ptr(out), N, ptr(rd), rows, N]
        shapes += (rows, N, rd is not None)
    call("vtdge_linear_layernorm_pair", *args, a0.shape[-1], dtype_code(a0), stream_ptr(),
         tag=("linear_layernorm_pair",) + shapes)
    return outs[0], outs[1]


def sparse_attention(q, k, v, offsets, scale, num_heads, max_rows_per_sample, out=None):
    """Strided form.  q [L, h*d]; k, v [B, n, h*d]-like views (last dim contiguous, any batch/token strides);
    offsets int64 [B+1] on the device.  Returns [L, h*d] with channel = head*d + j."""
    _need_gpu(q, k, v, offsets)
    _check_like(q, k=k, v=v, out=out)
    L, C = q.shape
    d = C // num_heads
    B, n = k.shape[0], k.shape[1]
    if k.shape != v.shape or k.shape[-1] != C or C % num_heads:
        raise ValueError(f"q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} do not share {num_heads} heads")
    if offsets.dtype != torch.int64 or offsets.numel() != B + 1:
        raise ValueError("offsets must be int64 [B + 1]")
    if not (k.stride(-1) == 1 and v.stride(-1) == 1 and q.stride(-1) == 1 and k.stride() == v.stride()):
        raise ValueError("q, k and v need a contiguous last dimension, k and v the same strides")
    if out is None:
        out = torch.empty((L, C), dtype=q.dtype, device=q.device)
    call("vtdge_sparse_attention", ptr(q), q.stride(0), d, ptr(k), ptr(v), k.stride(0), k.stride(1), d,
         ptr(offsets), ptr(out), out.stride(0), d, B, num_heads, d, n, int(max_rows_per_sample), float(scale),
         dtype_code(q), stream_ptr(), tag=("attention", B, num_heads, d, n))
    return out
