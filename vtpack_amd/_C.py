"""HIP-backed stand-in for the reference's native module `vtpack._C`.

Same Python-visible names, argument order and return values as the functions
the reference registers in vtpack/layers/csrc/vision.cpp:9-29 for the DGE query
path; each forwards to one entry point of libvtdge.so.  Like the reference,
outputs are freshly allocated and `batch_lengths` comes back on the CPU (which
costs the one device->host copy per call that the reference also pays).
"""
import torch

from . import ops
from ._lib import call, dtype_code, ptr, stream_ptr


def _check_same_dtype(*ts):
    d = ts[0].dtype
    for t in ts[1:]:
        if t.dtype != d:
            raise TypeError(f"operand dtypes differ: {d} vs {t.dtype}")


def grained_sample_index_to_patch(indices, split_sizes, region_size, num_extra_tokens):
    """-> (patches int64 [L,4] on the GPU, batch_lengths int64 [B] on the CPU).

    vtpack/layers/csrc/grained_sample/grained_sample.cu:302-345."""
    if indices.dtype != torch.int64 or split_sizes.dtype != torch.int64:
        raise TypeError("indices and split_sizes must be int64")
    patches, offsets, lengths = ops.index_to_patch(indices, split_sizes, int(region_size), int(num_extra_tokens))
    batch_lengths = lengths.cpu()
    total = int(batch_lengths.sum())
    if total > patches.shape[0]:
        raise RuntimeError(
            f"split sizes produce {total} queries, more than one per token ({patches.shape[0]}): "
            "every split size must divide the region size")
    return patches[:total], batch_lengths


def grained_sample_index_to_patch_dense(indices, split_sizes, region_size, num_extra_tokens):
    """-> (patches of every granularity, batch_lengths on the CPU).  grained_sample.cu:393-433."""
    ops._need_gpu(indices)
    B, Hr, Wr = indices.shape
    splits_cpu = split_sizes.detach().to("cpu", torch.int64).contiguous()
    per = int(num_extra_tokens + (splits_cpu * splits_cpu).sum().item() * Hr * Wr)
    patches = torch.empty((B * per, 4), dtype=torch.int64, device=indices.device)
    call("vtdge_index_to_patch_dense", splits_cpu.data_ptr(), B, Hr, Wr, splits_cpu.numel(), int(region_size),
         int(num_extra_tokens), ptr(patches), stream_ptr())
    return patches, torch.full((B,), per, dtype=torch.int64)


def _pad_channels(t):
    """The kernels move 16 bytes per lane; a channel count that is not a multiple of that (the [B, N, 1] gate map
    of sparse training, vtpack/layers/dge.py:96-106) is zero-padded here and sliced back by the caller."""
    vec = 16 // t.element_size()
    C = t.shape[-1]
    if C % vec == 0:
        return t, C
    return torch.nn.functional.pad(t, (0, vec - C % vec)), C


def grained_sample_compress(input, patches, height, width, num_extra_tokens):
    """input [B,N,C], patches [L,4] -> [L,C].  grained_sample.cu:198-239."""
    input, C = _pad_channels(input)
    out = ops.compress(input, patches, int(width), int(num_extra_tokens))
    return out if out.shape[-1] == C else out[:, :C].contiguous()


def grained_sample_decompress(input, patches, reference, height, width, num_extra_tokens, is_add_ref):
    """input [L,C], reference [B,N,C] -> [B,N,C].  grained_sample.cu:241-300."""
    _check_same_dtype(input, reference)
    input, C = _pad_channels(input)
    reference, _ = _pad_channels(reference)
    out = ops.decompress(input, patches, reference, int(width), int(num_extra_tokens), add_ref=bool(is_add_ref))
    return out if out.shape[-1] == C else out[..., :C].contiguous()


def _offsets_from_lengths(lengths, device):
    lengths = lengths.detach().to("cpu", torch.int64)
    off = torch.zeros(lengths.numel() + 1, dtype=torch.int64)
    torch.cumsum(lengths, 0, out=off[1:])
    return off.to(device), lengths


def batched_sparse_attention_forward(a, b, c, batch_lengths, scale):
    """a [h,L,d], b and c [h,B,n,d], batch_lengths int64 [B] (CPU) -> [h,L,d].

    vtpack/layers/csrc/batched_sparse_gemm/batched_sparse_gemm.cu:219-305."""
    ops._need_gpu(a, b, c)
    _check_same_dtype(a, b, c)
    a, b, c = a.contiguous(), b.contiguous(), c.contiguous()
    h, L, d = a.shape
    _, B, n, _ = b.shape
    offsets, lengths = _offsets_from_lengths(batch_lengths, a.device)
    if lengths.numel() != B or int(lengths.sum()) != L:
        raise ValueError("batch_lengths must have one entry per sample and sum to the number of query rows")
    out = torch.empty_like(a)
    max_rows = int(lengths.max()) if B > 0 else 0
    call("vtdge_sparse_attention", ptr(a), d, L * d, ptr(b), ptr(c), n * d, d, B * n * d, ptr(offsets), ptr(out), d,
         L * d, B, h, d, n, max_rows, float(scale), dtype_code(a), stream_ptr())
    return out


def batched_sparse_gemm_forward(a, b, a_lengths, b_lengths, is_a_transposed, is_b_transposed):
    """a [h,La,ka], b [h,Lb,kb]; per-sample (optionally transposed) products, concatenated on dim 1.

    vtpack/layers/csrc/batched_sparse_gemm/batched_sparse_gemm.cu:150-195."""
    ops._need_gpu(a, b)
    _check_same_dtype(a, b)
    a, b = a.contiguous(), b.contiguous()
    h, La, ka = a.shape
    _, Lb, kb = b.shape
    a_off, al = _offsets_from_lengths(a_lengths, a.device)
    b_off, bl = _offsets_from_lengths(b_lengths, a.device)
    B = al.numel()
    if bl.numel() != B or int(al.sum()) != La or int(bl.sum()) != Lb:
        raise ValueError("length vectors must match each other and the packed row counts")
    inner_a = al if is_a_transposed else torch.full_like(al, ka)
    inner_b = torch.full_like(bl, kb) if is_b_transposed else bl
    if not torch.equal(inner_a, inner_b):
        raise ValueError("inner dimensions of the per-sample products differ")
    cols = bl if is_b_transposed else torch.full_like(bl, kb)
    if B > 0 and int(cols.min()) != int(cols.max()):
        raise ValueError("per-sample outputs have different widths and cannot be concatenated on dim 1")
    out_cols = int(cols[0]) if B > 0 else 0
    out_rows = B * ka if is_a_transposed else La
    max_m = ka if is_a_transposed else (int(al.max()) if B > 0 else 0)
    out = torch.empty((h, out_rows, out_cols), dtype=a.dtype, device=a.device)
    call("vtdge_batched_sparse_gemm", ptr(a), ptr(b), ptr(a_off), ptr(b_off), ptr(out), B, h, La, ka, Lb, kb,
         int(bool(is_a_transposed)), int(bool(is_b_transposed)), out_rows, out_cols, max_m, dtype_code(a),
         stream_ptr())
    return out


# The reference's second implementation (cuBLAS batched calls per sample, :83-148) computes the same thing.
batched_sparse_gemm_v2_forward = batched_sparse_gemm_forward
