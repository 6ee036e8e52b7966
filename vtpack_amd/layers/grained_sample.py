"""Autograd-level operators of the grained sampler (mirror of vtpack/layers/grained_sample.py:11-102).

`grained_sample_compress`, `grained_sample_decompress` and `grained_sample_index_to_patch` keep
the reference's positional signatures.  Forward passes run on the HIP kernels; the backward rules
are the reference's (compress and decompress are adjoint up to size**2) expressed with the same
two kernels.
"""
import torch
import torch.nn.functional as F
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import _C


def _area(patches):
    return (patches[:, 3:4] * patches[:, 3:4])


class _Compress(Function):
    # vtpack/layers/grained_sample.py:11-38
    @staticmethod
    def forward(ctx, input, patches, height, width, num_extra_tokens):
        input, patches = input.contiguous(), patches.contiguous()
        ctx.geom = (height, width, num_extra_tokens)
        ctx.save_for_backward(input, patches)
        return _C.grained_sample_compress(input, patches, height, width, num_extra_tokens)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        input, patches = ctx.saved_tensors
        grad = grad.contiguous() / _area(patches).to(grad.dtype)
        return _C.grained_sample_decompress(grad, patches, input, *ctx.geom, False), None, None, None, None


class _Decompress(Function):
    # vtpack/layers/grained_sample.py:44-78
    @staticmethod
    def forward(ctx, input, patches, ref_input, height, width, num_extra_tokens, is_add_ref):
        input, patches, ref_input = input.contiguous(), patches.contiguous(), ref_input.contiguous()
        ctx.geom = (height, width, num_extra_tokens)
        ctx.is_add_ref = is_add_ref
        ctx.save_for_backward(patches)
        return _C.grained_sample_decompress(input, patches, ref_input, height, width, num_extra_tokens, is_add_ref)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        patches, = ctx.saved_tensors
        grad = grad.contiguous()
        g_in = _C.grained_sample_compress(grad, patches, *ctx.geom) * _area(patches).to(grad.dtype)
        g_ref = grad if ctx.is_add_ref else torch.zeros_like(grad)
        return g_in, None, g_ref, None, None, None, None


class _IndexToPatch(Function):
    # vtpack/layers/grained_sample.py:84-99 (not differentiable)
    @staticmethod
    def forward(ctx, indices, split_sizes, region_size, num_extra_tokens):
        out = _C.grained_sample_index_to_patch(indices.contiguous(), split_sizes.contiguous(), region_size,
                                               num_extra_tokens)
        ctx.mark_non_differentiable(*out)
        return out

    @staticmethod
    def backward(ctx, *grads):
        return None, None, None, None


class _IndexToPatchDense(Function):
    # vtpack/layers/grained_sample.py:105-120
    @staticmethod
    def forward(ctx, indices, split_sizes, region_size, num_extra_tokens):
        out = _C.grained_sample_index_to_patch_dense(indices.contiguous(), split_sizes.contiguous(), region_size,
                                                     num_extra_tokens)
        ctx.mark_non_differentiable(*out)
        return out

    @staticmethod
    def backward(ctx, *grads):
        return None, None, None, None


grained_sample_compress = _Compress.apply
grained_sample_decompress = _Decompress.apply
grained_sample_index_to_patch = _IndexToPatch.apply
grained_sample_index_to_patch_dense = _IndexToPatchDense.apply


# ------------------------------------------------------------------ dense (training) forms
def grained_sample_compress_dense(x, split_sizes, region_size, H, W, num_extra_tokens):
    """Queries of EVERY granularity: the extra tokens, then for each split the whole grid pooled with that split's
    window.  Plain torch ops (differentiable), as in the reference (vtpack/layers/grained_sample.py:126-148).
    -> (comp [B * per_sample, C], batch_lengths int64 [B] on the CPU)."""
    B, N, C = x.shape
    grid = x[:, num_extra_tokens:, :].reshape(B, H, W, C).permute(0, 3, 1, 2)
    levels = [x[:, :num_extra_tokens, :]] if num_extra_tokens > 0 else []
    for ps in split_sizes.tolist():
        step = region_size // int(ps)
        pooled = F.avg_pool2d(grid, step, step) if step > 1 else grid
        levels.append(pooled.flatten(2).transpose(1, 2))
    comp = torch.cat(levels, dim=1)
    return comp.reshape(-1, C), torch.full((B,), comp.shape[1], dtype=torch.int64)


def grained_sample_decompress_dense(x, gate, reference, split_sizes, region_size, H, W, num_extra_tokens, is_add_ref):
    """Inverse of the dense form: every level is upsampled to the token grid and the levels are mixed with the
    per-region gate [B, Hr, Wr, S] (one-hot in the forward pass of training).
    vtpack/layers/grained_sample.py:151-177."""
    B, N, C = reference.shape
    x = x.reshape(B, -1, C)
    spatial = 0
    start = num_extra_tokens
    for i, ps in enumerate(split_sizes.tolist()):
        step = region_size // int(ps)
        Hi, Wi = H // step, W // step
        level = x[:, start:start + Hi * Wi, :].reshape(B, Hi, Wi, C)
        level = level.repeat_interleave(step, dim=1).repeat_interleave(step, dim=2)
        weight = gate[..., i].repeat_interleave(region_size, dim=1).repeat_interleave(region_size, dim=2)
        spatial = spatial + level * weight.unsqueeze(-1)
        start += Hi * Wi
    out = spatial.reshape(B, H * W, C)
    if num_extra_tokens > 0:
        out = torch.cat([x[:, :num_extra_tokens, :], out], dim=1)
    return out + reference if is_add_ref else out
