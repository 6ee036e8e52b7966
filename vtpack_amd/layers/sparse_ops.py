"""Variable-length batched operators (mirror of vtpack/layers/sparse_ops.py:11-78)."""
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import _C


class _SparseGEMM(Function):
    # vtpack/layers/sparse_ops.py:11-54; the backward is four more forward calls, as in the reference.
    @staticmethod
    def forward(ctx, a, b, a_lengths, b_lengths, is_a_transposed, is_b_transposed):
        a, b = a.contiguous(), b.contiguous()
        a_lengths, b_lengths = a_lengths.contiguous(), b_lengths.contiguous()
        ctx.flags = (is_a_transposed, is_b_transposed)
        ctx.save_for_backward(a, b, a_lengths, b_lengths)
        return _C.batched_sparse_gemm_forward(a, b, a_lengths, b_lengths, is_a_transposed, is_b_transposed)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, b, la, lb = ctx.saved_tensors
        ta, tb = ctx.flags
        f = _C.batched_sparse_gemm_forward
        g_a = f(grad, b, la, lb, ta, not tb) if not ta else f(b, grad, lb, la, tb, ta)
        g_b = f(a, grad, la, la, not ta, tb) if not tb else f(grad, a, la, la, tb, ta)
        return g_a, g_b, None, None, None, None


class _SparseAttention(Function):
    # vtpack/layers/sparse_ops.py:60-73 (forward only there as well)
    @staticmethod
    def forward(ctx, q, k, v, q_lengths, scale):
        return _C.batched_sparse_attention_forward(q.contiguous(), k.contiguous(), v.contiguous(),
                                                   q_lengths.contiguous(), scale)

    @staticmethod
    def backward(ctx, grad):
        raise NotImplementedError("Backward is not implemented.")


batched_sparse_gemm = _SparseGEMM.apply
batched_sparse_attention = _SparseAttention.apply
