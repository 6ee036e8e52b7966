"""Variable-length batched operators (mirror of vtpack/layers/sparse_ops.py:11-78)."""
import torch
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


def sparse_attention_train(q, k, v, q_lengths, scale):
    """Differentiable attention of packed queries for the training branch of the models
    (vtpack/models/dge/deit_dge.py:79-95): q [h, L, d]; k, v [h, B, n, d]; -> [L, h*d].

    Equal query counts (dense training: every granularity for every sample) use one batched matmul; otherwise the
    scores and the weighted sum are two `batched_sparse_gemm` calls around a softmax over the keys."""
    h, L, d = q.shape
    B, n = k.shape[1], k.shape[2]
    if int(q_lengths.max()) == int(q_lengths.min()):
        scores = torch.matmul(q.reshape(h, B, -1, d), k.transpose(-1, -2)) * scale
        ctx = torch.matmul(scores.softmax(dim=-1, dtype=v.dtype), v)              # [h, B, Lq, d]
        return ctx.permute(1, 2, 0, 3).reshape(-1, h * d)
    kv_lengths = q_lengths.new_full([B], n)
    scores = batched_sparse_gemm(q, k.reshape(h, -1, d), q_lengths, kv_lengths, False, True) * scale
    ctx = batched_sparse_gemm(scores.softmax(dim=-1, dtype=v.dtype), v.reshape(h, -1, d), q_lengths, kv_lengths,
                              False, False)
    return ctx.transpose(0, 1).reshape(-1, h * d)
