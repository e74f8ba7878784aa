"""``matmulam``: the counterpart of the reference's ``python/ops/math_ops.py``
(op ``MatMulAM`` and ``@RegisterGradient("MatMulAM")``, math_ops.py:12-157).

Differences from the reference, on purpose:
  * transposes are passed to the GEMM as operand strides instead of being
    materialised with ``matrix_transpose`` (math_ops.py:92-93);
  * the gradient passes the LUT on (the reference's gradient calls omit the
    required ``mant_mul_lut`` attr, math_ops.py:100-156); its LUT operand order
    is the one the reference's op-level rule gives: (grad, b) and (a, grad);
  * operands of rank > 3 (the (batch, heads, seq, depth) tensors that the
    reference's attention layer feeds, multihead_attention.py:56-57) are
    flattened to a strided batch; the reference's C++ op accepts rank <= 3."""
import torch

from . import functors


def _flat3(t):
    return t.reshape((-1,) + tuple(t.shape[-2:])) if t.dim() > 3 else t


class _MatMulAM(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, transpose_a, transpose_b, mant_mul_lut):
        ctx.save_for_backward(a, b)
        ctx.attrs = (transpose_a, transpose_b, mant_mul_lut)
        return functors.gemm(mant_mul_lut, a, b, trans_a=transpose_a, trans_b=transpose_b)

    @staticmethod
    def backward(ctx, grad):
        a, b = ctx.saved_tensors
        t_a, t_b, lut = ctx.attrs
        grad = grad.contiguous()
        g = functors.gemm
        grad_a = grad_b = None

        def unbroadcast(x, like):
            # a rank-2 / batch-1 operand shared by the whole batch receives the sum over the batch
            if x.dim() == 3 and (like.dim() == 2 or like.shape[0] == 1) and x.shape[0] >= 1:
                x = x.sum(dim=0, keepdim=like.dim() == 3)
            return x

        # The reference's op receives operands that Python has already transposed, with its own
        # transpose attrs at their default (math_ops.py:92-93), so its gradient always takes the
        # first branch of math_ops.py:145-147:
        #     d(a_op) = MatMulAM(grad, b_op^T)        d(b_op) = MatMulAM(a_op^T, grad)
        # and autodiff transposes d(a_op) / d(b_op) back.  Here the transposes are strides; a
        # gradient produced transposed keeps its LUT operand order through swap_operands.
        if ctx.needs_input_grad[0]:
            if not t_a:
                grad_a = g(lut, grad, b, trans_b=not t_b)                                  # P(grad, b)
            else:
                grad_a = g(lut, b, grad, trans_a=t_b, trans_b=True, swap_operands=True)    # transposed, still P(grad, b)
            grad_a = unbroadcast(grad_a, a)
        if ctx.needs_input_grad[1]:
            if not t_b:
                grad_b = g(lut, a, grad, trans_a=not t_a)                                  # P(a, grad)
            else:
                grad_b = g(lut, grad, a, trans_a=True, trans_b=t_a, swap_operands=True)    # transposed, still P(a, grad)
            grad_b = unbroadcast(grad_b, b)
        return grad_a, grad_b, None, None, None


def matmulam(a, b, transpose_a=False, transpose_b=False, adjoint_a=False, adjoint_b=False, a_is_sparse=False,
             b_is_sparse=False, mant_mul_lut='', name=None):
    if adjoint_a or adjoint_b or a_is_sparse or b_is_sparse:
        raise ValueError("Matmulam unsupported args: adjoint_a, adjoint_b, a_is_sparse, b_is_sparse.")
    if not mant_mul_lut:
        raise ValueError("mant_mul_lut: the LUT file name attr has no default (matmulam.cc:55)")
    if a.dim() < 2 or b.dim() < 2:
        raise ValueError("Input a and b should be 2 dimensional or 3 dimensional and compitable batch size")
    lead = a.shape[:-2] if a.dim() >= b.dim() else b.shape[:-2]
    if a.dim() > 3 or b.dim() > 3:
        if a.dim() != b.dim() or a.shape[:-2] != b.shape[:-2]:
            raise ValueError("operands of rank > 3 need identical leading dimensions")
    out = _MatMulAM.apply(_flat3(a), _flat3(b), bool(transpose_a), bool(transpose_b), mant_mul_lut)
    if a.dim() > 3 or b.dim() > 3:
        out = out.reshape(tuple(lead) + tuple(out.shape[-2:]))
    return out
