"""Autograd wiring of the grouped GEMM.

Mirror of the reference's grouped_gemm/ops.py:5-33.  Forward is one grouped GEMM;
backward is two more: the input gradient with the opposite layout of `b`, and the
weight gradient with `trans_a` (per expert a_e^T @ grad_e, zeros for an expert
without tokens).
"""
import torch

from grouped_gemm_amd import backend


class GroupedGemm(torch.autograd.Function):

    @staticmethod
    def forward(ctx, a, b, batch_sizes, trans_b):
        ctx.save_for_backward(a, b, batch_sizes)
        ctx.trans_b = trans_b
        return backend.gmm(a, b, batch_sizes, trans_a=False, trans_b=trans_b)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, b, batch_sizes = ctx.saved_tensors
        trans_b = ctx.trans_b

        agrad = None
        if ctx.needs_input_grad[0]:
            agrad = backend.gmm(grad, b, batch_sizes, trans_a=False, trans_b=not trans_b)

        bgrad = None
        if ctx.needs_input_grad[1]:
            lhs, rhs = (grad, a) if trans_b else (a, grad)
            bgrad = backend.gmm(lhs, rhs, batch_sizes, trans_a=True, trans_b=False)
        return agrad, bgrad, None, None


def gmm(a, b, batch_sizes, trans_b=False):
    return GroupedGemm.apply(a, b, batch_sizes, trans_b)


# ------------------------------------------------------------------ traceable form
#
# The same operator registered with torch.library, so that torch.compile sees one opaque node
# with a known output shape instead of a call into an extension it cannot trace.  Not part of
# the reference's surface (its ops.py stops at gmm above); results and gradients are those of
# GroupedGemm, through the same backend calls.

def _register_traceable():
    @torch.library.custom_op("grouped_gemm_amd::gmm", mutates_args=())
    def _gmm_op(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, trans_a: bool,
                trans_b: bool) -> torch.Tensor:
        return backend.gmm(a, b, batch_sizes, trans_a=trans_a, trans_b=trans_b)

    @_gmm_op.register_fake
    def _gmm_op_fake(a, b, batch_sizes, trans_a, trans_b):
        return backend._allocate_output(a, b, batch_sizes, trans_a, trans_b)

    def _gmm_op_setup_context(ctx, inputs, output):
        a, b, batch_sizes, trans_a, trans_b = inputs
        if trans_a:   # only reached when a gradient is wanted
            raise RuntimeError("grouped_gemm_amd::gmm is differentiable as a @ b or a @ b^T only "
                               "(trans_a=False), as GroupedGemm is")
        ctx.save_for_backward(a, b, batch_sizes)
        ctx.trans_b = trans_b

    def _gmm_op_backward(ctx, grad):
        grad = grad.contiguous()
        a, b, batch_sizes = ctx.saved_tensors
        agrad = bgrad = None
        if ctx.needs_input_grad[0]:
            agrad = _gmm_op(grad, b, batch_sizes, False, not ctx.trans_b)
        if ctx.needs_input_grad[1]:
            lhs, rhs = (grad, a) if ctx.trans_b else (a, grad)
            bgrad = _gmm_op(lhs, rhs, batch_sizes, True, False)
        return agrad, bgrad, None, None, None

    torch.library.register_autograd("grouped_gemm_amd::gmm", _gmm_op_backward,
                                    setup_context=_gmm_op_setup_context)
    return _gmm_op


# torch.library.custom_op exists from PyTorch 2.4 on; the reference's surface above must import
# on older versions too, so only gmm_traceable depends on it.
try:
    _gmm_op = _register_traceable()
except AttributeError:  # pragma: no cover - depends on the installed PyTorch
    _gmm_op = None


def gmm_traceable(a, b, batch_sizes, trans_b=False):
    """gmm for code that goes through torch.compile: same results and gradients as gmm."""
    if _gmm_op is None:
        raise RuntimeError("gmm_traceable needs torch.library.custom_op (PyTorch 2.4 or newer)")
    return _gmm_op(a, b, batch_sizes, False, trans_b)
