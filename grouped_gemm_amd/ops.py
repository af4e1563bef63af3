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


# --------------------------------------------------- fused permutation (gather / scatter)
#
# MoE layers sort their tokens by expert before the first grouped GEMM and put the rows back after
# the last one.  The reference's operator takes rows already sorted (ops.py:8); these two forms
# take the permutation as an index and do the move inside the GEMM's loads or stores, which saves
# a full pass over the activations each.  Not part of the reference's surface.

class GroupedGemmGather(torch.autograd.Function):
    """out[r] = x[row_index[r]] @ w[expert of r]: rows are gathered while they are loaded.  An
    index may name a row of x several times (top-k routing)."""

    @staticmethod
    def forward(ctx, x, w, batch_sizes, row_index, trans_b):
        ctx.save_for_backward(x, w, batch_sizes, row_index)
        ctx.trans_b = trans_b
        return backend.gmm_indexed(x, w, batch_sizes, trans_b=trans_b, a_rows=row_index)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        x, w, batch_sizes, row_index = ctx.saved_tensors
        xgrad = wgrad = None
        if ctx.needs_input_grad[0]:
            # rows of x that several sorted rows came from collect several gradients: a sum, not
            # a store, so it is not fused
            sorted_grad = backend.gmm(grad, w, batch_sizes, trans_b=not ctx.trans_b)
            xgrad = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
            xgrad.index_add_(0, row_index.long(), sorted_grad.float())
            xgrad = xgrad.to(x.dtype)
        if ctx.needs_input_grad[1]:
            # The weight-gradient layout takes row indices on the general kernels only, which are
            # several times slower than the streaming ones: one explicit gather and the streaming
            # kernel is the faster way to the same result.
            sorted_x = x.index_select(0, row_index.long())
            lhs, rhs = (grad, sorted_x) if ctx.trans_b else (sorted_x, grad)
            wgrad = backend.gmm(lhs, rhs, batch_sizes, trans_a=True)
        return xgrad, wgrad, None, None, None


class GroupedGemmScatter(torch.autograd.Function):
    """out[row_index[r]] = a[r] @ w[expert of r] for a permutation row_index of 0..rows-1: rows are
    put back in their original order while they are stored."""

    @staticmethod
    def forward(ctx, a, w, batch_sizes, row_index, trans_b):
        ctx.save_for_backward(a, w, batch_sizes, row_index)
        ctx.trans_b = trans_b
        hidden_out = w.shape[1] if trans_b else w.shape[2]
        out = torch.empty(a.shape[0], hidden_out, dtype=a.dtype, device=a.device)
        return backend.gmm_indexed(a, w, batch_sizes, trans_b=trans_b, c=out, c_rows=row_index)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, w, batch_sizes, row_index = ctx.saved_tensors
        agrad = wgrad = None
        if ctx.needs_input_grad[0]:
            agrad = backend.gmm_indexed(grad, w, batch_sizes, trans_b=not ctx.trans_b, a_rows=row_index)
        if ctx.needs_input_grad[1]:
            # (as in GroupedGemmGather: an explicit gather, then the streaming weight-gradient kernel)
            sorted_grad = grad.index_select(0, row_index.long())
            lhs, rhs = (sorted_grad, a) if ctx.trans_b else (a, sorted_grad)
            wgrad = backend.gmm(lhs, rhs, batch_sizes, trans_a=True)
        return agrad, wgrad, None, None, None


def gmm_gather(x, w, batch_sizes, row_index, trans_b=False):
    """gmm(x[row_index], w, batch_sizes, trans_b) with the gather fused into the GEMM."""
    return GroupedGemmGather.apply(x, w, batch_sizes, row_index, trans_b)


def gmm_scatter(a, w, batch_sizes, row_index, trans_b=False):
    """out with out[row_index] = gmm(a, w, batch_sizes, trans_b): the scatter fused into the GEMM.
    row_index must be a permutation of the rows."""
    return GroupedGemmScatter.apply(a, w, batch_sizes, row_index, trans_b)


# ------------------------------------------------------------------ gated activation

class GroupedGemmSwiGLU(torch.autograd.Function):
    """silu(a @ gate) * (a @ up) with w = [gate | up] per expert, the activation fused into the
    GEMM's epilogue.  The backward recomputes the two products with a plain grouped GEMM (they are
    not stored by the forward), applies the derivative elementwise and runs the two usual
    gradient GEMMs on the result."""

    @staticmethod
    def forward(ctx, a, w, batch_sizes, trans_b):
        ctx.save_for_backward(a, w, batch_sizes)
        ctx.trans_b = trans_b
        return backend.gmm_swiglu(a, w, batch_sizes, trans_b=trans_b)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, w, batch_sizes = ctx.saved_tensors
        gate_up = backend.gmm(a, w, batch_sizes, trans_b=ctx.trans_b).float()
        gate, up = gate_up.chunk(2, dim=-1)
        sig = torch.sigmoid(gate)
        g32 = grad.float()
        dgate = g32 * up * sig * (1.0 + gate * (1.0 - sig))
        dup = g32 * gate * sig
        dgu = torch.cat([dgate, dup], dim=-1).to(a.dtype)
        agrad = wgrad = None
        if ctx.needs_input_grad[0]:
            agrad = backend.gmm(dgu, w, batch_sizes, trans_b=not ctx.trans_b)
        if ctx.needs_input_grad[1]:
            lhs, rhs = (dgu, a) if ctx.trans_b else (a, dgu)
            wgrad = backend.gmm(lhs, rhs, batch_sizes, trans_a=True)
        return agrad, wgrad, None, None


def gmm_swiglu(a, w, batch_sizes, trans_b=False):
    """silu(a @ gate) * (a @ up) per expert, w = [gate | up]; see backend.gmm_swiglu."""
    return GroupedGemmSwiGLU.apply(a, w, batch_sizes, trans_b)


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
