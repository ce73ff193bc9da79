"""``BlockSparseLinear``: drop-in for ``torch.nn.Linear`` with a block-sparse weight.

Same constructor, attributes and state_dict keys as the reference's
``pytorch_block_sparse/block_sparse_linear.py`` (:157-233); the three matmuls of the autograd
function (:40, :80, :123) run as HIP kernels on the GPU.  The bias is added in the forward
kernel's epilogue rather than by a separate ``x + bias`` pass (:231-232), and backward does not
read the weight gradient back to the host (the reference's ``(grad == 0).all()`` assert, :149-150).
"""
import math
from typing import Tuple

import torch
import torch.autograd
import torch.nn as nn

from .block_sparse import BlockSparseMatrix, BlockSparseMatrixBase, BlockSparseMatrixEmulator


class BlockSparseLinearFunction(torch.autograd.Function):
    """y = x @ W^T (+ bias).  reference: block_sparse_linear.py:15-154 (bias is an addition here)."""

    @staticmethod
    def forward(ctx, input, weight_data, weight, bias=None):
        assert isinstance(weight, BlockSparseMatrixBase)
        ctx.save_for_backward(input, weight_data)
        ctx.weight = weight
        ctx.has_bias = bias is not None
        return weight.reverse_matmul(input, transpose=True, bias=bias)

    @staticmethod
    def backward(ctx, grad_output):
        input, weight_data = ctx.saved_tensors
        weight = ctx.weight
        grad_input = grad_weight = grad_bias = None
        if ctx.needs_input_grad[0]:
            grad_input = weight.reverse_matmul(grad_output, transpose=False)
            assert grad_input.shape == input.shape
        if ctx.needs_input_grad[1]:
            grad_weight = weight.matmul_with_output_sparse_support(grad_output, input)
        if ctx.has_bias and ctx.needs_input_grad[3]:
            grad_bias = grad_output.reshape(-1, grad_output.shape[-1]).sum(0)
        return grad_input, grad_weight, None, grad_bias


class BlockSparseLinear(nn.Module):
    """reference: block_sparse_linear.py:157-233."""

    OPTIMIZED_BLOCK_SIZE = 32

    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = True,
        density: float = 0.5,
        torch_nn_linear=None,
        verbose: bool = False,
        block_shape: Tuple[int, int] = (32, 32),
        device="cuda",
        dtype=torch.float32,
    ):
        super().__init__()
        self.fn = BlockSparseLinearFunction.apply
        self.verbose = verbose
        self.block_shape = tuple(block_shape)
        self._optimized = self.block_shape == (self.OPTIMIZED_BLOCK_SIZE, self.OPTIMIZED_BLOCK_SIZE)

        if torch_nn_linear is not None:
            in_features = torch_nn_linear.in_features
            out_features = torch_nn_linear.out_features
            bias = torch_nn_linear.bias is not None
            device = torch_nn_linear.weight.device
            dtype = torch_nn_linear.weight.dtype

        if in_features % self.block_shape[1] != 0:
            raise Exception(
                f"BlockSparseLinear invalid in_features={in_features}, should be multiple of {self.block_shape[1]}"
            )
        if out_features % self.block_shape[0] != 0:
            raise Exception(
                f"BlockSparseLinear invalid out_features={out_features}, should be multiple of {self.block_shape[0]}"
            )
        if density < 0 or density > 1:
            raise Exception(f"BlockSparseLinear invalid density={density}")

        # truncation, not rounding (reference :195)
        self.block_count = int(density * (in_features * out_features / (self.block_shape[0] * self.block_shape[1])))
        self.in_features = in_features
        self.out_features = out_features

        ctor = BlockSparseMatrix if self._optimized else BlockSparseMatrixEmulator
        if torch_nn_linear is not None:
            with torch.no_grad():
                weight = ctor.from_dense(torch_nn_linear.weight, self.block_shape, self.block_count)
            weight.multiply_(1.0 / math.sqrt(density))
        else:
            weight = ctor.randn(
                (out_features, in_features), self.block_count, blocks=None, block_shape=self.block_shape,
                device=device, dtype=dtype,
            )
        self.weight = weight

        if bias:
            self.bias = nn.Parameter(torch.zeros(out_features, device=device, dtype=dtype))
            if torch_nn_linear is not None:
                with torch.no_grad():
                    self.bias.copy_(torch_nn_linear.bias)
        else:
            self.register_parameter("bias", None)

    def forward(self, x):
        return self.fn(x, self.weight.get_differentiable_data(), self.weight, self.bias)

    def extra_repr(self):
        return "in_features={}, out_features={}, bias={}, block_count={}".format(
            self.in_features, self.out_features, self.bias is not None, self.block_count
        )


class PseudoBlockSparseLinear(torch.nn.Module):
    """Dense weight times block mask, plain torch; a debugging twin.  reference: block_sparse_linear.py:236-262."""

    def __init__(self, block_sparse_linear):
        super().__init__()
        matrix = block_sparse_linear.weight
        self.weight = torch.nn.Parameter(matrix.to_dense().detach().clone())
        mask = matrix.to_dense(data_replace=torch.ones_like(matrix.data)) == 1
        if block_sparse_linear.bias is not None:
            self.bias = torch.nn.Parameter(block_sparse_linear.bias.detach().clone())
        else:
            self.register_parameter("bias", None)
        self.register_buffer("mask", mask)
        self.in_features = block_sparse_linear.in_features
        self.out_features = block_sparse_linear.out_features
        self.density = mask.sum().item() / (mask.shape[0] * mask.shape[1])

    def forward(self, input):
        return torch.nn.functional.linear(input, self.weight * self.mask, self.bias)

    def extra_repr(self):
        return "in_features={}, out_features={}, bias={}, fill_ratio={}".format(
            self.in_features, self.out_features, self.bias is not None, self.density
        )
