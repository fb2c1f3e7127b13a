"""Tensor-parallel + sequence-parallel linears of the attention block
(utils/linear_tpsp.py of the reference), with the dense products on the HIP library.

One rank's compute only: the three products (forward X W^T, dgrad dY W, wgrad
dY^T X) run through ody_gemm; the sequence all-gather / reduce-scatter around
them is the identity at world_size = 1 and raises for larger groups.
"""
from __future__ import annotations

import os
import warnings
from typing import Callable, List, Optional

import torch
import torch.nn.init as init
from torch.nn.parameter import Parameter

from .. import ops
from ..parallel_state import (divide_and_check_no_remainder, get_model_parallel_group,
                              get_model_parallel_rank, get_model_parallel_world_size, require_single_rank)
from .comm import prepare_input_tensors_for_wgrad_compute


# ---------------------------------------------------------------- sequence-dim collectives
def _reduce_scatter_along_first_dim(input_):
    """(1, L, h) -> (1, L / N, h), summed over ranks (utils/linear_tpsp.py:35-58)."""
    if get_model_parallel_world_size() == 1:
        return input_
    bs_, seqlen, _ = input_.shape
    assert bs_ == 1, f"Batch size should be 1, got {bs_}"
    assert seqlen % get_model_parallel_world_size() == 0, \
        "First dimension of the tensor should be divisible by tensor parallel size"
    require_single_rank("reduce-scatter along the sequence")


def _gather_along_first_dim(input_):
    """(1, L / N, h) -> (1, L, h) (utils/linear_tpsp.py:61-81)."""
    if get_model_parallel_world_size() == 1:
        return input_
    bs_, _, _ = input_.shape
    assert bs_ == 1, f"Batch size should be 1, got {bs_}"
    require_single_rank("all-gather along the sequence")


class _ReduceScatterToSequenceParallelRegion(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_):
        return _reduce_scatter_along_first_dim(input_)

    @staticmethod
    def backward(ctx, grad_output):
        return _gather_along_first_dim(grad_output)


class AllgatherToSequenceParallelRegion(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_):
        return _gather_along_first_dim(input_)

    @staticmethod
    def backward(ctx, grad_output):
        return _reduce_scatter_along_first_dim(grad_output)


def reducescatter_from_model_parallel_region(input_: torch.Tensor) -> torch.Tensor:
    return _ReduceScatterToSequenceParallelRegion.apply(input_)


def allgather_along_first_dim_from_model_parallel_region(input_: torch.Tensor) -> torch.Tensor:
    return AllgatherToSequenceParallelRegion.apply(input_)


# ---------------------------------------------------------------- the three products
def _autocast(*ts):
    """What torch.matmul does under autocast, which the reference relies on through custom_fwd /
    custom_bwd (utils/linear_tpsp.py:129,180, utils/linear_zero3.py:24,51): operands are cast to
    the autocast dtype.  Outside autocast the tensors pass through and a dtype mismatch raises."""
    if torch.is_autocast_enabled("cuda"):
        dt = torch.get_autocast_dtype("cuda")
        return tuple(t if t is None or t.dtype == dt else t.to(dt) for t in ts)
    return ts


def _as_2d(t: torch.Tensor) -> torch.Tensor:
    t2 = t.reshape(-1, t.shape[-1])
    return t2 if t2.stride(-1) == 1 else t2.contiguous()


def linear_forward(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """Y = X W^T (+ b) over the last dimension of x.  The result is allocated in its final
    shape (not returned as a view), so that a following in-place op may own it."""
    x, weight, bias = _autocast(x, weight, bias)
    y = torch.empty((*x.shape[:-1], weight.shape[0]), dtype=x.dtype, device=x.device)
    ops.gemm(ops.GEMM_NT, _as_2d(x), weight, bias=bias, out=y.view(-1, weight.shape[0]))
    return y


def linear_dgrad(grad_output: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """dX = dY W."""
    grad_output, weight = _autocast(grad_output, weight)
    dx = torch.empty((*grad_output.shape[:-1], weight.shape[1]), dtype=grad_output.dtype, device=grad_output.device)
    ops.gemm(ops.GEMM_NN, _as_2d(grad_output), weight, out=dx.view(-1, weight.shape[1]))
    return dx


def linear_wgrad(grad_output_2d: torch.Tensor, input_2d: torch.Tensor) -> torch.Tensor:
    """dW = dY^T X on the flattened, contiguous pair."""
    grad_output_2d, input_2d = _autocast(grad_output_2d, input_2d)
    return ops.gemm(ops.GEMM_TN, grad_output_2d, input_2d)


class LinearWithGradAccumulationAndAsyncCommunication(torch.autograd.Function):
    """Y = gather(X) W^T + b with dX reduce-scattered in backward
    (utils/linear_tpsp.py:125-303).  Only the un-gathered input and the weight are
    saved; backward re-gathers the input."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, input, weight, bias, gradient_accumulation_fusion, async_grad_allreduce, sequence_parallel,
                grad_output_buffer):
        ctx.save_for_backward(input, weight)
        ctx.use_bias = bias is not None
        ctx.gradient_accumulation_fusion = gradient_accumulation_fusion
        ctx.async_grad_allreduce = async_grad_allreduce
        ctx.sequence_parallel = sequence_parallel
        ctx.grad_output_buffer = grad_output_buffer
        if sequence_parallel:
            bs_, _, _ = input.shape
            assert bs_ == 1, f"Batch size should be 1, got {bs_}"
            total_input = _gather_along_first_dim(input)
        else:
            total_input = input
        return linear_forward(total_input, weight, bias)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        wgrad_compute = True
        if ctx.grad_output_buffer is not None:
            ctx.grad_output_buffer.append(grad_output)
            wgrad_compute = False
        if ctx.sequence_parallel:
            bs_, _, _ = input.shape
            assert bs_ == 1, f"Batch size should be 1, got {bs_}"
            assert not ctx.async_grad_allreduce
            total_input = _gather_along_first_dim(input)
        else:
            total_input = input
        grad_input = linear_dgrad(grad_output, weight)
        if ctx.async_grad_allreduce:
            require_single_rank("all-reduce of the input gradient")
        if ctx.sequence_parallel:
            grad_input = _reduce_scatter_along_first_dim(grad_input)
        grad_weight = None
        if ctx.gradient_accumulation_fusion:
            if wgrad_compute:
                raise NotImplementedError("Gradient accumulation fusion is not supported for sequence parallelism")
        elif wgrad_compute:
            g2, x2 = prepare_input_tensors_for_wgrad_compute(grad_output, total_input)
            grad_weight = linear_wgrad(g2, x2)
        grad_bias = None
        if ctx.use_bias:
            grad_bias = grad_output.reshape(-1, grad_output.shape[-1]).sum(dim=0)
        return grad_input, grad_weight, grad_bias, None, None, None, None


def linear_with_grad_accumulation_and_async_allreduce(
        input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], gradient_accumulation_fusion: bool,
        async_grad_allreduce: bool, sequence_parallel: bool,
        grad_output_buffer: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Functional form (utils/linear_tpsp.py:306-399).  The reference warns once when
    CUDA_DEVICE_MAX_CONNECTIONS != 1 because its overlap relies on launch order; the
    same variable is honoured here so that scripts behave alike."""
    fn = linear_with_grad_accumulation_and_async_allreduce
    if not fn.warned and os.environ.get("CUDA_DEVICE_MAX_CONNECTIONS") != "1":
        if sequence_parallel or async_grad_allreduce:
            what = "sequence parallelism" if sequence_parallel else "async grad allreduce"
            warnings.warn(f"When using {what} it is recommended to set the environment variable "
                          "CUDA_DEVICE_MAX_CONNECTIONS to 1 for maximum speedup")
            fn.warned = True
    return LinearWithGradAccumulationAndAsyncCommunication.apply(
        input, weight, bias, gradient_accumulation_fusion, async_grad_allreduce, sequence_parallel,
        grad_output_buffer)


linear_with_grad_accumulation_and_async_allreduce.warned = False


def _init_partitioned_weight(weight, out_features, in_features, per_partition, partition_dim, init_method,
                             stride=1, return_master_weight=False):
    """Initialises the full ("master") weight with `init_method`, then keeps this rank's
    strided partition along `partition_dim` -- so every rank of a group derives its shard
    from the same random stream (what fairscale's _initialize_affine_weight does, called
    at utils/linear_tpsp.py:463-472 and :567-576)."""
    world = get_model_parallel_world_size()
    if world == 1:
        init_method(weight)
        return weight.detach().clone() if return_master_weight else None
    master = torch.empty(out_features, in_features, dtype=weight.dtype, requires_grad=False)
    init_method(master)
    per_stride = divide_and_check_no_remainder(per_partition, stride)
    pieces = torch.split(master, per_stride, dim=partition_dim)
    mine = pieces[get_model_parallel_rank()::world]
    with torch.no_grad():
        torch.cat(mine, dim=partition_dim, out=weight)
    return master if return_master_weight else None


class _ColumnParallelLinearBase(torch.nn.Module):
    """Y = X A_i^T: the weight is split along its OUTPUT rows.  The two public classes differ in one
    flag only: whether the input is the sequence shard that the layer gathers itself."""

    sequence_parallel: bool = False

    def __init__(self, in_features: int, out_features: int, bias: bool = True, gather_output: bool = True,
                 init_method: Callable[[torch.Tensor], torch.Tensor] = init.xavier_normal_, stride: int = 1,
                 keep_master_weight_for_test: bool = False) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.gather_output = gather_output
        world_size = get_model_parallel_world_size()
        self.output_size_per_partition = divide_and_check_no_remainder(out_features, world_size)
        self.weight = Parameter(torch.empty(self.output_size_per_partition, self.in_features))
        if bias:
            self.bias = Parameter(torch.zeros(self.output_size_per_partition))
        else:
            self.register_parameter("bias", None)
        self.master_weight = _init_partitioned_weight(
            self.weight, self.out_features, self.in_features, self.output_size_per_partition, 0, init_method,
            stride=stride, return_master_weight=keep_master_weight_for_test)

    def get_master_weight(self) -> torch.Tensor:
        require_single_rank("gather of the column-split weight")
        return self.weight.data.clone()

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        output_parallel = linear_with_grad_accumulation_and_async_allreduce(
            input=input_, weight=self.weight, bias=self.bias, gradient_accumulation_fusion=False,
            async_grad_allreduce=False, sequence_parallel=self.sequence_parallel)
        if self.gather_output:
            require_single_rank("gather of the column-split output")
        return output_parallel


class ColumnParallelLinearAG(_ColumnParallelLinearBase):
    """Y = gather(X) A_i^T: the input is the sequence shard and is gathered inside
    (utils/linear_tpsp.py:405-500)."""

    sequence_parallel = True


class ColumnParallelLinear(_ColumnParallelLinearBase):
    """Column-split linear WITHOUT the sequence gather: the unpacked q/k/v branch and the
    non-sequence-parallel branch of the attention block (decoder/odysseus.py:96-137) take
    it from fairscale; the caller gathers the sequence first."""

    sequence_parallel = False


class _PlainLinearFunc(torch.autograd.Function):
    """F.linear without bias on the HIP products (forward of utils/linear_tpsp.py:588 and
    the backward autograd derives for it)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, input, weight):
        ctx.save_for_backward(input, weight)
        return linear_forward(input, weight, None)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        grad_input = linear_dgrad(grad_output, weight)
        g2, x2 = prepare_input_tensors_for_wgrad_compute(grad_output, input)
        if x2.dim() != 2:
            x2 = x2.reshape(-1, x2.shape[-1])
        if g2.dim() != 2:
            g2 = g2.reshape(-1, g2.shape[-1])
        return grad_input, linear_wgrad(g2, _as_2d(x2))


class RowParallelLinearRS(torch.nn.Module):
    """Y = reduce_scatter(X_i A_i^T) + b: the weight is split along its INPUT columns, the
    output is reduce-scattered to the sequence shard, the (unsplit) bias is added after
    (utils/linear_tpsp.py:503-596)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, input_is_parallel: bool = False,
                 init_method: Callable[[torch.Tensor], torch.Tensor] = init.xavier_normal_, stride: int = 1,
                 keep_master_weight_for_test: bool = False):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.input_is_parallel = input_is_parallel
        world_size = get_model_parallel_world_size()
        self.input_size_per_partition = divide_and_check_no_remainder(in_features, world_size)
        self.weight = Parameter(torch.empty(self.out_features, self.input_size_per_partition))
        if bias:
            self.bias = Parameter(torch.zeros(self.out_features))
        else:
            self.register_parameter("bias", None)
        self.master_weight = _init_partitioned_weight(
            self.weight, self.out_features, self.in_features, self.input_size_per_partition, 1, init_method,
            stride=stride, return_master_weight=keep_master_weight_for_test)

    def get_master_weight(self) -> torch.Tensor:
        require_single_rank("gather of the row-split weight")
        return self.weight.data.clone()

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        if not self.input_is_parallel:
            require_single_rank("scatter of the input over the model-parallel group")
        output_parallel = _PlainLinearFunc.apply(input_, self.weight)
        output_ = reducescatter_from_model_parallel_region(output_parallel)
        return output_ if self.bias is None else output_ + self.bias
