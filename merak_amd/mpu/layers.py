"""Megatron-style tensor-parallel layers on the gfx950 kernels.

Same constructors, attributes, parameter names/layouts and ``(output, bias)``
returns as Merak/core/mpu/layers.py:92-369; the compute behind ``forward`` and
``backward`` is ``libmerak_tp_gfx950.so`` instead of ``F.linear`` /
``F.embedding``.  One extension over the reference: ``activation=`` fuses the
elementwise op that follows a column-parallel layer (HF ``gelu_new`` for
GPT-2, ``silu(gate) * up`` for Llama) into the GEMM epilogue.
"""
from __future__ import annotations

import contextlib

import torch
import torch.nn.init as init
from torch.nn.parameter import Parameter

from .. import ops
from ..args import get_args
from .initialize import get_model_parallel_rank, get_model_parallel_world_size
from .mappings import (copy_to_model_parallel_region, gather_from_model_parallel_region,
                       reduce_from_model_parallel_region, scatter_to_model_parallel_region)
from .random import get_rng_tracker
from .utils import VocabUtility, divide

_ACTIVATIONS = {None: None, "gelu_new": "gelu_new", "swiglu": "swiglu"}


def _initialize_affine_weight_gpu(weight, init_method, partition_dim, stride=1, rng_context=None):
    """Tag and initialise a device-resident shard (layers.py:44-53).

    The reference draws under ``get_rng_tracker().fork()``, the model-parallel generator state, so that ranks of one
    tensor-parallel group get different shards from one seed.  Here: under ``rng_context`` when one is given (any
    context manager), else under this package's tracker when ``mpu.model_parallel_manual_seed`` has registered the
    model-parallel state, else on the current generator (the reference would refuse; a caller that never seeded
    the tracker builds one rank's shard with its own generator)."""
    weight.model_parallel = True
    weight.partition_dim = partition_dim
    weight.partition_stride = stride
    if rng_context is None:
        tracker = get_rng_tracker()
        rng_context = tracker.fork() if tracker.has() else contextlib.nullcontext()
    with rng_context:
        init_method(weight)


def _initialize_affine_weight_cpu(weight, output_size, input_size, per_partition_size, partition_dim, init_method,
                                  stride=1, return_master_weight=False):
    """Build the full fp32 master weight, cast, and keep this rank's strided chunks (layers.py:56-89)."""
    weight.model_parallel = True
    weight.partition_dim = partition_dim
    weight.partition_stride = stride

    master_weight = torch.empty(output_size, input_size, dtype=torch.float, requires_grad=False)
    init_method(master_weight)
    args = get_args()
    master_weight = master_weight.to(dtype=args.params_dtype)

    per_partition_per_stride_size = divide(per_partition_size, stride)
    weight_list = torch.split(master_weight, per_partition_per_stride_size, dim=partition_dim)
    rank = get_model_parallel_rank()
    world_size = get_model_parallel_world_size()
    my_weight_list = weight_list[rank::world_size]

    with torch.no_grad():
        torch.cat(my_weight_list, dim=partition_dim, out=weight)
    if return_master_weight:
        return master_weight
    return None


def _param_device():
    if not torch.cuda.is_available():
        raise RuntimeError("use_cpu_initialization=False needs a GPU; set_args(use_cpu_initialization=True) "
                           "builds the parameters on the host (move the module to the GPU before calling it)")
    return torch.device("cuda", torch.cuda.current_device())


# --------------------------------------------------------------------------- autograd
class _LinearFunction(torch.autograd.Function):
    """y = x W^T (+ b), optionally followed by a fused activation.

    backward: dX = dY W, dW = dY^T X, db = sum dY — what autograd derives for
    ``F.linear`` (layers.py:252,354), one call of the library for all three."""

    @staticmethod
    def forward(ctx, x, weight, bias, activation):
        lead = x.shape[:-1]
        x2d = x.reshape(-1, x.shape[-1])
        if activation is None:
            epi = ops.EPI_BIAS if bias is not None else ops.EPI_NONE
        elif activation == "gelu_new":
            epi = ops.EPI_BIAS_GELU if bias is not None else ops.EPI_GELU
        else:
            epi = ops.EPI_SWIGLU
        need_pre = activation is None or any(ctx.needs_input_grad[:3])
        # outputs are allocated in their final shape: what this function returns owns its storage (a view made here
        # could not be version-bumped by a later in-place consumer such as the one-launch cross entropy)
        y, act = ops.linear_fwd(x2d, weight, bias, epi, want_pre=need_pre, lead=tuple(lead))
        ctx.activation = activation
        ctx.epi = epi
        ctx.has_bias = bias is not None
        ctx.lead = lead
        ctx.save_for_backward(x2d, weight, y if activation is not None else None)
        return y if activation is None else act

    @staticmethod
    def backward(ctx, grad_out):
        x2d, weight, pre = ctx.saved_tensors
        g2d = grad_out.reshape(-1, grad_out.shape[-1])
        if ctx.activation is not None:
            g2d = ops.activation_bwd(g2d, pre.view(-1, pre.shape[-1]), ctx.epi)
        dx = dw = db = None
        want_db = ctx.has_bias and ctx.needs_input_grad[2]
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[1] and g2d.shape[0] > 0:
            # both products in one call (one launch where their tiles share rounds of workgroups)
            dx, dw, db = ops.linear_bwd(g2d, x2d, weight, want_db)
            return dx.view(*ctx.lead, weight.shape[1]), dw, db, None
        if ctx.needs_input_grad[0]:
            dx = ops.linear_dgrad(g2d, weight).view(*ctx.lead, weight.shape[1])
        if ctx.needs_input_grad[1]:
            dw, db = ops.linear_wgrad(g2d, x2d, want_db)
        elif want_db:
            _, db = ops.linear_wgrad(g2d, x2d, True)
        return dx, dw, db, None


class _EmbeddingFunction(torch.autograd.Function):
    """out = weight[ids - start] for ids in [start, end), zero rows otherwise (layers.py:145-162)."""

    @staticmethod
    def forward(ctx, ids, weight, vocab_start, vocab_end):
        ctx.save_for_backward(ids)
        ctx.range = (vocab_start, vocab_end)
        ctx.wshape = weight.shape
        ctx.wdtype = weight.dtype
        return ops.embedding_gather(ids, weight, vocab_start, vocab_end)

    @staticmethod
    def backward(ctx, grad_out):
        (ids,) = ctx.saved_tensors
        grad_out = grad_out if grad_out.dtype == ctx.wdtype else grad_out.to(ctx.wdtype)
        dtable = ops.embedding_bwd(ids, grad_out, ctx.wshape[0], *ctx.range, dtype=ctx.wdtype)
        return None, dtable, None, None


# --------------------------------------------------------------------------- modules
class VocabParallelEmbedding(torch.nn.Module):
    """Embedding parallelized in the vocabulary dimension (layers.py:92-165).

    Arguments:
        num_embeddings: vocabulary size.
        embedding_dim: size of hidden state.
        init_method: method to initialize weights.
    """

    def __init__(self, num_embeddings, embedding_dim, init_method=init.xavier_normal_):
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        # torch.nn.Embedding defaults, kept for compatibility (layers.py:109-115)
        self.padding_idx = None
        self.max_norm = None
        self.norm_type = 2.
        self.scale_grad_by_freq = False
        self.sparse = False
        self._weight = None
        self.model_parallel_size = get_model_parallel_world_size()
        self.vocab_start_index, self.vocab_end_index = VocabUtility.vocab_range_from_global_vocab_size(
            self.num_embeddings, get_model_parallel_rank(), self.model_parallel_size)
        self.num_embeddings_per_partition = self.vocab_end_index - self.vocab_start_index

        args = get_args()
        if args.use_cpu_initialization:
            self.weight = Parameter(torch.empty(self.num_embeddings_per_partition, self.embedding_dim,
                                                dtype=args.params_dtype))
            _initialize_affine_weight_cpu(self.weight, self.num_embeddings, self.embedding_dim,
                                          self.num_embeddings_per_partition, 0, init_method)
        else:
            self.weight = Parameter(torch.empty(self.num_embeddings_per_partition, self.embedding_dim,
                                                device=_param_device(), dtype=args.params_dtype))
            _initialize_affine_weight_gpu(self.weight, init_method, partition_dim=0, stride=1)

    def forward(self, input_):
        # The kernel applies the range mask itself (ids outside [start, end) give zero rows), which is
        # layers.py:148-152,162 at p > 1 and plain F.embedding at p == 1.
        output_parallel = _EmbeddingFunction.apply(input_, self.weight, self.vocab_start_index,
                                                   self.vocab_end_index)
        return reduce_from_model_parallel_region(output_parallel)


class ColumnParallelLinear(torch.nn.Module):
    """Linear layer with column parallelism: Y_i = X A_i + b_i (layers.py:168-265).

    Arguments are the reference's; ``activation`` (None, "gelu_new", "swiglu")
    is this build's fused-epilogue extension.  With "swiglu" the weight holds
    the gate rows followed by the up rows and the output width is
    ``output_size_per_partition // 2``.
    """

    def __init__(self, input_size, output_size, bias=True, gather_output=True, init_method=init.xavier_normal_,
                 stride=1, keep_master_weight_for_test=False, skip_bias_add=False, activation=None):
        super().__init__()
        if activation not in _ACTIVATIONS:
            raise ValueError(f"activation must be one of {list(_ACTIVATIONS)}, got {activation!r}")
        if activation is not None and skip_bias_add and bias:
            raise ValueError("a fused activation needs the bias added first: skip_bias_add must be False")
        self.input_size = input_size
        self.output_size = output_size
        self.gather_output = gather_output
        world_size = get_model_parallel_world_size()
        self.output_size_per_partition = divide(output_size, world_size)
        self.skip_bias_add = skip_bias_add
        self.activation = activation

        # F.linear computes X A^T + b, so the transpose is what gets allocated: [out/p, in] (layers.py:207-216)
        args = get_args()
        empty_tensor = torch.empty(self.output_size_per_partition, self.input_size, dtype=args.params_dtype)
        if args.use_cpu_initialization:
            self.weight = Parameter(empty_tensor)
            self.master_weight = _initialize_affine_weight_cpu(
                self.weight, self.output_size, self.input_size, self.output_size_per_partition, 0, init_method,
                stride=stride, return_master_weight=keep_master_weight_for_test)
        else:
            self.weight = Parameter(empty_tensor.to(device=_param_device()))
            _initialize_affine_weight_gpu(self.weight, init_method, partition_dim=0, stride=stride)

        if bias:
            if args.use_cpu_initialization:
                self.bias = Parameter(torch.empty(self.output_size_per_partition, dtype=args.params_dtype))
            else:
                self.bias = Parameter(torch.empty(self.output_size_per_partition, device=_param_device(),
                                                  dtype=args.params_dtype))
            self.bias.model_parallel = True
            self.bias.partition_dim = 0
            self.bias.stride = stride
            with torch.no_grad():
                self.bias.zero_()
        else:
            self.register_parameter('bias', None)

    def forward(self, input_):
        input_parallel = copy_to_model_parallel_region(input_)
        bias = self.bias if not self.skip_bias_add else None
        output_parallel = _LinearFunction.apply(input_parallel, self.weight, bias, self.activation)
        if self.gather_output:
            output = gather_from_model_parallel_region(output_parallel)
        else:
            output = output_parallel
        output_bias = self.bias if self.skip_bias_add else None
        return output, output_bias

    def extra_repr(self) -> str:
        return 'in_features={}, out_features={}, bias={}'.format(
            self.input_size, self.output_size_per_partition, self.bias is not None)


class RowParallelLinear(torch.nn.Module):
    """Linear layer with row parallelism: Y = sum_i X_i A_i + b (layers.py:268-369)."""

    def __init__(self, input_size, output_size, bias=True, input_is_parallel=False, init_method=init.xavier_normal_,
                 stride=1, keep_master_weight_for_test=False, skip_bias_add=False):
        super().__init__()
        self.input_size = input_size
        self.output_size = output_size
        self.input_is_parallel = input_is_parallel
        world_size = get_model_parallel_world_size()
        self.input_size_per_partition = divide(input_size, world_size)
        self.skip_bias_add = skip_bias_add

        args = get_args()
        empty_tensor = torch.empty(self.output_size, self.input_size_per_partition, dtype=args.params_dtype)
        if args.use_cpu_initialization:
            self.weight = Parameter(empty_tensor)
            self.master_weight = _initialize_affine_weight_cpu(
                self.weight, self.output_size, self.input_size, self.input_size_per_partition, 1, init_method,
                stride=stride, return_master_weight=keep_master_weight_for_test)
        else:
            self.weight = Parameter(empty_tensor.to(_param_device()))
            _initialize_affine_weight_gpu(self.weight, init_method, partition_dim=1, stride=stride)
        if bias:
            if args.use_cpu_initialization:
                self.bias = Parameter(torch.empty(self.output_size, dtype=args.params_dtype))
            else:
                self.bias = Parameter(torch.empty(self.output_size, device=_param_device(),
                                                  dtype=args.params_dtype))
            with torch.no_grad():
                self.bias.zero_()
        else:
            self.register_parameter('bias', None)

    def forward(self, input_):
        if self.input_is_parallel:
            input_parallel = input_
        else:
            input_parallel = scatter_to_model_parallel_region(input_)
        # The reference multiplies without bias, all-reduces, then adds the bias (layers.py:354-358).  The
        # reduce is the identity on one rank, so the add is fused into the GEMM epilogue; with p > 1 the
        # result is this rank's partial sum and the bias must wait for the (caller's) reduction.
        fuse_bias = (not self.skip_bias_add) and self.bias is not None and get_model_parallel_world_size() == 1
        output_parallel = _LinearFunction.apply(input_parallel, self.weight, self.bias if fuse_bias else None, None)
        output_ = reduce_from_model_parallel_region(output_parallel)
        if not self.skip_bias_add:
            if self.bias is not None and not fuse_bias:
                raise RuntimeError("RowParallelLinear with bias at tensor-parallel size > 1 needs the all-reduce "
                                   "before the bias add; use skip_bias_add=True and add the bias after reducing")
            output = output_
            output_bias = None
        else:
            output = output_
            output_bias = self.bias
        return output, output_bias

    def extra_repr(self) -> str:
        return 'in_features={}, out_features={}, bias={}'.format(
            self.input_size_per_partition, self.output_size, self.bias is not None)
