"""Vocab-parallel cross entropy on the gfx950 kernels.

Same call as Merak/core/mpu/cross_entropy.py:109-118: per-position loss of the
shape of ``target`` from this rank's slice of the logits; targets outside the
slice (``-100`` included) contribute no one-hot term, exactly like the
reference's mask (:48-62).  Differences in *how*, not in *what*:

* one pass computes max and sum-exp together in fp32 (the reference makes
  about eight passes over the logits in the logits' own dtype);
* the forward leaves the logits untouched; the backward overwrites them with
  the gradient and returns that same storage, so — like the reference, which
  reuses the buffer for the softmax (:37,70,80,92) — no second
  [tokens, vocab] tensor is ever allocated;
* for bf16 logits the loss is returned in fp32 unless
  ``loss_in_logits_dtype=True``;
* ``fused_backward_scale=g`` (an extension) runs forward and backward in one
  launch for the case where the upstream gradient of every per-position loss
  is known to be ``g`` before the forward — ``vocab_loss_fn`` below, the
  trainer's ``mean`` (Merak/merak_trainer.py:313-326), passes ``1/n``.  Like
  the reference, this forward overwrites the caller's logits (there with the
  softmax, here with the finished gradient); ``backward`` checks the real
  upstream gradient on the device and rescales only the rows where it differs.
"""
from __future__ import annotations

import torch

from .. import ops
from .initialize import get_model_parallel_rank, get_model_parallel_world_size
from .utils import VocabUtility


def _vocab_range(partition_vocab_size):
    get_vocab_range = VocabUtility.vocab_range_from_per_partition_vocab_size
    rank = get_model_parallel_rank()
    world_size = get_model_parallel_world_size()
    return get_vocab_range(partition_vocab_size, rank, world_size)


class _VocabParallelCrossEntropy(torch.autograd.Function):

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, loss_in_logits_dtype, materialize_softmax):
        if get_model_parallel_world_size() != 1:
            raise RuntimeError(
                "vocab_parallel_cross_entropy at tensor-parallel size > 1 needs the MAX/SUM/SUM exchange of "
                "cross_entropy.py:33,64,72; on one rank use vocab_parallel_cross_entropy_partials() and "
                "vocab_parallel_cross_entropy_backward_() around your own reduction")
        partition_vocab_size = vocab_parallel_logits.size()[-1]
        vocab_start_index, _ = _vocab_range(partition_vocab_size)
        # [*, partition-vocab-size] view; like the reference (:55) this requires contiguous logits
        logits_2d = vocab_parallel_logits.view(-1, partition_vocab_size)
        target_1d = target.reshape(-1)
        loss, row_max, row_sumexp, _ = ops.vocab_ce_fwd(logits_2d, target_1d, vocab_start_index)
        ctx.vocab_start = vocab_start_index
        ctx.materialized = bool(materialize_softmax)
        if materialize_softmax:
            # reproduce the reference's side effect: the caller's logits now hold the softmax (:80)
            ops.vocab_ce_bwd_(logits_2d, torch.full_like(target_1d, -1), row_max, row_sumexp, None,
                              vocab_start_index)
        ctx.save_for_backward(vocab_parallel_logits, target_1d, row_max, row_sumexp)
        loss = loss.view_as(target)
        if loss_in_logits_dtype:
            loss = loss.to(vocab_parallel_logits.dtype)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        logits, target_1d, row_max, row_sumexp = ctx.saved_tensors
        partition_vocab_size = logits.size()[-1]
        grad_2d = logits.view(-1, partition_vocab_size)
        g = grad_output.reshape(-1)
        if ctx.materialized:
            # the buffer already holds the softmax (cross_entropy.py:92-104)
            row_max = row_sumexp = None
        ops.vocab_ce_bwd_(grad_2d, target_1d, row_max, row_sumexp, g, ctx.vocab_start)
        return logits, None, None, None


class _VocabParallelCrossEntropyFused(torch.autograd.Function):
    """Forward that already writes the gradient for an assumed uniform upstream gradient."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, loss_in_logits_dtype, assumed_grad):
        partition_vocab_size = vocab_parallel_logits.size()[-1]
        vocab_start_index, _ = _vocab_range(partition_vocab_size)
        logits_2d = vocab_parallel_logits.view(-1, partition_vocab_size)
        target_1d = target.reshape(-1)
        loss, _, _, _ = ops.vocab_ce_fwd_bwd_(logits_2d, target_1d, vocab_start_index, None, assumed_grad)
        # the kernel wrote through a raw pointer: tell autograd that the caller's logits have changed, so that
        # another function that saved them for its own backward fails loudly instead of using the gradient.
        # The linear layers return tensors that own their storage, so their logits are marked.  A view handed out
        # by some other custom Function cannot be: autograd refuses to rebuild such a view's history, and there
        # the overwrite is only documented.
        if not vocab_parallel_logits._is_view():
            torch.autograd.graph.increment_version(vocab_parallel_logits)
        ctx.assumed_grad = float(assumed_grad)
        ctx.save_for_backward(vocab_parallel_logits)
        loss = loss.view_as(target)
        if loss_in_logits_dtype:
            loss = loss.to(vocab_parallel_logits.dtype)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        (grad,) = ctx.saved_tensors
        grad_2d = grad.view(-1, grad.size()[-1])
        ops.vocab_ce_rescale_(grad_2d, grad_output.reshape(-1), ctx.assumed_grad)
        return grad, None, None, None


def vocab_parallel_cross_entropy(vocab_parallel_logits, target, loss_in_logits_dtype=False,
                                 materialize_softmax=False, fused_backward_scale=None):
    """Cross entropy loss when logits are split across tensor parallel ranks.

    Args:
        vocab_parallel_logits: logits split across tensor parallel ranks,
            [sequence_length, batch_size, vocab_size / num_parallel_ranks], contiguous
        target: correct vocab ids of dimension [sequence_length, micro_batch_size]
    """
    if fused_backward_scale is not None and not materialize_softmax:
        g = float(fused_backward_scale)
        if g == 0.0 or g != g:
            raise ValueError("fused_backward_scale must be a non-zero number")
        fits = vocab_parallel_logits.size()[-1] <= ops.vocab_ce_fused_max_vocab(vocab_parallel_logits.dtype)
        if fits and get_model_parallel_world_size() == 1:
            return _VocabParallelCrossEntropyFused.apply(vocab_parallel_logits, target, loss_in_logits_dtype, g)
    return _VocabParallelCrossEntropy.apply(vocab_parallel_logits, target, loss_in_logits_dtype,
                                            materialize_softmax)


def vocab_loss_fn(outputs, labels, loss_scale=1.0):
    """The trainer's loss over vocab-parallel logits, Merak/merak_trainer.py:313-326:
    ``mean`` of the per-position losses.  The mean makes every position's upstream gradient
    ``loss_scale / n``, which is handed to the one-launch forward+backward kernel; multiply the
    returned loss by ``loss_scale`` (or anything else) as usual — a different factor only costs the
    rescale pass in backward."""
    if isinstance(outputs, tuple):
        outputs = outputs[0]
    if isinstance(labels, tuple):
        labels = labels[0]
    n = labels.numel()
    # The one-launch kernel overwrites the logits with their gradient during forward; that is only wanted when a
    # backward pass will follow.  Evaluation (no_grad, or logits that take no gradient: the reference's eval_batch
    # hands the logits back after the loss) runs the plain forward, which leaves the logits as they are.
    wants_grad = torch.is_grad_enabled() and outputs.requires_grad
    losses = vocab_parallel_cross_entropy(outputs, labels,
                                          fused_backward_scale=(float(loss_scale) / n) if (n and wants_grad) else None)
    return torch.mean(losses.view(-1))


def vocab_parallel_cross_entropy_partials(vocab_parallel_logits, target):
    """This rank's (row_max, row_sumexp, predicted_logit) over its vocab slice, fp32, each shaped like ``target``.

    They are what the reference all-reduces with MAX, SUM and SUM (cross_entropy.py:33,64,72), except
    that row_sumexp is relative to the *local* row_max (rescale by exp(local_max - global_max) before
    summing) and predicted_logit is the raw logit (0 where the target is outside this slice)."""
    partition_vocab_size = vocab_parallel_logits.size()[-1]
    vocab_start_index, _ = _vocab_range(partition_vocab_size)
    logits_2d = vocab_parallel_logits.view(-1, partition_vocab_size)
    _, row_max, row_sumexp, pred = ops.vocab_ce_fwd(logits_2d, target.reshape(-1), vocab_start_index)
    return row_max.view_as(target), row_sumexp.view_as(target), pred.view_as(target)


def vocab_parallel_cross_entropy_backward_(vocab_parallel_logits, target, global_row_max, global_row_sumexp,
                                           grad_output):
    """In place gradient of this rank's logits slice given the globally combined max / sum-exp."""
    partition_vocab_size = vocab_parallel_logits.size()[-1]
    vocab_start_index, _ = _vocab_range(partition_vocab_size)
    logits_2d = vocab_parallel_logits.view(-1, partition_vocab_size)
    ops.vocab_ce_bwd_(logits_2d, target.reshape(-1), global_row_max.reshape(-1).contiguous(),
                      global_row_sumexp.reshape(-1).contiguous(), grad_output.reshape(-1), vocab_start_index)
    return vocab_parallel_logits


class _LMHeadCrossEntropy(torch.autograd.Function):
    """Vocab-parallel LM head and cross entropy over row chunks: the [tokens, vocab] logits exist one chunk at
    a time.  Forward already produces the gradients (for an assumed uniform upstream gradient of the
    per-position losses), as the one-launch cross entropy does."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, target, assumed_grad, chunk_rows, accum_dtype):
        vocab_start_index, _ = _vocab_range(weight.shape[0])
        lead = hidden.shape[:-1]
        h2d = hidden.reshape(-1, hidden.shape[-1])
        t1d = target.reshape(-1)
        n = h2d.shape[0]
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_b = bias is not None and ctx.needs_input_grad[2]
        losses = torch.empty((n,), dtype=torch.float32, device=h2d.device)
        dh = torch.empty_like(h2d) if need_h else None
        # The first chunk writes the weight and bias gradients, the later ones add to them (a read-modify-write of
        # the whole gradient per chunk), in accum_dtype: the weight's dtype, or fp32 with one cast at the end.
        one_chunk = chunk_rows >= n
        acc_dt = weight.dtype if one_chunk else accum_dtype
        dw = torch.empty(weight.shape, dtype=acc_dt, device=weight.device) if need_w else None
        db = torch.empty(bias.shape, dtype=acc_dt, device=bias.device) if need_b else None
        epi = ops.EPI_BIAS if bias is not None else ops.EPI_NONE
        backward_wanted = need_h or need_w or need_b
        for r0 in range(0, n, chunk_rows):
            r1 = min(n, r0 + chunk_rows)
            logits, _ = ops.linear_fwd(h2d[r0:r1], weight, bias, epi)          # layers.py:251-252
            if backward_wanted:
                loss_c, _, _, _ = ops.vocab_ce_fwd_bwd_(logits, t1d[r0:r1], vocab_start_index, None, assumed_grad)
                if need_h:
                    dh[r0:r1] = ops.linear_dgrad(logits, weight)
                if need_w:
                    ops.linear_wgrad(logits, h2d[r0:r1], need_b, dw=dw, db=db, accumulate=r0 > 0)
                elif need_b:
                    ops.colsum(logits, db, accumulate=r0 > 0)
            else:
                loss_c, _, _, _ = ops.vocab_ce_fwd(logits, t1d[r0:r1], vocab_start_index)
            losses[r0:r1] = loss_c
            del logits
        if dw is not None and dw.dtype != weight.dtype:
            dw = dw.to(weight.dtype)
        if db is not None and db.dtype != bias.dtype:
            db = db.to(bias.dtype)
        ctx.assumed_grad = float(assumed_grad)
        ctx.lead = lead
        ctx.save_for_backward(dh, dw, db)
        return losses.view(*target.shape)

    @staticmethod
    def backward(ctx, grad_losses):
        dh, dw, db = ctx.saved_tensors
        g = grad_losses.reshape(-1)
        first = g[:1]
        if not bool((g == first).all()):
            raise RuntimeError("lm_head_cross_entropy needs one upstream gradient for all positions (a mean or a "
                               "sum of the losses); weight the positions through the unfused layers instead")
        ratio = float(first) / ctx.assumed_grad
        if ratio != 1.0:
            # out of place: the saved gradients stay valid for a second backward over a retained graph
            dh, dw, db = (None if t is None else t * ratio for t in (dh, dw, db))
        return (dh.view(*ctx.lead, dh.shape[-1]) if dh is not None else None), dw, db, None, None, None, None


def lm_head_cross_entropy(hidden, lm_head, target, loss_scale=1.0, chunk_rows=4096, grad_accum_dtype=None):
    """Per-position losses of ``vocab_parallel_cross_entropy(lm_head(hidden)[0], target)`` without ever holding
    the full logits: the head's product, the cross entropy and both of the head's backward products run per
    chunk of ``chunk_rows`` tokens, so the largest temporary is [chunk_rows, vocab/p].

    ``lm_head``: a ``ColumnParallelLinear(hidden, vocab, gather_output=False)`` (model_parallel.py:143-156) or
    its weight.  The per-position losses must be reduced with one common factor — ``.mean()`` as the
    trainer does (merak_trainer.py:325), times ``loss_scale`` if any; that factor is assumed in forward
    (``loss_scale / n``) and checked in backward.

    What it is and is not: the logits still make their trip through memory, one chunk at a time (product ->
    cross entropy and gradient in place -> the two backward products); what is saved is memory — the largest
    temporary is one chunk — not traffic, and every chunk after the first pays a read-modify-write of the whole
    weight gradient, so on a shape whose full logits fit it is a little slower than the unfused sequence.
    ``grad_accum_dtype``: dtype the weight (and bias) gradient is summed in across chunks.  Default: the
    weight's own dtype, which is how the reference's ``.grad`` sums micro-batches (one rounding to 16 bits per
    chunk: at 32 chunks in bf16 the gradient stays within twice the tolerance of the one-piece product);
    ``torch.float32`` sums in an fp32 buffer (4 bytes per weight more while the call runs) and rounds once."""
    weight, bias = (lm_head.weight, lm_head.bias) if isinstance(lm_head, torch.nn.Module) else (lm_head, None)
    if get_model_parallel_world_size() != 1:
        raise RuntimeError("lm_head_cross_entropy at tensor-parallel size > 1 needs the MAX/SUM/SUM exchange of "
                           "cross_entropy.py:33,64,72 between the head and the loss")
    n = target.numel()
    if n == 0:
        return torch.zeros(target.shape, dtype=torch.float32, device=hidden.device)
    if weight.shape[0] > ops.vocab_ce_fused_max_vocab(hidden.dtype):
        raise ValueError("vocabulary slice too long for the one-launch cross entropy; use the unfused layers")
    accum = weight.dtype if grad_accum_dtype is None else grad_accum_dtype
    if accum not in (weight.dtype, torch.float32):
        raise ValueError("grad_accum_dtype must be the weight's dtype or torch.float32")
    return _LMHeadCrossEntropy.apply(hidden, weight, bias, target, float(loss_scale) / n, int(chunk_rows), accum)
